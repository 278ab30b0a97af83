/* synth.c — see synth.h. */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>

#include "gguf.h"
#include "quant.h"
#include "synth.h"
#include "../../include/lg_math.h"

static uint64_t mix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
static uint64_t name_hash(const char *s) {
    uint64_t h = 0xCBF29CE484222325ull;
    while (*s) h = (h ^ (unsigned char)*s++) * 0x100000001B3ull;
    return h;
}
/* two independent N(0,1) from one counter value */
static void normal_pair(uint64_t key, uint64_t ctr, float *a, float *b) {
    uint64_t r = mix64(key ^ mix64(ctr));
    float u1 = ((float)(uint32_t)(r >> 40) + 1.0f) * (1.0f / 16777216.0f);        /* (0,1] */
    float u2 = (float)(uint32_t)((r >> 8) & 0xFFFFFFu) * (1.0f / 16777216.0f);    /* [0,1) */
    float rad = sqrtf(-2.0f * logf(u1)), ang = 6.28318530717958648f * u2;
    *a = rad * cosf(ang);
    *b = rad * sinf(ang);
}
static float uniform_pm1(uint64_t key, uint64_t ctr) {
    uint64_t r = mix64(key ^ mix64(ctr));
    return (float)(uint32_t)(r >> 40) * (2.0f / 16777216.0f) - 1.0f;
}

struct planned { int index; uint32_t type; uint64_t rows, cols; float centre; uint64_t key; };

struct plan { struct lg_gguf_writer *w; struct planned *t; int n, cap; uint64_t seed; };

static int plan_add(struct plan *p, const char *name, uint32_t type, uint64_t cols, uint64_t rows, float centre) {
    if (p->n == p->cap) {
        p->cap = p->cap ? p->cap * 2 : 256;
        p->t = realloc(p->t, (size_t)p->cap * sizeof *p->t);
        if (!p->t) return -1;
    }
    uint64_t dims[2] = { cols, rows };
    int idx = lg_gw_add_tensor(p->w, name, type, rows > 1 || type == GGML_TYPE_Q4_0 ? 2 : 1, dims);
    if (idx < 0) return -1;
    p->t[p->n++] = (struct planned){ idx, type, rows, cols, centre, mix64(p->seed ^ name_hash(name)) };
    return 0;
}
static int add_layer(struct plan *p, int L, const char *leaf, uint32_t type, uint64_t cols, uint64_t rows, float centre) {
    char name[96];
    snprintf(name, sizeof name, "blk.%d.%s", L, leaf);
    return plan_add(p, name, type, cols, rows, centre);
}

static void fill(const struct planned *t, void *dst, float norm_jitter, float w_std) {
    if (t->type != GGML_TYPE_Q4_0 && t->centre == 0.0f) {    /* a matrix kept in a float type: N(0, w_std) like the q4_0 ones */
        const uint64_t n = t->cols * t->rows;
        for (uint64_t i = 0; i < n; i += 2) {
            float a, b;
            normal_pair(t->key, i / 2, &a, &b);
            const float v[2] = { a * w_std, b * w_std };
            for (int e = 0; e < 2 && i + e < n; e++) {
                if (t->type == GGML_TYPE_F32) ((float *)dst)[i + e] = v[e];
                else if (t->type == GGML_TYPE_F16) ((uint16_t *)dst)[i + e] = lg_f32_to_f16(v[e]);
                else { uint32_t u; memcpy(&u, &v[e], 4); ((uint16_t *)dst)[i + e] = (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16); }
            }
        }
        return;
    }
    if (t->type == GGML_TYPE_F32) {
        float *o = dst;
        for (uint64_t i = 0; i < t->cols * t->rows; i++)
            o[i] = t->centre * (1.0f + norm_jitter * uniform_pm1(t->key, i));
        return;
    }
    const uint64_t row_bytes = t->cols / 32 * LG_Q4_0_BYTES;
    #pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < (int64_t)t->rows; r++) {
        float buf[32];
        unsigned char *o = (unsigned char *)dst + (uint64_t)r * row_bytes;
        for (uint64_t b = 0; b < t->cols / 32; b++) {
            uint64_t ctr = ((uint64_t)r * (t->cols / 32) + b) * 16;
            for (int j = 0; j < 16; j++) {
                normal_pair(t->key, ctr + (uint64_t)j, &buf[2 * j], &buf[2 * j + 1]);
                buf[2 * j] *= w_std; buf[2 * j + 1] *= w_std;
            }
            lg_quantize_q4_0(buf, o + b * LG_Q4_0_BYTES, 32);
        }
    }
}

int lg_synth_write(const char *path, const struct lg_synth_spec *s) {
    const int hd_l = s->head_dim, hd_g = s->head_dim_full > 0 ? s->head_dim_full : s->head_dim;
    if (s->n_layer <= 0 || s->n_embd % 32 || s->n_ff % 32 || hd_l % 32 || hd_g % 32 ||
        (s->ple && s->ple % 32) || s->n_head % s->n_head_kv || s->shared_kv_layers >= s->n_layer ||
        (s->shared_kv_layers > 0 && s->n_layer - s->shared_kv_layers < 2)) {
        fprintf(stderr, "lg_synth_write: invalid spec\n");
        return -1;
    }
    struct lg_gguf_writer *w = lg_gw_open(path, 3, 32);
    if (!w) { perror(path); return -2; }
    const char *A = "gemma4";
    char key[128];
    int rc = lg_gw_meta_str(w, "general.architecture", A);
#define KU(leaf, v) (snprintf(key, sizeof key, "%s.%s", A, leaf), rc |= lg_gw_meta_u32(w, key, (uint32_t)(v)))
#define KF(leaf, v) (snprintf(key, sizeof key, "%s.%s", A, leaf), rc |= lg_gw_meta_f32(w, key, (v)))
    KU("block_count", s->n_layer);
    KU("embedding_length", s->n_embd);
    KU("attention.head_count", s->n_head);
    KU("attention.head_count_kv", s->n_head_kv);
    KU("feed_forward_length", s->n_ff);
    KU("context_length", s->n_ctx);
    KU("attention.sliding_window", s->sliding_window);
    KU("embedding_length_per_layer_input", s->ple);
    KF("attention.layer_norm_rms_epsilon", s->rms_eps);
    KF("rope.freq_base", s->rope_base);
    KF("rope.freq_base_swa", s->rope_base_swa);
    KF("final_logit_softcapping", s->softcap);
    KU("attention.key_length", hd_g);
    KU("attention.key_length_swa", hd_l);
    KU("attention.shared_kv_layers", s->shared_kv_layers);
    int8_t *pat = calloc((size_t)s->n_layer, 1);
    if (!pat) { lg_gw_close(w); return -3; }
    for (int L = 0; L < s->n_layer; L++)
        pat[L] = s->local_period > 0 && (L % s->local_period) != s->local_period - 1;
    snprintf(key, sizeof key, "%s.attention.sliding_window_pattern", A);
    rc |= lg_gw_meta_array(w, key, GGUF_TYPE_BOOL, (uint64_t)s->n_layer, pat);
    rc |= lg_gw_meta_empty_strings(w, "tokenizer.ggml.tokens", (uint64_t)s->n_vocab);
    if (rc) { free(pat); lg_gw_close(w); return -4; }

    struct plan p = { w, NULL, 0, 0, s->seed };
    const uint64_t E = (uint64_t)s->n_embd, F = (uint64_t)s->n_ff, P = (uint64_t)s->ple;
    const int n_kv_start = s->n_layer - s->shared_kv_layers;
    const uint32_t ple_t = s->ple_float == 1 ? GGML_TYPE_F32 : s->ple_float == 2 ? GGML_TYPE_F16 : s->ple_float == 3 ? GGML_TYPE_BF16 : GGML_TYPE_Q4_0;
    rc |= plan_add(&p, "token_embd.weight", GGML_TYPE_Q4_0, E, (uint64_t)s->n_vocab, 0);
    rc |= plan_add(&p, "output_norm.weight", GGML_TYPE_F32, E, 1, 1.0f);
    if (s->has_rope_freqs) rc |= plan_add(&p, "rope_freqs.weight", GGML_TYPE_F32, (uint64_t)hd_g / 2, 1, 1.0f);
    if (P) {
        rc |= plan_add(&p, "per_layer_token_embd.weight", GGML_TYPE_Q4_0, P * (uint64_t)s->n_layer, (uint64_t)s->n_vocab, 0);
        rc |= plan_add(&p, "per_layer_model_proj.weight", ple_t, E, P * (uint64_t)s->n_layer, 0);
        rc |= plan_add(&p, "per_layer_proj_norm.weight", GGML_TYPE_F32, P, 1, 1.0f);
    }
    for (int L = 0; L < s->n_layer && !rc; L++) {
        const uint64_t hd = pat[L] ? (uint64_t)hd_l : (uint64_t)hd_g;
        const uint64_t qd = hd * (uint64_t)s->n_head, kd = hd * (uint64_t)s->n_head_kv;
        const float qk = s->qk_norm > 0 ? s->qk_norm : sqrtf(1.28f / sqrtf((float)hd));
        rc |= add_layer(&p, L, "attn_norm.weight", GGML_TYPE_F32, E, 1, 1.0f);
        rc |= add_layer(&p, L, "attn_q.weight", GGML_TYPE_Q4_0, E, qd, 0);
        rc |= add_layer(&p, L, "attn_q_norm.weight", GGML_TYPE_F32, hd, 1, qk);
        if (L < n_kv_start) {
            rc |= add_layer(&p, L, "attn_k.weight", GGML_TYPE_Q4_0, E, kd, 0);
            if (s->has_v) rc |= add_layer(&p, L, "attn_v.weight", GGML_TYPE_Q4_0, E, kd, 0);
            rc |= add_layer(&p, L, "attn_k_norm.weight", GGML_TYPE_F32, hd, 1, qk);
        }
        rc |= add_layer(&p, L, "attn_output.weight", GGML_TYPE_Q4_0, qd, E, 0);
        rc |= add_layer(&p, L, "post_attention_norm.weight", GGML_TYPE_F32, E, 1, 1.0f);
        rc |= add_layer(&p, L, "ffn_norm.weight", GGML_TYPE_F32, E, 1, 1.0f);
        rc |= add_layer(&p, L, "ffn_gate.weight", GGML_TYPE_Q4_0, E, F, 0);
        rc |= add_layer(&p, L, "ffn_up.weight", GGML_TYPE_Q4_0, E, F, 0);
        rc |= add_layer(&p, L, "ffn_down.weight", GGML_TYPE_Q4_0, F, E, 0);
        rc |= add_layer(&p, L, "post_ffw_norm.weight", GGML_TYPE_F32, E, 1, 1.0f);
        if (P) {
            rc |= add_layer(&p, L, "inp_gate.weight", ple_t, E, P, 0);
            rc |= add_layer(&p, L, "proj.weight", ple_t, P, E, 0);
            rc |= add_layer(&p, L, "post_norm.weight", GGML_TYPE_F32, E, 1, 1.0f);
        }
        if (s->out_scale > 0) rc |= add_layer(&p, L, "layer_output_scale.weight", GGML_TYPE_F32, 1, 1, s->out_scale);
    }
    free(pat);
    if (rc || lg_gw_commit(w) != 0) { fprintf(stderr, "lg_synth_write: cannot lay out %s\n", path); free(p.t); lg_gw_close(w); return -5; }
    for (int i = 0; i < p.n; i++) {
        size_t bytes;
        void *dst = lg_gw_tensor_data(w, p.t[i].index, &bytes);
        fill(&p.t[i], dst, s->norm_jitter, s->w_std);
    }
    free(p.t);
    return lg_gw_close(w) == 0 ? 0 : -6;
}

/* The draft head file the reference's mtp_open reads (src/mtp.c:124-215): architecture
 * "gemma4-assistant", its keys under that prefix, the two next-token projections, its own
 * token_embd (the head's LM head, inner width) and per block q / output / FFN matrices and norms;
 * no k/v projections (the blocks read the target's cache). */
int lg_synth_write_assistant(const char *path, const struct lg_synth_assistant_spec *s) {
    if (s->n_layer <= 0 || s->n_inner % 32 || s->n_backbone % 32 || s->n_ff % 32 || s->head_dim_swa % 32 ||
        s->head_dim_full % 32 || s->n_full < 0 || s->n_full > s->n_layer || s->n_head <= 0) {
        fprintf(stderr, "lg_synth_write_assistant: invalid spec\n");
        return -1;
    }
    struct lg_gguf_writer *w = lg_gw_open(path, 3, 32);
    if (!w) { perror(path); return -2; }
    const char *A = "gemma4-assistant";
    char key[128];
    int rc = lg_gw_meta_str(w, "general.architecture", A);
#define KU(leaf, v) (snprintf(key, sizeof key, "%s.%s", A, leaf), rc |= lg_gw_meta_u32(w, key, (uint32_t)(v)))
#define KF(leaf, v) (snprintf(key, sizeof key, "%s.%s", A, leaf), rc |= lg_gw_meta_f32(w, key, (v)))
    KU("block_count", s->n_layer);
    KU("embedding_length", s->n_inner);
    KU("embedding_length_out", s->n_backbone);
    KU("attention.head_count", s->n_head);
    KU("feed_forward_length", s->n_ff);
    KF("attention.layer_norm_rms_epsilon", s->rms_eps);
    KF("rope.freq_base", s->rope_base);
    KF("rope.freq_base_swa", s->rope_base_swa);
    KF("final_logit_softcapping", s->softcap);
#undef KU
#undef KF
    if (rc) { lg_gw_close(w); return -4; }
    struct plan p = { w, NULL, 0, 0, s->seed };
    const uint64_t I = (uint64_t)s->n_inner, B = (uint64_t)s->n_backbone, F = (uint64_t)s->n_ff;
    rc |= plan_add(&p, "token_embd.weight", GGML_TYPE_Q4_0, I, (uint64_t)s->n_vocab, 0);
    rc |= plan_add(&p, "output_norm.weight", GGML_TYPE_F32, I, 1, 1.0f);
    rc |= plan_add(&p, "nextn.pre_projection.weight", GGML_TYPE_Q4_0, 2 * B, I, 0);
    if (s->has_post) rc |= plan_add(&p, "nextn.post_projection.weight", GGML_TYPE_Q4_0, I, B, 0);
    for (int L = 0; L < s->n_layer && !rc; L++) {
        const int full = L >= s->n_layer - s->n_full;
        const uint64_t hd = (uint64_t)(full ? s->head_dim_full : s->head_dim_swa), qd = hd * (uint64_t)s->n_head;
        const float qk = s->qk_norm > 0 ? s->qk_norm : sqrtf(1.28f / sqrtf((float)hd));
        rc |= add_layer(&p, L, "attn_norm.weight", GGML_TYPE_F32, I, 1, 1.0f);
        rc |= add_layer(&p, L, "attn_q.weight", GGML_TYPE_Q4_0, I, qd, 0);
        rc |= add_layer(&p, L, "attn_q_norm.weight", GGML_TYPE_F32, hd, 1, qk);
        rc |= add_layer(&p, L, "attn_output.weight", GGML_TYPE_Q4_0, qd, I, 0);
        rc |= add_layer(&p, L, "post_attention_norm.weight", GGML_TYPE_F32, I, 1, 1.0f);
        rc |= add_layer(&p, L, "ffn_norm.weight", GGML_TYPE_F32, I, 1, 1.0f);
        rc |= add_layer(&p, L, "ffn_gate.weight", GGML_TYPE_Q4_0, I, F, 0);
        rc |= add_layer(&p, L, "ffn_up.weight", GGML_TYPE_Q4_0, I, F, 0);
        rc |= add_layer(&p, L, "ffn_down.weight", GGML_TYPE_Q4_0, F, I, 0);
        rc |= add_layer(&p, L, "post_ffw_norm.weight", GGML_TYPE_F32, I, 1, 1.0f);
        if (s->out_scale > 0) rc |= add_layer(&p, L, "layer_output_scale.weight", GGML_TYPE_F32, 1, 1, s->out_scale);
    }
    if (rc || lg_gw_commit(w) != 0) { fprintf(stderr, "lg_synth_write_assistant: cannot lay out %s\n", path); free(p.t); lg_gw_close(w); return -5; }
    for (int i = 0; i < p.n; i++) {
        size_t bytes;
        void *dst = lg_gw_tensor_data(w, p.t[i].index, &bytes);
        fill(&p.t[i], dst, s->norm_jitter, s->w_std);
    }
    free(p.t);
    return lg_gw_close(w) == 0 ? 0 : -6;
}
