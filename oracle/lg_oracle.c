/* lg_oracle.c — CPU oracle for the MTP speculative-verify path.  TEST INFRASTRUCTURE ONLY:
 * nothing shipped may link or call this file (see lg_oracle.h).
 *
 * What pins each part (the tests named here live in tests/):
 *   lgo_block_dot, q4_0 layout     closed form sum((nib-8)*q) by brute force in numpy; q4_0 bytes->floats
 *                                  fixture produced by the reference's dequantize_into (test_oracle_primitives)
 *   lgo_quant_q8                   numpy restatement with ties-to-even, zero group, saturating cases
 *   lgo_matmul_q4q8                float64 accumulation of d_w*d_x*dot within 1e-5; both orders agree
 *   lgo_matmul_fw                  f32/f16/bf16 weight rows: float64 product within 1e-6 of the sum of magnitudes, unit
 *                                  rows and small-integer operands exactly, the serial-order matmul within rounding
 *                                  (test_oracle_primitives); models whose per-layer-embedding matrices are float-typed:
 *                                  LGO_REF bit-identical to the reference build and its fixture, LGO_I8_F32 within 1e-3
 *   lgo_f32_to_f16 / f16_to_f32    numpy float16 over dense samples incl. subnormals, ties, overflow
 *   lgo_expf/tanhf/sincosf/gelu    double-precision libm within a few ulp (test_lg_math)
 *   lgo_rmsnorm, lgo_rope          float64 closed forms
 *   lgo_attention_f16              float64 softmax(QK^T)V over the ring; tiled == two-pass within 1e-6
 *   lgo_accept                     exhaustive over all match patterns, rows <= 5
 *   lgo_forward(LGO_REF)           bit-identical logits and tokens against the reference's own CPU
 *                                  backend built from its sources (oracle/_ref), and against the
 *                                  committed fixtures those runs produced (tests/golden)
 *   lgo_forward(LGO_I8 / _LIBM)    built from the pinned primitives above.  The reference's CUDA int8 path
 *                                  it restates cannot run without an NVIDIA device: PARITY UNPINNED for the
 *                                  last bits of its float sums (this file fixes its own summation orders).
 *                                  The composition (quantization points, op order) is held by LGO_I8_F32: the
 *                                  same function with the quantization switched off agrees with LGO_REF to
 *                                  float reordering noise (1e-3 relative L2 of the logits at every step, every
 *                                  argmax equal), and with it on stays inside the q8 noise band; plus
 *                                  spec == decode (tests/test_oracle_model.py).
 *   lgo_mtp_draft(LGO_REF)         bit-identical tokens, hidden state and logits against the reference's host
 *                                  draft head (src/mtp.c, in oracle/_ref) and its committed fixtures
 *                                  (tests/test_oracle_draft.py), including that file's f16 subnormal reading
 *   lgo_mtp_draft(LGO_I8), lgo_mtp_post   same code path with q8 activations and this build's orders; the
 *                                  reference's device draft (f16 weights, CUDA sums) cannot run here: PARITY
 *                                  UNPINNED for its last bits and for the chained draft's post-projection,
 *                                  which has no CPU counterpart in the reference.  Held by LGO_I8_F32 (same
 *                                  code path, quantization off) agreeing with LGO_REF to 1e-3, by the q8 gap to
 *                                  LGO_REF and by the key-range test (a draft at pos reads positions < pos only).
 *   lgo_forward_spec_all           equal to lgo_forward_spec in adv, out[0..adv-1] and hidden
 */
#define _GNU_SOURCE
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#include <omp.h>

#include "lg_oracle.h"
#include "../include/lg_math.h"
#include "../little-gemma_amd/host/gguf.h"
#include "../little-gemma_amd/host/quant.h"
#include "../little-gemma_amd/host/model.h"

void lgo_set_threads(int n) { if (n > 0) omp_set_num_threads(n); }

float lgo_expf(float x) { return lg_expf(x); }
float lgo_tanhf(float x) { return lg_tanhf(x); }
void  lgo_sincosf(float x, float *s, float *c) { lg_sincosf(x, s, c); }
uint16_t lgo_f32_to_f16(float f) { return lg_f32_to_f16(f); }
float lgo_f16_to_f32(uint16_t h) { return lg_f16_to_f32(h); }

/* GELU, tanh form (src/cpu/model-cpu.c:108-111; src/cuda/model-cuda.cuh:663-666) */
float lgo_gelu(float x, int exact) {
    if (exact) return lg_gelu(x);
    const float k = 0.7978845608028654f;
    return 0.5f * x * (1.0f + tanhf(k * (x + 0.044715f * x * x * x)));
}

/* adjacent-pair binary tree over w lane values (w a power of two) */
static float tree_sum(float *p, int w) {
    for (int s = 1; s < w; s <<= 1)
        for (int l = 0; l + s < w; l += 2 * s) p[l] = p[l] + p[l + s];
    return p[0];
}

/* ---- activation quantization (src/cuda/model-cuda.cuh:84-92): per 32 floats
 * amax, d = amax/127, id = 1/d (0 when d == 0), q = rint_even(x*id); scale stays f32 */
void lgo_quant_q8(const float *x, int n, int8_t *q, float *d, int32_t *sum) {
    for (int g = 0; g < n / 32; g++) {
        const float *xb = x + g * 32;
        float amax = 0.0f;
        for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(xb[i]));
        float dd = amax / 127.0f, id = dd > 0.0f ? 1.0f / dd : 0.0f;
        int s = 0;
        for (int i = 0; i < 32; i++) { int v = (int)lg_rintf(xb[i] * id); q[g * 32 + i] = (int8_t)v; s += v; }
        d[g] = dd;
        if (sum) sum[g] = s;
    }
}

/* ---- int32 dot of one q4_0 block with 32 int8 (src/quant.c:276-285 element order,
 * src/cuda/model-cuda-i8.cu:200-213 arithmetic) */
int32_t lgo_block_dot(const unsigned char *blk, const int8_t *q) {
    int32_t acc = 0;
    for (int j = 0; j < 16; j++) {
        acc += ((int)(blk[2 + j] & 15) - 8) * (int)q[j];
        acc += ((int)(blk[2 + j] >> 4) - 8) * (int)q[j + 16];
    }
    return acc;
}

/* K segments of this build's matmul order: 8, or 32 for rows of more than 128 blocks whose
 * block count 32 divides (the wide ffn_down rows), so that every lane's serial chain stays
 * short; a row of 240 blocks (two 3840-wide halves) stays at 8 segments of 30. */
int lgo_segments(int k) { return (k / 32 > 128 && (k / 32) % 32 == 0) ? 32 : 8; }

/* ---- q4_0 x q8 matmul.  out[j*m+i] = sum_b (xd[j][b]*dw[i][b]) * dot(i,j,b)
 * (src/cuda/model-cuda-i8.cu:813-903); `order` picks how the f32 terms are summed. */
void lgo_matmul_q4q8(const void *w, int k, int m, const int8_t *xq, const float *xd, int rows,
                     float *out, int32_t *dots, int order) {
    const int nb = k / 32, S = lgo_segments(k);
    const unsigned char *base = w;
    if (order == LGO_ORDER_SEG && nb % S) { fprintf(stderr, "lgo_matmul_q4q8: k=%d not a multiple of %d\n", k, 32 * S); abort(); }
    #pragma omp parallel for schedule(static)
    for (int i = 0; i < m; i++) {
        const unsigned char *row = base + (size_t)i * nb * LG_Q4_0_BYTES;
        for (int j = 0; j < rows; j++) {
            const int8_t *aq = xq + (size_t)j * k;
            const float *ad = xd + (size_t)j * nb;
            float lane[32];
            if (order == LGO_ORDER_SEG) {
                const int per = nb / S;
                for (int s = 0; s < S; s++) {
                    float p = 0.0f;
                    for (int b = s * per; b < (s + 1) * per; b++) {
                        const unsigned char *blk = row + (size_t)b * LG_Q4_0_BYTES;
                        uint16_t h; memcpy(&h, blk, 2);
                        int32_t dot = lgo_block_dot(blk, aq + b * 32);
                        if (dots) dots[((size_t)j * m + i) * nb + b] = dot;
                        p = lg_fmaf(ad[b] * lg_f16_to_f32(h), (float)dot, p);
                    }
                    lane[s] = p;
                }
                out[(size_t)j * m + i] = tree_sum(lane, S);
            } else {
                for (int l = 0; l < 32; l++) lane[l] = 0.0f;
                for (int b = 0; b < nb; b++) {
                    const unsigned char *blk = row + (size_t)b * LG_Q4_0_BYTES;
                    uint16_t h; memcpy(&h, blk, 2);
                    int32_t dot = lgo_block_dot(blk, aq + b * 32);
                    if (dots) dots[((size_t)j * m + i) * nb + b] = dot;
                    lane[b & 31] = lg_fmaf(ad[b] * lg_f16_to_f32(h), (float)dot, lane[b & 31]);
                }
                for (int o = 16; o > 0; o >>= 1)              /* shfl_down tree */
                    for (int l = 0; l < o; l++) lane[l] = lane[l] + lane[l + o];
                out[(size_t)j * m + i] = lane[0];
            }
        }
    }
}

/* ---- f32-activation matmul: dequantize the row, serial left-to-right dot
 * (src/cpu/model-cpu.c:147-164) */
void lgo_matmul_f32(const void *w, uint32_t type, int k, int m, const float *x, float *out) {
    const size_t row_bytes = (size_t)(k / ggml_blck_size(type)) * ggml_type_size(type);
    #pragma omp parallel
    {
        float *buf = malloc((size_t)k * sizeof(float));
        #pragma omp for schedule(static)
        for (int i = 0; i < m; i++) {
            dequantize_into(type, (const unsigned char *)w + (size_t)i * row_bytes, buf, k);
            float s = 0.0f;
            for (int j = 0; j < k; j++) s += buf[j] * x[j];
            out[i] = s;
        }
        free(buf);
    }
}

/* ---- matmul against a weight matrix kept in a float type (f32 / f16 / bf16), f32 activations: what the int8
 * backend does for the per-layer-embedding matrices of QAT conversions, which stay at full precision
 * (src/cuda/model-cuda-i8.cu:645-653, :846-895: w * x summed per lane, then a lane tree; nothing is quantized).
 * This build's order: 64 lane partials, element e belongs to lane (e/4)%64, fma in ascending e, adjacent-pair tree
 * over the lanes. */
void lgo_matmul_fw(const void *w, uint32_t type, int k, int m, const float *x, float *out) {
    const size_t row_bytes = (size_t)(k / ggml_blck_size(type)) * ggml_type_size(type);
    #pragma omp parallel
    {
        float *buf = malloc((size_t)k * sizeof(float));
        #pragma omp for schedule(static)
        for (int i = 0; i < m; i++) {
            dequantize_into(type, (const unsigned char *)w + (size_t)i * row_bytes, buf, k);
            float lane[64] = { 0 };
            for (int e = 0; e < k; e++) lane[(e >> 2) & 63] = lg_fmaf(buf[e], x[e], lane[(e >> 2) & 63]);
            out[i] = tree_sum(lane, 64);
        }
        free(buf);
    }
}

/* ---- rmsnorm: x * (1/sqrt(mean(x^2)+eps)) * w   (src/cpu/model-cpu.c:78-83,100-105).
 * tree = 0: serial sum like the reference CPU; tree = 1: this build's order
 * (256 lane partials, element i belongs to lane (i/4)%256, fma in ascending i, adjacent-pair
 * tree over the lanes). w may be NULL. */
void lgo_rmsnorm(float *out, const float *x, const float *w, int n, float eps, int tree) {
    float ss = 0.0f;
    if (!tree) for (int i = 0; i < n; i++) ss += x[i] * x[i];
    else {
        float lane[256] = { 0 };
        for (int i = 0; i < n; i++) lane[(i >> 2) & 255] = lg_fmaf(x[i], x[i], lane[(i >> 2) & 255]);
        ss = tree_sum(lane, 256);
    }
    float s = 1.0f / sqrtf(ss / (float)n + eps);
    if (w) for (int i = 0; i < n; i++) out[i] = x[i] * s * w[i];
    else   for (int i = 0; i < n; i++) out[i] = x[i] * s;
}

/* ---- NeoX rotary on one head (src/cpu/model-cpu.c:87-97); freq_tab[i] = powf(base, -2i/d) */
void lgo_rope(float *v, int d, int pos, const float *tab, const float *ff, int exact) {
    int half = d / 2;
    for (int i = 0; i < half; i++) {
        float ang = (float)pos * tab[i] / (ff ? ff[i] : 1.0f);
        float c, s;
        if (exact) lg_sincosf(ang, &s, &c); else { c = cosf(ang); s = sinf(ang); }
        float a = v[i], b = v[i + half];
        v[i] = a * c - b * s;
        v[i + half] = a * s + b * c;
    }
}

/* ---- attention of one query head over an f16 cache, scale 1.0 (src/cpu/model-cpu.c:382-400).
 * tiled = 0: two-pass softmax in the reference CPU's order.
 * tiled = 1: this build's order — 32-key tiles aligned to absolute positions; per tile
 *   score = (a0+a1)+(a2+a3) with a_c the fma chain over dims i%4==c; m = max; e = exp(s-m);
 *   l = adjacent tree over the 32 key slots; acc[d] = fma chain over slots ascending;
 *   tiles merged ascending with weights exp(m_tile - M), then out = acc / L. */
static float kvf(const void *base, size_t i, int f16) {
    return f16 ? lg_f16_to_f32(((const uint16_t *)base)[i]) : ((const float *)base)[i];
}
static void attention_tiled(float *out, const float *q, const void *kc, const void *vc, int f16,
                            int hd, int kv_dim, int kvh, int seq, int start, int pos, int exact);
void lgo_attention_f16(float *out, const float *q, const uint16_t *kc, const uint16_t *vc,
                       int hd, int kv_dim, int kvh, int seq, int start, int pos, int tiled, int exact) {
    if (tiled) { attention_tiled(out, q, kc, vc, 1, hd, kv_dim, kvh, seq, start, pos, exact); return; }
    {
        int T = pos - start + 1;
        float *att = malloc((size_t)T * sizeof(float));
        float mx = -INFINITY;
        for (int t = start; t <= pos; t++) {
            const uint16_t *kr = kc + (size_t)(t % seq) * kv_dim + (size_t)kvh * hd;
            float s = 0.0f;
            for (int i = 0; i < hd; i++) s += q[i] * lg_f16_to_f32(kr[i]);
            att[t - start] = s;
            if (s > mx) mx = s;
        }
        float sum = 0.0f;
        for (int t = 0; t < T; t++) { att[t] = exact ? lg_expf(att[t] - mx) : expf(att[t] - mx); sum += att[t]; }
        for (int t = 0; t < T; t++) att[t] /= sum;
        for (int i = 0; i < hd; i++) out[i] = 0.0f;
        for (int t = start; t <= pos; t++) {
            const uint16_t *vr = vc + (size_t)(t % seq) * kv_dim + (size_t)kvh * hd;
            float a = att[t - start];
            for (int i = 0; i < hd; i++) out[i] += a * lg_f16_to_f32(vr[i]);
        }
        free(att);
    }
}
/* the tiled order over a cache of binary16 (f16 = 1) or float rows */
static void attention_tiled(float *out, const float *q, const void *kc, const void *vc, int f16,
                            int hd, int kv_dim, int kvh, int seq, int start, int pos, int exact) {
    const int TK = 32, n_lo = start / TK, n_hi = pos / TK, nt = n_hi - n_lo + 1;
    float *tm = malloc((size_t)nt * sizeof(float)), *tl = malloc((size_t)nt * sizeof(float));
    float *tacc = malloc((size_t)nt * hd * sizeof(float));
    for (int n = n_lo; n <= n_hi; n++) {
        float sc[32], e[32];
        int valid[32];
        float m = -INFINITY;
        for (int sl = 0; sl < TK; sl++) {
            int t = n * TK + sl;
            valid[sl] = t >= start && t <= pos;
            if (!valid[sl]) continue;
            const size_t ko = (size_t)(t % seq) * kv_dim + (size_t)kvh * hd;
            float a[4] = { 0, 0, 0, 0 };
            for (int i = 0; i < hd; i++) a[i & 3] = lg_fmaf(q[i], kvf(kc, ko + i, f16), a[i & 3]);
            sc[sl] = (a[0] + a[1]) + (a[2] + a[3]);
            if (sc[sl] > m) m = sc[sl];
        }
        for (int sl = 0; sl < TK; sl++)
            e[sl] = valid[sl] ? (exact ? lg_expf(sc[sl] - m) : expf(sc[sl] - m)) : 0.0f;
        float *acc = tacc + (size_t)(n - n_lo) * hd;
        for (int i = 0; i < hd; i++) acc[i] = 0.0f;
        for (int sl = 0; sl < TK; sl++) {
            if (!valid[sl]) continue;
            int t = n * TK + sl;
            const size_t vo = (size_t)(t % seq) * kv_dim + (size_t)kvh * hd;
            for (int i = 0; i < hd; i++) acc[i] = lg_fmaf(e[sl], kvf(vc, vo + i, f16), acc[i]);
        }
        tm[n - n_lo] = m;
        tl[n - n_lo] = tree_sum(e, 32);
    }
    float M = -INFINITY, L = 0.0f;
    for (int n = 0; n < nt; n++) if (tm[n] > M) M = tm[n];
    for (int i = 0; i < hd; i++) out[i] = 0.0f;
    for (int n = 0; n < nt; n++) {
        float wn = exact ? lg_expf(tm[n] - M) : expf(tm[n] - M);
        L = lg_fmaf(tl[n], wn, L);
        for (int i = 0; i < hd; i++) out[i] = lg_fmaf(tacc[(size_t)n * hd + i], wn, out[i]);
    }
    for (int i = 0; i < hd; i++) out[i] = out[i] / L;
    free(tm); free(tl); free(tacc);
}

/* ---- greedy accept rule (src/cuda/mtp-kernel.cuh:114-116, src/cpu/model-cpu.c:51-58) */
int lgo_accept(const int *toks, const int *out, int rows) {
    int adv = 1;
    while (adv < rows && out[adv - 1] == toks[adv]) adv++;
    return adv;
}

/* sliding-window ring length of the int8 class: the window plus spare rows for the widest block written before any
 * of its queries runs (512 prompt rows for caches of 1024 positions and more, 128 below; src/cuda/model-cuda.cuh:1016-1035
 * uses window + widest chunk), rounded to the 32-key attention tile.  A layout choice, not arithmetic: results do not
 * depend on it; it is restated here so that cache rows can be compared ring row by ring row. */
int lgo_ring_rows(int window, int max_seq) {
    int r = (window + (max_seq >= 1024 ? 512 : 128) + 31) / 32 * 32;
    return r < max_seq ? r : max_seq;
}

/* ======================  whole model  ===================================== */

struct lgo_layer {
    const float *attn_norm, *q_norm, *k_norm, *post_attn, *ffn_norm, *post_ffw, *post_norm, *out_scale;
    const struct gguf_tensor *wq, *wk, *wv, *wo, *gate, *up, *down, *inp_gate, *proj;
};
struct lgo_model {
    struct gguf_context *ctx;
    struct model m;
    struct lgo_layer *l;
    const struct gguf_tensor *token_embd, *pte, *pmp;
    const float *output_norm, *rope_freqs, *pl_proj_norm;
    float *tab_full, *tab_swa;          /* powf(base, -2i/hd) per layer kind */
};
struct lgo_kv {
    int n_layer, max_seq, mode;
    int *kv_dim, *seq, *f16;
    void **k, **v;
};

static const float *f32_tensor(const struct gguf_context *g, const char *name) {
    const struct gguf_tensor *t = gguf_find_tensor(g, name);
    return t ? (const float *)t->data : NULL;
}
static const struct gguf_tensor *layer_t(const struct gguf_context *g, int L, const char *leaf) {
    char name[96];
    snprintf(name, sizeof name, "blk.%d.%s", L, leaf);
    return gguf_find_tensor(g, name);
}
static const float *layer_f(const struct gguf_context *g, int L, const char *leaf) {
    const struct gguf_tensor *t = layer_t(g, L, leaf);
    return t ? (const float *)t->data : NULL;
}

struct lgo_model *lgo_model_open(const char *path) {
    struct lgo_model *o = calloc(1, sizeof *o);
    if (!o) return NULL;
    o->ctx = load_gguf(path);
    if (!o->ctx || model_init(&o->m, o->ctx) != 0) { lgo_model_close(o); return NULL; }
    const struct config *c = &o->m.cfg;
    const struct gguf_context *g = o->ctx;
    o->l = calloc((size_t)c->n_layer, sizeof *o->l);
    o->token_embd = gguf_find_tensor(g, "token_embd.weight");
    o->output_norm = f32_tensor(g, "output_norm.weight");
    o->rope_freqs = f32_tensor(g, "rope_freqs.weight");
    o->pte = gguf_find_tensor(g, "per_layer_token_embd.weight");
    o->pmp = gguf_find_tensor(g, "per_layer_model_proj.weight");
    o->pl_proj_norm = f32_tensor(g, "per_layer_proj_norm.weight");
    if (!o->l || !o->token_embd || !o->output_norm) { lgo_model_close(o); return NULL; }
    int maxhd = 0;
    for (int L = 0; L < c->n_layer; L++) {
        struct lgo_layer *y = &o->l[L];
        if (o->m.head_dim[L] > maxhd) maxhd = o->m.head_dim[L];
        y->attn_norm = layer_f(g, L, "attn_norm.weight");
        y->q_norm = layer_f(g, L, "attn_q_norm.weight");
        y->k_norm = layer_f(g, L, "attn_k_norm.weight");
        y->post_attn = layer_f(g, L, "post_attention_norm.weight");
        y->ffn_norm = layer_f(g, L, "ffn_norm.weight");
        y->post_ffw = layer_f(g, L, "post_ffw_norm.weight");
        y->post_norm = layer_f(g, L, "post_norm.weight");
        y->out_scale = layer_f(g, L, "layer_output_scale.weight");
        y->wq = layer_t(g, L, "attn_q.weight");   y->wk = layer_t(g, L, "attn_k.weight");
        y->wv = layer_t(g, L, "attn_v.weight");   y->wo = layer_t(g, L, "attn_output.weight");
        y->gate = layer_t(g, L, "ffn_gate.weight"); y->up = layer_t(g, L, "ffn_up.weight");
        y->down = layer_t(g, L, "ffn_down.weight");
        y->inp_gate = layer_t(g, L, "inp_gate.weight"); y->proj = layer_t(g, L, "proj.weight");
    }
    o->tab_full = malloc((size_t)maxhd * sizeof(float));
    o->tab_swa = malloc((size_t)maxhd * sizeof(float));
    return o;
}

void lgo_model_close(struct lgo_model *o) {
    if (!o) return;
    free(o->l); free(o->tab_full); free(o->tab_swa);
    model_free(&o->m);
    free_gguf(o->ctx);
    free(o);
}

int lgo_model_info(const struct lgo_model *o, int32_t *out, int cap) {
    const struct config *c = &o->m.cfg;
    int32_t v[] = { c->n_layer, c->n_embd, c->n_head, c->n_vocab, c->n_embd_per_layer, c->n_kv_start,
                    c->sliding_window, c->n_ff, c->n_head_kv, c->head_dim_swa, c->head_dim_full, c->n_ctx };
    int n = (int)(sizeof v / sizeof v[0]);
    for (int i = 0; i < n && i < cap; i++) out[i] = v[i];
    return n;
}
int lgo_layer_info(const struct lgo_model *o, int L, int32_t *out4) {
    if (L < 0 || L >= o->m.cfg.n_layer) return -1;
    out4[0] = o->m.is_local[L]; out4[1] = o->m.head_dim[L]; out4[2] = o->m.n_head_kv[L]; out4[3] = o->m.ffn_len[L];
    return 0;
}

/* which layer's cache layer L reads (src/cpu/model-cpu.c:175-179) */
static int kv_source(const struct model *m, int L) {
    if (L < m->cfg.n_kv_start) return L;
    return m->cfg.n_kv_start - (m->is_local[L] ? 2 : 1);
}

/* LGO_REF: src/cpu/model-cpu.c:216-250 (global f16 max_seq rows, sliding f32 `window` rows).
 * int8 class: src/cuda/model-cuda.cuh:998-1051 (f16 everywhere, sliding rings with spare rows). */
struct lgo_kv *lgo_kv_new(const struct lgo_model *o, int max_seq, int mode) {
    const struct config *c = &o->m.cfg;
    struct lgo_kv *kv = calloc(1, sizeof *kv);
    if (!kv) return NULL;
    kv->n_layer = c->n_layer; kv->max_seq = max_seq; kv->mode = mode;
    kv->kv_dim = calloc((size_t)c->n_layer, sizeof(int));
    kv->seq = calloc((size_t)c->n_layer, sizeof(int));
    kv->f16 = calloc((size_t)c->n_layer, sizeof(int));
    kv->k = calloc((size_t)c->n_layer, sizeof(void *));
    kv->v = calloc((size_t)c->n_layer, sizeof(void *));
    for (int L = 0; L < c->n_layer; L++) {
        kv->kv_dim[L] = o->m.n_head_kv[L] * o->m.head_dim[L];
        if (L >= c->n_kv_start) continue;
        int seq = max_seq, local = o->m.is_local[L] && c->sliding_window > 0;
        const int reflike = mode == LGO_REF || mode == LGO_I8_F32;
        if (reflike) { if (local && c->sliding_window < max_seq) seq = c->sliding_window; }
        else if (local) seq = lgo_ring_rows(c->sliding_window, max_seq);
        kv->seq[L] = seq;
        kv->f16[L] = reflike ? !o->m.is_local[L] : 1;
        size_t n = (size_t)seq * kv->kv_dim[L];
        kv->k[L] = calloc(n, kv->f16[L] ? 2 : 4);
        kv->v[L] = calloc(n, kv->f16[L] ? 2 : 4);
    }
    return kv;
}
void lgo_kv_free(struct lgo_kv *kv) {
    if (!kv) return;
    for (int L = 0; L < kv->n_layer; L++) { free(kv->k[L]); free(kv->v[L]); }
    free(kv->k); free(kv->v); free(kv->kv_dim); free(kv->seq); free(kv->f16); free(kv);
}
void *lgo_kv_layer(struct lgo_kv *kv, int L, int which, int *rows, int *width, int *is_f16) {
    if (L < 0 || L >= kv->n_layer) return NULL;
    if (rows) *rows = kv->seq[L];
    if (width) *width = kv->kv_dim[L];
    if (is_f16) *is_f16 = kv->f16[L];
    return which ? kv->v[L] : kv->k[L];
}

static void fill_tab(float *tab, float base, int hd) {
    for (int i = 0; i < hd / 2; i++) tab[i] = powf(base, -2.0f * (float)i / (float)hd);
}

/* ---- the reference `run` forward, restated line for line in meaning
 * (src/cpu/model-cpu.c:267-294 build_per_layer, :301-448 forward_core, :450-457 embedding) */
static int forward_ref(struct lgo_model *o, struct lgo_kv *kv, int token, int pos, float *logits, float *hidden) {
    const struct model *m = &o->m;
    const struct config *c = &m->cfg;
    const int E = c->n_embd, H = c->n_head, ple = c->n_embd_per_layer;
    const float eps = c->rms_eps;
    int maxhd = 0, maxkv = 0;
    for (int L = 0; L < c->n_layer; L++) {
        if (m->head_dim[L] > maxhd) maxhd = m->head_dim[L];
        if (m->n_head_kv[L] * m->head_dim[L] > maxkv) maxkv = m->n_head_kv[L] * m->head_dim[L];
    }
    float *x = dequantize_row(o->token_embd, token, E);
    for (int i = 0; i < E; i++) x[i] *= sqrtf((float)E);
    float *h = malloc((size_t)E * 4), *q = malloc((size_t)H * maxhd * 4), *kb = malloc((size_t)maxkv * 4);
    float *vb = malloc((size_t)maxkv * 4), *xb = malloc((size_t)H * maxhd * 4), *ob = malloc((size_t)E * 4);
    float *g1 = malloc((size_t)c->n_ff * 4), *g2 = malloc((size_t)c->n_ff * 4), *att = malloc((size_t)(pos + 1) * 4);
    float *pg = ple > 0 ? malloc((size_t)ple * 4) : NULL, *ipl = NULL;

    if (ple > 0 && o->pte) {
        const int64_t total = (int64_t)ple * c->n_layer;
        float *tok = dequantize_row(o->pte, token, total);
        float ts = sqrtf((float)ple);
        for (int64_t i = 0; i < total; i++) tok[i] *= ts;
        ipl = malloc((size_t)total * 4);
        lgo_matmul_f32(o->pmp->data, o->pmp->type, E, (int)total, x, ipl);
        float ps = 1.0f / sqrtf((float)E);
        for (int64_t i = 0; i < total; i++) ipl[i] *= ps;
        for (int L = 0; L < c->n_layer; L++) lgo_rmsnorm(ipl + L * ple, ipl + L * ple, o->pl_proj_norm, ple, eps, 0);
        float r2 = 1.0f / sqrtf(2.0f);
        for (int64_t i = 0; i < total; i++) ipl[i] = (ipl[i] + tok[i]) * r2;
        free(tok);
    }

    for (int L = 0; L < c->n_layer; L++) {
        const struct lgo_layer *y = &o->l[L];
        const int local = m->is_local[L], hd = m->head_dim[L], nkv = m->n_head_kv[L];
        const int qd = H * hd, kd = nkv * hd;
        const float base = local ? c->rope_freq_base_swa : c->rope_freq_base;
        const float *ff = local ? NULL : o->rope_freqs;
        float *tab = local ? o->tab_swa : o->tab_full;
        fill_tab(tab, base, hd);

        lgo_rmsnorm(h, x, y->attn_norm, E, eps, 0);
        lgo_matmul_f32(y->wq->data, y->wq->type, E, qd, h, q);
        for (int hh = 0; hh < H; hh++) lgo_rmsnorm(q + hh * hd, q + hh * hd, y->q_norm, hd, eps, 0);
        for (int hh = 0; hh < H; hh++) lgo_rope(q + hh * hd, hd, pos, tab, ff, 0);

        const int src = kv_source(m, L);
        if (L < c->n_kv_start) {
            lgo_matmul_f32(y->wk->data, y->wk->type, E, kd, h, kb);
            if (y->wv) lgo_matmul_f32(y->wv->data, y->wv->type, E, kd, h, vb);
            else memcpy(vb, kb, (size_t)kd * 4);
            for (int hh = 0; hh < nkv; hh++) lgo_rmsnorm(kb + hh * hd, kb + hh * hd, y->k_norm, hd, eps, 0);
            for (int hh = 0; hh < nkv; hh++) lgo_rmsnorm(vb + hh * hd, vb + hh * hd, NULL, hd, eps, 0);
            for (int hh = 0; hh < nkv; hh++) lgo_rope(kb + hh * hd, hd, pos, tab, ff, 0);
            int row = pos % kv->seq[L];
            if (kv->f16[L]) {
                uint16_t *kr = (uint16_t *)kv->k[L] + (size_t)row * kd, *vr = (uint16_t *)kv->v[L] + (size_t)row * kd;
                for (int i = 0; i < kd; i++) { kr[i] = lg_f32_to_f16(kb[i]); vr[i] = lg_f32_to_f16(vb[i]); }
            } else {
                memcpy((float *)kv->k[L] + (size_t)row * kd, kb, (size_t)kd * 4);
                memcpy((float *)kv->v[L] + (size_t)row * kd, vb, (size_t)kd * 4);
            }
        }
        const void *Kc = kv->k[src], *Vc = kv->v[src];
        const int seq = kv->seq[src], kf16 = kv->f16[src];
        int start = (local && c->sliding_window > 0 && pos - c->sliding_window + 1 > 0) ? pos - c->sliding_window + 1 : 0;
        const int gqa = H / nkv;
        for (int hh = 0; hh < H; hh++) {
            const float *qh = q + hh * hd;
            const int kvh = hh / gqa;
            for (int t = start; t <= pos; t++) {
                size_t off = (size_t)(t % seq) * kd + (size_t)kvh * hd;
                float s = 0.0f;
                if (kf16) for (int i = 0; i < hd; i++) s += qh[i] * lg_f16_to_f32(((const uint16_t *)Kc)[off + i]);
                else      for (int i = 0; i < hd; i++) s += qh[i] * ((const float *)Kc)[off + i];
                att[t] = s;
            }
            {   /* softmax (src/cpu/model-cpu.c:113-119) */
                float *a = att + start; int n = pos - start + 1;
                float mx = a[0];
                for (int i = 1; i < n; i++) if (a[i] > mx) mx = a[i];
                float sum = 0.0f;
                for (int i = 0; i < n; i++) { a[i] = expf(a[i] - mx); sum += a[i]; }
                for (int i = 0; i < n; i++) a[i] /= sum;
            }
            float *outh = xb + hh * hd;
            for (int i = 0; i < hd; i++) outh[i] = 0.0f;
            for (int t = start; t <= pos; t++) {
                size_t off = (size_t)(t % seq) * kd + (size_t)kvh * hd;
                float a = att[t];
                if (kf16) for (int i = 0; i < hd; i++) outh[i] += a * lg_f16_to_f32(((const uint16_t *)Vc)[off + i]);
                else      for (int i = 0; i < hd; i++) outh[i] += a * ((const float *)Vc)[off + i];
            }
        }
        lgo_matmul_f32(y->wo->data, y->wo->type, qd, E, xb, ob);
        lgo_rmsnorm(ob, ob, y->post_attn, E, eps, 0);
        for (int i = 0; i < E; i++) x[i] += ob[i];

        const int nff = m->ffn_len[L];
        lgo_rmsnorm(h, x, y->ffn_norm, E, eps, 0);
        lgo_matmul_f32(y->gate->data, y->gate->type, E, nff, h, g1);
        lgo_matmul_f32(y->up->data, y->up->type, E, nff, h, g2);
        for (int i = 0; i < nff; i++) g1[i] = lgo_gelu(g1[i], 0) * g2[i];
        lgo_matmul_f32(y->down->data, y->down->type, nff, E, g1, ob);
        lgo_rmsnorm(ob, ob, y->post_ffw, E, eps, 0);
        for (int i = 0; i < E; i++) x[i] += ob[i];

        if (ipl) {
            const float *ile = ipl + (size_t)L * ple;
            lgo_matmul_f32(y->inp_gate->data, y->inp_gate->type, E, ple, x, pg);
            for (int i = 0; i < ple; i++) pg[i] = lgo_gelu(pg[i], 0) * ile[i];
            lgo_matmul_f32(y->proj->data, y->proj->type, ple, E, pg, ob);
            lgo_rmsnorm(ob, ob, y->post_norm, E, eps, 0);
            for (int i = 0; i < E; i++) x[i] += ob[i];
        }
        if (y->out_scale) for (int i = 0; i < E; i++) x[i] *= y->out_scale[0];
    }
    int best = -1;
    if (logits || hidden) {
        lgo_rmsnorm(x, x, o->output_norm, E, eps, 0);
        if (hidden) memcpy(hidden, x, (size_t)E * 4);
    }
    if (logits) {
        lgo_matmul_f32(o->token_embd->data, o->token_embd->type, E, c->n_vocab, x, logits);
        if (c->logit_softcap > 0.0f) {
            float sc = c->logit_softcap;
            for (int v = 0; v < c->n_vocab; v++) logits[v] = sc * tanhf(logits[v] / sc);
        }
        best = 0;
        for (int v = 1; v < c->n_vocab; v++) if (logits[v] > logits[best]) best = v;
    }
    free(x); free(h); free(q); free(kb); free(vb); free(xb); free(ob); free(g1); free(g2); free(att); free(pg); free(ipl);
    return best;
}

/* ---- int8 class: the reference's run-cuda-i8 verify row (src/cuda/prefill-kernel.cuh:374-542 layer
 * loop, src/cuda/model-cuda.cuh:1121-1147 PLE build, src/cuda/mtp-kernel.cuh:21-30 head), one row.
 * Every matmul input is quantized once where the reference quantizes it; sums and elementary functions
 * follow this build's definitions when exact = 1. */
struct qact { int8_t *q; float *d; float *f; int noq; };
/* noq: the quantization is switched off and the matmul takes the f32 vector itself (LGO_I8_F32): the same op
 * sequence, norm / attention orders and elementary functions, without the int8 rounding of the activations */
static void quant_into(struct qact *a, const float *x, int n) {
    memcpy(a->f, x, (size_t)n * 4);                          /* (a float-typed weight takes the vector itself) */
    if (!a->noq) lgo_quant_q8(x, n, a->q, a->d, NULL);
}
static int float_typed(uint32_t t) { return t == GGML_TYPE_F32 || t == GGML_TYPE_F16 || t == GGML_TYPE_BF16; }
static void mm(const struct gguf_tensor *w, int k, int mrows, const struct qact *a, float *out) {
    if (w->type != GGML_TYPE_Q4_0 && !float_typed(w->type)) { fprintf(stderr, "oracle: matmul weight %s is %s; the int8 path takes q4_0 and f32/f16/bf16\n", w->name, ggml_type_name(w->type)); abort(); }
    if (a->noq) lgo_matmul_f32(w->data, w->type, k, mrows, a->f, out);
    else if (float_typed(w->type)) lgo_matmul_fw(w->data, w->type, k, mrows, a->f, out);
    else lgo_matmul_q4q8(w->data, k, mrows, a->q, a->d, 1, out, NULL, LGO_ORDER_SEG);
}

static int forward_i8(struct lgo_model *o, struct lgo_kv *kv, int token, int pos, int exact, int noq, float *logits, float *hidden) {
    const struct model *m = &o->m;
    const struct config *c = &m->cfg;
    const int E = c->n_embd, H = c->n_head, ple = c->n_embd_per_layer;
    const float eps = c->rms_eps;
    int maxhd = 0, maxkv = 0;
    for (int L = 0; L < c->n_layer; L++) {
        if (m->head_dim[L] > maxhd) maxhd = m->head_dim[L];
        if (m->n_head_kv[L] * m->head_dim[L] > maxkv) maxkv = m->n_head_kv[L] * m->head_dim[L];
    }
    int widest = E;
    if (c->n_ff > widest) widest = c->n_ff;
    if (H * maxhd > widest) widest = H * maxhd;
    struct qact a = { malloc((size_t)widest), malloc((size_t)widest / 32 * 4), malloc((size_t)widest * 4), noq };
    float *x = dequantize_row(o->token_embd, token, E);
    const float es = sqrtf((float)E);
    for (int i = 0; i < E; i++) x[i] = x[i] * es;
    float *h = malloc((size_t)E * 4), *q = malloc((size_t)H * maxhd * 4), *kb = malloc((size_t)maxkv * 4);
    float *vb = malloc((size_t)maxkv * 4), *xb = malloc((size_t)H * maxhd * 4), *ob = malloc((size_t)E * 4);
    float *g1 = malloc((size_t)c->n_ff * 4), *g2 = malloc((size_t)c->n_ff * 4);
    float *pg = ple > 0 ? malloc((size_t)ple * 4) : NULL, *ipl = NULL;

    if (ple > 0 && o->pte) {
        const int64_t total = (int64_t)ple * c->n_layer;
        float *tok = dequantize_row(o->pte, token, total);
        const float ts = sqrtf((float)ple);
        for (int64_t i = 0; i < total; i++) tok[i] = tok[i] * ts;
        ipl = malloc((size_t)total * 4);
        quant_into(&a, x, E);
        mm(o->pmp, E, (int)total, &a, ipl);
        const float ps = 1.0f / sqrtf((float)E);
        for (int64_t i = 0; i < total; i++) ipl[i] = ipl[i] * ps;
        for (int L = 0; L < c->n_layer; L++) lgo_rmsnorm(ipl + L * ple, ipl + L * ple, o->pl_proj_norm, ple, eps, 1);
        const float r2 = 1.0f / sqrtf(2.0f);
        for (int64_t i = 0; i < total; i++) ipl[i] = (ipl[i] + tok[i]) * r2;
        free(tok);
    }

    for (int L = 0; L < c->n_layer; L++) {
        const struct lgo_layer *y = &o->l[L];
        const int local = m->is_local[L], hd = m->head_dim[L], nkv = m->n_head_kv[L];
        const int qd = H * hd, kd = nkv * hd;
        const float base = local ? c->rope_freq_base_swa : c->rope_freq_base;
        const float *ff = local ? NULL : o->rope_freqs;
        float *tab = local ? o->tab_swa : o->tab_full;
        fill_tab(tab, base, hd);

        lgo_rmsnorm(h, x, y->attn_norm, E, eps, 1);
        quant_into(&a, h, E);
        mm(y->wq, E, qd, &a, q);
        const int src = kv_source(m, L);
        if (L < c->n_kv_start) {
            mm(y->wk, E, kd, &a, kb);
            if (y->wv) mm(y->wv, E, kd, &a, vb);
            else memcpy(vb, kb, (size_t)kd * 4);
        }
        for (int hh = 0; hh < H; hh++) {
            lgo_rmsnorm(q + hh * hd, q + hh * hd, y->q_norm, hd, eps, 1);
            lgo_rope(q + hh * hd, hd, pos, tab, ff, exact);
        }
        if (L < c->n_kv_start) {
            for (int hh = 0; hh < nkv; hh++) {
                lgo_rmsnorm(kb + hh * hd, kb + hh * hd, y->k_norm, hd, eps, 1);
                lgo_rmsnorm(vb + hh * hd, vb + hh * hd, NULL, hd, eps, 1);
                lgo_rope(kb + hh * hd, hd, pos, tab, ff, exact);
            }
            const int row = pos % kv->seq[L];
            if (kv->f16[L]) {
                uint16_t *kr = (uint16_t *)kv->k[L] + (size_t)row * kd, *vr = (uint16_t *)kv->v[L] + (size_t)row * kd;
                for (int i = 0; i < kd; i++) { kr[i] = lg_f32_to_f16(kb[i]); vr[i] = lg_f32_to_f16(vb[i]); }
            } else {                                          /* LGO_I8_F32: the reference's f32 sliding rings */
                memcpy((float *)kv->k[L] + (size_t)row * kd, kb, (size_t)kd * 4);
                memcpy((float *)kv->v[L] + (size_t)row * kd, vb, (size_t)kd * 4);
            }
        }
        const int start = (local && c->sliding_window > 0 && pos - c->sliding_window + 1 > 0) ? pos - c->sliding_window + 1 : 0;
        const int gqa = H / nkv;
        #pragma omp parallel for schedule(static)
        for (int hh = 0; hh < H; hh++)
            attention_tiled(xb + hh * hd, q + hh * hd, kv->k[src], kv->v[src], kv->f16[src], hd, kd, hh / gqa,
                            kv->seq[src], start, pos, exact);
        quant_into(&a, xb, qd);
        mm(y->wo, qd, E, &a, ob);
        lgo_rmsnorm(ob, ob, y->post_attn, E, eps, 1);
        for (int i = 0; i < E; i++) x[i] = x[i] + ob[i];

        const int nff = m->ffn_len[L];
        lgo_rmsnorm(h, x, y->ffn_norm, E, eps, 1);
        quant_into(&a, h, E);
        mm(y->gate, E, nff, &a, g1);
        mm(y->up, E, nff, &a, g2);
        for (int i = 0; i < nff; i++) g1[i] = lgo_gelu(g1[i], exact) * g2[i];
        quant_into(&a, g1, nff);
        mm(y->down, nff, E, &a, ob);
        lgo_rmsnorm(ob, ob, y->post_ffw, E, eps, 1);
        for (int i = 0; i < E; i++) {
            float v = x[i] + ob[i];
            x[i] = (!ipl && y->out_scale) ? v * y->out_scale[0] : v;
        }
        if (ipl) {
            const float *ile = ipl + (size_t)L * ple;
            quant_into(&a, x, E);
            mm(y->inp_gate, E, ple, &a, pg);
            for (int i = 0; i < ple; i++) pg[i] = lgo_gelu(pg[i], exact) * ile[i];
            quant_into(&a, pg, ple);
            mm(y->proj, ple, E, &a, ob);
            lgo_rmsnorm(ob, ob, y->post_norm, E, eps, 1);
            for (int i = 0; i < E; i++) {
                float v = x[i] + ob[i];
                x[i] = y->out_scale ? v * y->out_scale[0] : v;
            }
        }
    }
    int best = -1;
    if (logits || hidden) {
        lgo_rmsnorm(x, x, o->output_norm, E, eps, 1);
        if (hidden) memcpy(hidden, x, (size_t)E * 4);
    }
    if (logits) {
        quant_into(&a, x, E);
        mm(o->token_embd, E, c->n_vocab, &a, logits);
        if (c->logit_softcap > 0.0f) {
            const float sc = c->logit_softcap;
            for (int v = 0; v < c->n_vocab; v++) logits[v] = sc * (exact ? lg_tanhf(logits[v] / sc) : tanhf(logits[v] / sc));
        }
        best = 0;
        for (int v = 1; v < c->n_vocab; v++) if (logits[v] > logits[best]) best = v;
    }
    free(a.q); free(a.d); free(a.f);
    free(x); free(h); free(q); free(kb); free(vb); free(xb); free(ob); free(g1); free(g2); free(pg); free(ipl);
    return best;
}

int lgo_forward(struct lgo_model *o, struct lgo_kv *kv, int token, int pos, int mode, float *logits, float *hidden) {
    if (token < 0 || token >= o->m.cfg.n_vocab || pos < 0 || pos >= kv->max_seq) return -1;
    if ((mode == LGO_REF || mode == LGO_I8_F32) != (kv->mode == LGO_REF || kv->mode == LGO_I8_F32)) { fprintf(stderr, "oracle: kv cache was created for another mode\n"); return -1; }
    float *own = NULL;
    if (!logits) logits = own = malloc((size_t)o->m.cfg.n_vocab * 4);
    int best = mode == LGO_REF ? forward_ref(o, kv, token, pos, logits, hidden)
                               : forward_i8(o, kv, token, pos, mode != LGO_I8_LIBM, mode == LGO_I8_F32, logits, hidden);
    free(own);
    return best;
}

/* prompt positions whose outputs nobody reads: cache writes only, head skipped
 * (src/cpu/model-cpu.c:482-487) */
void lgo_prefill(struct lgo_model *o, struct lgo_kv *kv, const int *tokens, int n, int pos0, int mode) {
    for (int i = 0; i < n; i++) {
        if (mode == LGO_REF) forward_ref(o, kv, tokens[i], pos0 + i, NULL, NULL);
        else forward_i8(o, kv, tokens[i], pos0 + i, mode != LGO_I8_LIBM, mode == LGO_I8_F32, NULL, NULL);
    }
}

/* the verify step as the reference CPU backend runs it: forwards in sequence while the
 * drafts hold (src/cpu/model-cpu.c:51-58); `hidden` ends at the last valid row */
int lgo_forward_spec(struct lgo_model *o, struct lgo_kv *kv, const int *toks, int rows, int pos,
                     int mode, int *out, float *hidden) {
    int j = 0;
    do {
        out[j] = lgo_forward(o, kv, toks[j], pos + j, mode, NULL, hidden);
        j++;
    } while (j < rows && out[j - 1] == toks[j]);
    return j;
}

/* ======================  draft head  ====================================== */
/* The gemma4-assistant network (src/mtp.c).  LGO_REF restates the reference's host draft
 * (src/mtp.c:258-356) in its own order of operations and is pinned by running that file from the
 * reference build (oracle/_ref) on the same GGUFs.  The int8 class is what the device computes:
 * q8 activations at every matmul input, this build's float orders, the cache seen through the
 * tiled attention as a query at pos-1 (src/cuda/mtp-kernel.cuh:170-182).  The reference's device
 * draft (f16 weights, f32 activations, CUDA summation order) cannot run here: PARITY UNPINNED for
 * its last bits, and for the chained draft's post-projection, which has no CPU counterpart. */
struct lgo_mtp_layer {
    const float *attn_norm, *q_norm, *post_attn, *ffn_norm, *post_ffw, *out_scale;
    const struct gguf_tensor *q, *o, *gate, *up, *down;
    int hd, local, src;
};
struct lgo_mtp {
    struct gguf_context *ctx;
    int n_layer, n_inner, n_bb, n_vocab, n_head, n_ff;
    float eps, base_full, base_swa, softcap;
    const struct gguf_tensor *pre, *post, *head;
    const float *out_norm;
    struct lgo_mtp_layer *l;
};

void lgo_mtp_close(struct lgo_mtp *t) {
    if (!t) return;
    free(t->l);
    free_gguf(t->ctx);
    free(t);
}

struct lgo_mtp *lgo_mtp_open(const char *path, const struct lgo_model *target) {
    struct lgo_mtp *t = calloc(1, sizeof *t);
    if (!t) return NULL;
    t->ctx = load_gguf(path);
    if (!t->ctx) { free(t); return NULL; }
    const struct gguf_context *g = t->ctx;
    const char *arch = gguf_get_str(g, "general.architecture", "");
    char key[96];
#define AK(leaf) (snprintf(key, sizeof key, "%s.%s", arch, leaf), key)
    t->n_layer = (int)gguf_get_u32(g, AK("block_count"), 0);
    t->n_inner = (int)gguf_get_u32(g, AK("embedding_length"), 0);
    t->n_bb = (int)gguf_get_u32(g, AK("embedding_length_out"), 0);
    t->n_head = (int)gguf_get_u32(g, AK("attention.head_count"), 0);
    t->n_ff = (int)gguf_get_u32(g, AK("feed_forward_length"), 0);
    t->eps = gguf_get_f32(g, AK("attention.layer_norm_rms_epsilon"), 1e-6f);
    t->base_full = gguf_get_f32(g, AK("rope.freq_base"), 1e6f);
    t->base_swa = gguf_get_f32(g, AK("rope.freq_base_swa"), 1e4f);
    t->softcap = gguf_get_f32(g, AK("final_logit_softcapping"), 0.0f);
#undef AK
    t->pre = gguf_find_tensor(g, "nextn.pre_projection.weight");
    t->post = gguf_find_tensor(g, "nextn.post_projection.weight");
    t->head = gguf_find_tensor(g, "token_embd.weight");
    t->out_norm = f32_tensor(g, "output_norm.weight");
    const struct model *m = &target->m;
    if (!t->n_layer || !t->pre || !t->head || !t->out_norm || t->n_bb != m->cfg.n_embd || m->cfg.n_kv_start < 2) { lgo_mtp_close(t); return NULL; }
    t->n_vocab = (int)t->head->dims[1];
    const int src_full = m->cfg.n_kv_start - 1, src_swa = m->cfg.n_kv_start - 2;      /* src/mtp.c:173-176 */
    t->l = calloc((size_t)t->n_layer, sizeof *t->l);
    for (int L = 0; L < t->n_layer; L++) {
        struct lgo_mtp_layer *b = &t->l[L];
        b->attn_norm = layer_f(g, L, "attn_norm.weight");   b->q_norm = layer_f(g, L, "attn_q_norm.weight");
        b->post_attn = layer_f(g, L, "post_attention_norm.weight"); b->ffn_norm = layer_f(g, L, "ffn_norm.weight");
        b->post_ffw = layer_f(g, L, "post_ffw_norm.weight"); b->out_scale = layer_f(g, L, "layer_output_scale.weight");
        b->q = layer_t(g, L, "attn_q.weight"); b->o = layer_t(g, L, "attn_output.weight");
        b->gate = layer_t(g, L, "ffn_gate.weight"); b->up = layer_t(g, L, "ffn_up.weight"); b->down = layer_t(g, L, "ffn_down.weight");
        if (!b->attn_norm || !b->q_norm || !b->post_attn || !b->ffn_norm || !b->post_ffw || !b->q || !b->o || !b->gate || !b->up || !b->down) { lgo_mtp_close(t); return NULL; }
        b->hd = (int)b->q->dims[1] / t->n_head;
        b->local = b->hd == m->head_dim[src_swa];                                    /* src/mtp.c:196-198 */
        b->src = b->local ? src_swa : src_full;
        if (b->hd != m->head_dim[b->src]) { lgo_mtp_close(t); return NULL; }
    }
    return t;
}

int lgo_mtp_info(const struct lgo_mtp *t, int32_t *out, int cap) {
    int32_t v[] = { t->n_layer, t->n_inner, t->n_bb, t->n_vocab, t->n_head, t->n_ff, t->post != NULL };
    int n = (int)(sizeof v / sizeof v[0]);
    for (int i = 0; i < n && i < cap; i++) out[i] = v[i];
    return n;
}

/* A cache element as the reference's HOST draft reads it (src/mtp.c:96-113): its private f16
 * reader gives f16 subnormals half their value (exponent 127-15+e+1 with e starting at -1 and one
 * further decrement per shift; model-cpu.c:201-210 starts one higher and is exact).  LGO_REF keeps
 * that so that it stays bit-identical with the reference build; the int8 class, like the
 * reference's device draft (__half loads), converts exactly. */
static float kv_elem(const void *base, size_t i, int f16) {
    if (!f16) return ((const float *)base)[i];
    const uint16_t h = ((const uint16_t *)base)[i];
    const float v = lg_f16_to_f32(h);
    return ((h & 0x7C00u) == 0 && (h & 0x03FFu) != 0) ? 0.5f * v : v;
}

/* One draft.  h_prev: n_bb floats (the target's post-norm hidden of the accepted row, or a chained
 * head hidden lifted by lgo_mtp_post).  hidden_out (n_inner, post output norm) and logits
 * (n_vocab) may be NULL.  Returns the first maximum of the soft-capped logits. */
int lgo_mtp_draft(struct lgo_mtp *t, struct lgo_model *target, struct lgo_kv *kv, int token, int pos,
                  const float *h_prev, int mode, float *hidden_out, float *logits_out) {
    const struct model *m = &target->m;
    const struct config *c = &m->cfg;
    const int ni = t->n_inner, nb = t->n_bb, ref = mode == LGO_REF, exact = mode == LGO_I8 || mode == LGO_I8_F32, noq = mode == LGO_I8_F32;
    const float eps = t->eps;
    if (pos < 1 || token < 0 || token >= c->n_vocab) return -1;
    if ((ref || noq) != (kv->mode == LGO_REF || kv->mode == LGO_I8_F32)) { fprintf(stderr, "oracle: kv cache was created for another mode\n"); return -1; }
    int qmax = 0, widest = 2 * nb;
    for (int L = 0; L < t->n_layer; L++) if (t->n_head * t->l[L].hd > qmax) qmax = t->n_head * t->l[L].hd;
    if (qmax > widest) widest = qmax;
    if (t->n_ff > widest) widest = t->n_ff;
    struct qact a = { malloc((size_t)widest), malloc((size_t)widest / 32 * 4), malloc((size_t)widest * 4), noq };
    float *cat = malloc((size_t)2 * nb * 4), *x = malloc((size_t)ni * 4), *h = malloc((size_t)ni * 4);
    float *q = malloc((size_t)qmax * 4), *xb = malloc((size_t)qmax * 4), *o = malloc((size_t)ni * 4);
    float *g1 = malloc((size_t)t->n_ff * 4), *g2 = malloc((size_t)t->n_ff * 4), *att = malloc((size_t)(pos + 1) * 4);
    float *tab = malloc((size_t)qmax * 4), *logits = logits_out ? logits_out : malloc((size_t)t->n_vocab * 4);

    float *erow = dequantize_row(target->token_embd, token, nb);                     /* src/mtp.c:268-276 */
    const float es = sqrtf((float)nb);
    for (int i = 0; i < nb; i++) cat[i] = erow[i] * es;
    free(erow);
    memcpy(cat + nb, h_prev, (size_t)nb * 4);
    if (ref) lgo_matmul_f32(t->pre->data, t->pre->type, 2 * nb, ni, cat, x);
    else { quant_into(&a, cat, 2 * nb); mm(t->pre, 2 * nb, ni, &a, x); }

    for (int L = 0; L < t->n_layer; L++) {
        const struct lgo_mtp_layer *b = &t->l[L];
        const int hd = b->hd, src = b->src, qd = t->n_head * hd;
        const int kd = kv->kv_dim[src], nkv = m->n_head_kv[src], gqa = t->n_head / nkv, seq = kv->seq[src];
        fill_tab(tab, b->local ? t->base_swa : t->base_full, hd);
        lgo_rmsnorm(h, x, b->attn_norm, ni, eps, !ref);
        if (ref) lgo_matmul_f32(b->q->data, b->q->type, ni, qd, h, q);
        else { quant_into(&a, h, ni); mm(b->q, ni, qd, &a, q); }
        for (int hh = 0; hh < t->n_head; hh++) {
            lgo_rmsnorm(q + hh * hd, q + hh * hd, b->q_norm, hd, eps, !ref);
            lgo_rope(q + hh * hd, hd, pos, tab, NULL, exact);
        }
        /* the cache holds positions < pos; sliding blocks see the window back from pos (src/mtp.c:298-302) */
        const int start = (b->local && c->sliding_window > 0 && pos - c->sliding_window + 1 > 0) ? pos - c->sliding_window + 1 : 0;
        if (ref) {
            const void *Kc = kv->k[src], *Vc = kv->v[src];
            const int f16 = kv->f16[src];
            for (int hh = 0; hh < t->n_head; hh++) {
                const float *qh = q + hh * hd;
                const int kvh = hh / gqa;
                for (int p = start; p < pos; p++) {
                    const size_t off = (size_t)(p % seq) * kd + (size_t)kvh * hd;
                    float s = 0.0f;
                    for (int i = 0; i < hd; i++) s += qh[i] * kv_elem(Kc, off + i, f16);
                    att[p] = s;
                }
                {   /* softmax (src/mtp.c:62-68) */
                    float *v = att + start; const int n = pos - start;
                    float mx = v[0];
                    for (int i = 1; i < n; i++) if (v[i] > mx) mx = v[i];
                    float sum = 0.0f;
                    for (int i = 0; i < n; i++) { v[i] = expf(v[i] - mx); sum += v[i]; }
                    for (int i = 0; i < n; i++) v[i] /= sum;
                }
                float *outh = xb + hh * hd;
                for (int i = 0; i < hd; i++) outh[i] = 0.0f;
                for (int p = start; p < pos; p++) {
                    const size_t off = (size_t)(p % seq) * kd + (size_t)kvh * hd;
                    const float w = att[p];
                    for (int i = 0; i < hd; i++) outh[i] += w * kv_elem(Vc, off + i, f16);
                }
            }
        } else {
            /* a query at pos-1 with the window one shorter: keys max(0, pos-window+1) .. pos-1 */
            #pragma omp parallel for schedule(static)
            for (int hh = 0; hh < t->n_head; hh++)
                attention_tiled(xb + hh * hd, q + hh * hd, kv->k[src], kv->v[src], kv->f16[src], hd, kd, hh / gqa, seq, start, pos - 1, exact);
        }
        if (ref) lgo_matmul_f32(b->o->data, b->o->type, qd, ni, xb, o);
        else { quant_into(&a, xb, qd); mm(b->o, qd, ni, &a, o); }
        lgo_rmsnorm(o, o, b->post_attn, ni, eps, !ref);
        for (int i = 0; i < ni; i++) h[i] = x[i] + o[i];

        lgo_rmsnorm(x, h, b->ffn_norm, ni, eps, !ref);
        if (ref) {
            lgo_matmul_f32(b->gate->data, b->gate->type, ni, t->n_ff, x, g1);
            lgo_matmul_f32(b->up->data, b->up->type, ni, t->n_ff, x, g2);
        } else { quant_into(&a, x, ni); mm(b->gate, ni, t->n_ff, &a, g1); mm(b->up, ni, t->n_ff, &a, g2); }
        for (int i = 0; i < t->n_ff; i++) g1[i] = lgo_gelu(g1[i], exact) * g2[i];
        if (ref) lgo_matmul_f32(b->down->data, b->down->type, t->n_ff, ni, g1, o);
        else { quant_into(&a, g1, t->n_ff); mm(b->down, t->n_ff, ni, &a, o); }
        lgo_rmsnorm(o, o, b->post_ffw, ni, eps, !ref);
        if (ref) {
            for (int i = 0; i < ni; i++) x[i] = h[i] + o[i];
            if (b->out_scale) for (int i = 0; i < ni; i++) x[i] *= b->out_scale[0];
        } else {
            for (int i = 0; i < ni; i++) { const float v = h[i] + o[i]; x[i] = b->out_scale ? v * b->out_scale[0] : v; }
        }
    }
    lgo_rmsnorm(x, x, t->out_norm, ni, eps, !ref);
    if (hidden_out) memcpy(hidden_out, x, (size_t)ni * 4);
    if (ref) lgo_matmul_f32(t->head->data, t->head->type, ni, t->n_vocab, x, logits);
    else { quant_into(&a, x, ni); mm(t->head, ni, t->n_vocab, &a, logits); }
    if (t->softcap > 0.0f)
        for (int v = 0; v < t->n_vocab; v++) logits[v] = t->softcap * (exact ? lg_tanhf(logits[v] / t->softcap) : tanhf(logits[v] / t->softcap));
    int best = 0;
    for (int v = 1; v < t->n_vocab; v++) if (logits[v] > logits[best]) best = v;
    if (!logits_out) free(logits);
    free(a.q); free(a.d); free(a.f); free(cat); free(x); free(h); free(q); free(xb); free(o); free(g1); free(g2); free(att); free(tab);
    return best;
}

/* h_prev of a chained draft: post-projection of the head's own post-norm hidden
 * (src/cuda/mtp-kernel.cuh:372-389).  Returns -1 when the file has no post-projection. */
int lgo_mtp_post(struct lgo_mtp *t, const float *hidden, int mode, float *h_out) {
    if (!t->post) return -1;
    if (mode == LGO_REF) { lgo_matmul_f32(t->post->data, t->post->type, t->n_inner, t->n_bb, hidden, h_out); return 0; }
    struct qact a = { malloc((size_t)t->n_inner), malloc((size_t)t->n_inner / 32 * 4), malloc((size_t)t->n_inner * 4), mode == LGO_I8_F32 };
    quant_into(&a, hidden, t->n_inner);
    mm(t->post, t->n_inner, t->n_bb, &a, h_out);
    free(a.q); free(a.d); free(a.f);
    return 0;
}

/* The verify step as the DEVICE runs it: every row goes through the decoder (so the cache rows of
 * rejected drafts are written too), then the accept rule.  Same result as lgo_forward_spec for
 * out[0..adv-1] and adv; differs in what the cache holds at pos+adv .. pos+rows-1 afterwards, which
 * only a chained draft ever reads. */
int lgo_forward_spec_all(struct lgo_model *o, struct lgo_kv *kv, const int *toks, int rows, int pos,
                         int mode, int *out, float *hidden) {
    float *hrow = malloc((size_t)o->m.cfg.n_embd * 4 * (size_t)rows);
    for (int j = 0; j < rows; j++) out[j] = lgo_forward(o, kv, toks[j], pos + j, mode, NULL, hrow + (size_t)j * o->m.cfg.n_embd);
    const int adv = lgo_accept(toks, out, rows);
    if (hidden) memcpy(hidden, hrow + (size_t)(adv - 1) * o->m.cfg.n_embd, (size_t)o->m.cfg.n_embd * 4);
    free(hrow);
    return adv;
}
