/* model.c — hyper-parameters and per-layer geometry out of GGUF metadata.
 *
 * Restates the reference's src/model.c:67-210: same keys, same defaults, same
 * derivations (head size from the attn_q tensor shape, kv-head count from
 * attn_k, kv-sharing layers inheriting their source layer's geometry), so a
 * file that loads there loads here with identical numbers.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "model.h"

static const struct gguf_meta *arch_meta(const struct gguf_context *g, const char *arch, const char *leaf) {
    char key[160];
    snprintf(key, sizeof key, "%s.%s", arch, leaf);
    return gguf_find_meta(g, key);
}
static int is_i32_array(const struct gguf_meta *m) {
    return m && m->type == GGUF_TYPE_ARRAY && m->value.arr.type == GGUF_TYPE_INT32;
}
static uint32_t arch_u32(const struct gguf_context *g, const char *arch, const char *leaf, uint32_t fb) {
    char key[160];
    snprintf(key, sizeof key, "%s.%s", arch, leaf);
    return gguf_get_u32(g, key, fb);
}
static float arch_f32(const struct gguf_context *g, const char *arch, const char *leaf, float fb) {
    char key[160];
    snprintf(key, sizeof key, "%s.%s", arch, leaf);
    return gguf_get_f32(g, key, fb);
}
/* scalar, or element 0 of a per-layer i32 array (src/model.c:45-54) */
static int arch_first(const struct gguf_context *g, const char *arch, const char *leaf, int fb) {
    const struct gguf_meta *m = arch_meta(g, arch, leaf);
    if (is_i32_array(m) && m->value.arr.n > 0) return ((const int32_t *)m->value.arr.data)[0];
    return (int)arch_u32(g, arch, leaf, (uint32_t)fb);
}

int config_load(struct config *c, const struct gguf_context *g) {
    memset(c, 0, sizeof *c);
    const char *arch = gguf_get_str(g, "general.architecture", "");
    snprintf(c->arch, sizeof c->arch, "%s", arch);
    if (!arch[0]) { fprintf(stderr, "config: missing general.architecture\n"); return -1; }

    c->n_layer   = (int)arch_u32(g, arch, "block_count", 0);
    c->n_embd    = (int)arch_u32(g, arch, "embedding_length", 0);
    c->n_head    = arch_first(g, arch, "attention.head_count", 0);
    c->n_head_kv = arch_first(g, arch, "attention.head_count_kv", c->n_head);

    /* widest layer when feed_forward_length is a per-layer array (src/model.c:28-41) */
    const struct gguf_meta *ff = arch_meta(g, arch, "feed_forward_length");
    if (is_i32_array(ff) && ff->value.arr.n > 0) {
        const int32_t *a = ff->value.arr.data;
        for (uint64_t i = 0; i < ff->value.arr.n; i++) if (a[i] > c->n_ff) c->n_ff = a[i];
    } else c->n_ff = (int)arch_u32(g, arch, "feed_forward_length", 0);

    c->n_ctx              = (int)arch_u32(g, arch, "context_length", 0);
    c->sliding_window     = (int)arch_u32(g, arch, "attention.sliding_window", 0);
    c->n_embd_per_layer   = (int)arch_u32(g, arch, "embedding_length_per_layer_input", 0);
    c->rms_eps            = arch_f32(g, arch, "attention.layer_norm_rms_epsilon", 1e-5f);
    c->rope_freq_base     = arch_f32(g, arch, "rope.freq_base", 10000.0f);
    c->rope_freq_base_swa = arch_f32(g, arch, "rope.freq_base_swa", c->rope_freq_base);
    c->logit_softcap      = arch_f32(g, arch, "final_logit_softcapping", 0.0f);
    c->head_dim_full      = (int)arch_u32(g, arch, "attention.key_length", 0);
    c->head_dim_swa       = (int)arch_u32(g, arch, "attention.key_length_swa", (uint32_t)c->head_dim_full);

    int shared = (int)arch_u32(g, arch, "attention.shared_kv_layers", 0);
    c->n_kv_start = shared > 0 ? c->n_layer - shared : c->n_layer;

    const struct gguf_meta *tok = gguf_find_meta(g, "tokenizer.ggml.tokens");
    if (tok && tok->type == GGUF_TYPE_ARRAY) c->n_vocab = (int)tok->value.arr.n;

    if (c->n_layer <= 0 || c->n_layer > 4096) {
        fprintf(stderr, "config: %s.block_count is %d - missing or not a plausible layer count\n", arch, c->n_layer);
        return -1;
    }
    return 0;
}

void config_print(const struct config *c) {
    printf("config %s: layers %d, embd %d, heads %d/%d kv, head_dim swa %d full %d, ff %d, vocab %d, ctx %d\n"
           "  window %d, ple %d, kv_start %d, eps %g, rope base %g (swa %g), softcap %g\n",
           c->arch, c->n_layer, c->n_embd, c->n_head, c->n_head_kv, c->head_dim_swa, c->head_dim_full,
           c->n_ff, c->n_vocab, c->n_ctx, c->sliding_window, c->n_embd_per_layer, c->n_kv_start,
           c->rms_eps, c->rope_freq_base, c->rope_freq_base_swa, c->logit_softcap);
}

static const struct gguf_tensor *layer_tensor(const struct gguf_context *g, int L, const char *leaf) {
    char name[96];
    snprintf(name, sizeof name, "blk.%d.%s", L, leaf);
    return gguf_find_tensor(g, name);
}

int model_init(struct model *m, const struct gguf_context *g) {
    memset(m, 0, sizeof *m);
    if (config_load(&m->cfg, g) != 0) return -1;
    m->ctx = g;
    const struct config *c = &m->cfg;
    const size_t nl = (size_t)(unsigned)c->n_layer;
    m->ffn_len = calloc(nl, sizeof(int));
    m->is_local = calloc(nl, sizeof(int));
    m->head_dim = calloc(nl, sizeof(int));
    m->n_head_kv = calloc(nl, sizeof(int));
    m->last_hidden = calloc((size_t)(c->n_embd > 0 ? c->n_embd : 1), sizeof(float));
    if (!m->ffn_len || !m->is_local || !m->head_dim || !m->n_head_kv || !m->last_hidden) return -1;

    const struct gguf_meta *ff = arch_meta(g, c->arch, "feed_forward_length");
    const struct gguf_meta *pat = arch_meta(g, c->arch, "attention.sliding_window_pattern");
    const int pat_ok = pat && pat->type == GGUF_TYPE_ARRAY && pat->value.arr.type == GGUF_TYPE_BOOL;
    for (int L = 0; L < c->n_layer; L++) {
        m->ffn_len[L] = (is_i32_array(ff) && (uint64_t)L < ff->value.arr.n)
                      ? ((const int32_t *)ff->value.arr.data)[L] : c->n_ff;
        if (pat_ok && (uint64_t)L < pat->value.arr.n) m->is_local[L] = ((const int8_t *)pat->value.arr.data)[L] != 0;
    }
    for (int L = 0; L < c->n_layer; L++) {
        const struct gguf_tensor *q = layer_tensor(g, L, "attn_q.weight");
        const struct gguf_tensor *k = layer_tensor(g, L, "attn_k.weight");
        if (!q || c->n_head == 0 || (!k && L < c->n_kv_start)) {
            fprintf(stderr, "model: missing attn_q/attn_k for layer %d\n", L);
            return -1;
        }
        m->head_dim[L] = (int)(q->dims[1] / (uint64_t)c->n_head);
        if (k) m->n_head_kv[L] = (int)(k->dims[1] / (uint64_t)m->head_dim[L]);
        else   m->n_head_kv[L] = m->n_head_kv[c->n_kv_start - (m->is_local[L] ? 2 : 1)];
    }
    return 0;
}

void model_free(struct model *m) {
    if (!m) return;
    free(m->is_local); free(m->ffn_len); free(m->head_dim); free(m->n_head_kv); free(m->last_hidden);
    m->is_local = m->ffn_len = m->head_dim = m->n_head_kv = NULL;
    m->last_hidden = NULL;
}
