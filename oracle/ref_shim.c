/* ref_shim.c — thin ctypes-friendly entry points around the REFERENCE's own CPU backend.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is compiled together with the reference's
 * src/gguf.c, src/quant.c, src/model.c, src/cpu/model-cpu.c and src/mtp.c, taken from where they lie
 * (see Makefile target _ref), into oracle/_ref/libref_n<N>.so; no reference source is copied
 * into this repository.  It supplies the one symbol those files expect from the CLI
 * (model_pick, src/run.c:83) and flattens the structs for Python.
 */
#include <stdlib.h>
#include <string.h>
#include "model.h"
#include "quant.h"
#include "mtp-internal.h"

int (*model_pick)(const float *logits, int n) = NULL;

struct ref_handle { struct gguf_context *ctx; struct model m; };

struct ref_handle *ref_open(const char *path) {
    struct ref_handle *h = calloc(1, sizeof *h);
    if (!h) return NULL;
    h->ctx = load_gguf(path);
    if (!h->ctx || model_init(&h->m, h->ctx) != 0) { free_gguf(h->ctx); free(h); return NULL; }
    return h;
}
void ref_close(struct ref_handle *h) { if (h) { model_free(&h->m); free_gguf(h->ctx); free(h); } }
int ref_mtp_n(void) { return LG_MTP_N; }
int ref_n_vocab(struct ref_handle *h) { return h->m.cfg.n_vocab; }
int ref_n_embd(struct ref_handle *h) { return h->m.cfg.n_embd; }
int ref_n_layer(struct ref_handle *h) { return h->m.cfg.n_layer; }
void ref_config(struct ref_handle *h, struct config *out) { *out = h->m.cfg; }
void ref_layer_info(struct ref_handle *h, int L, int *out4) {
    out4[0] = h->m.is_local[L]; out4[1] = h->m.head_dim[L]; out4[2] = h->m.n_head_kv[L]; out4[3] = h->m.ffn_len[L];
}

struct kvcache *ref_kv_new(struct ref_handle *h, int max_seq) {
    struct kvcache *kv = calloc(1, sizeof *kv);
    if (kv && kvcache_init(kv, &h->m, max_seq) != 0) { kvcache_free(kv); free(kv); return NULL; }
    return kv;
}
void ref_kv_free(struct kvcache *kv) { if (kv) { kvcache_free(kv); free(kv); } }
void *ref_kv_layer(struct kvcache *kv, int L, int which, int *rows, int *width, int *is_f16) {
    *rows = kv->seq[L]; *width = kv->kv_dim[L]; *is_f16 = kv->f16[L];
    return which ? kv->v[L] : kv->k[L];
}

void ref_forward(struct ref_handle *h, struct kvcache *kv, int token, int pos, float *logits) {
    model_forward(&h->m, kv, token, pos, logits);
}
int ref_forward_next(struct ref_handle *h, struct kvcache *kv, int token, int pos) {
    return model_forward_next(&h->m, kv, token, pos);
}
void ref_prefill(struct ref_handle *h, struct kvcache *kv, const int *tokens, int n, int pos0) {
    model_prefill(&h->m, kv, tokens, n, pos0);
}
int ref_forward_spec(struct ref_handle *h, struct kvcache *kv, const int *toks, int pos, int *out) {
    return model_forward_spec(&h->m, kv, toks, pos, out);
}
void ref_last_hidden(struct ref_handle *h, float *out) { memcpy(out, h->m.last_hidden, (size_t)h->m.cfg.n_embd * 4); }
int ref_dequantize(unsigned type, const void *src, float *out, long long n) { return dequantize_into(type, src, out, n) ? 0 : -1; }

/* the reference's host draft (src/mtp.c:258-356): it reads m.last_hidden, which the forwards above keep */
struct mtp *ref_mtp_open(struct ref_handle *h, const char *path) { return mtp_open(path, &h->m); }
void ref_mtp_free(struct mtp *t) { mtp_free(t); }
int  ref_mtp_draft(struct ref_handle *h, struct mtp *t, struct kvcache *kv, int token, int pos) { return mtp_draft(t, &h->m, kv, token, pos); }
int  ref_mtp_n_vocab(struct mtp *t) { return t->n_vocab; }
int  ref_mtp_n_inner(struct mtp *t) { return t->n_inner; }
void ref_mtp_logits(struct mtp *t, float *out) { memcpy(out, t->logits, (size_t)t->n_vocab * 4); }
void ref_mtp_hidden(struct mtp *t, float *out) { memcpy(out, t->x, (size_t)t->n_inner * 4); }
