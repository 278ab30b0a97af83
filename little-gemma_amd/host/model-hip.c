/* model-hip.c — the reference's backend interface (model.h) on the gfx950 library.
 *
 * A third interchangeable backend beside the reference's src/cpu/model-cpu.c and
 * src/cuda/model-cuda-i8.cu: it defines every symbol a backend translation unit must define
 * (include/model.h:79-190 and src/mtp-internal.h:33-37 of the reference) and is selected by
 * linking it instead of them.  All compute happens behind the C ABI of include/lg_hip.h; this
 * file only walks the GGUF tensors, keeps the handles and converts error codes into the
 * reference's behaviour (print and exit(1), like CUDA_CHECK, src/cuda/model-cuda.cuh:34-36).
 * It compiles against this directory's model.h and, unchanged, against the reference's headers.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "model.h"
#include "mtp-internal.h"
#include "lg_hip.h"

const int model_kv_host = 0;          /* cache rows live on the device */

/* one model per process, like the reference's file-static device state
 * (src/cuda/model-cuda.cuh:724-726) */
static lg_hip_model *g_dev;
static const struct model *g_owner;
static const void *g_owner_ctx;       /* the file the weights came from: a new model at a reused address is a new model */
static int g_live;                    /* caches and draft heads that hold pointers into g_dev */
static int g_logits_on;

static void die(const char *what) {
    fprintf(stderr, "run-hip: %s: %s\n", what, lg_hip_last_error());
    exit(1);
}

/* Weights go up on first use (the reference's ensure_weights, src/cuda/model-cuda.cuh:738-799). */
static lg_hip_model *device_model(const struct model *m) {
    if (g_dev && g_owner == m && g_owner_ctx == (const void *)m->ctx) return g_dev;
    if (g_dev) {
        if (g_live > 0) {
            fprintf(stderr, "run-hip: one model per process: %d cache(s) / draft head(s) of the previous model are still alive\n", g_live);
            exit(1);
        }
        lg_hip_model_destroy(g_dev); g_dev = NULL;
    }
    const struct config *c = &m->cfg;
    struct lg_hip_config hc = {
        .n_layer = c->n_layer, .n_embd = c->n_embd, .n_head = c->n_head, .n_vocab = c->n_vocab,
        .sliding_window = c->sliding_window, .n_embd_per_layer = c->n_embd_per_layer, .n_kv_start = c->n_kv_start,
        .rms_eps = c->rms_eps, .rope_freq_base = c->rope_freq_base, .rope_freq_base_swa = c->rope_freq_base_swa,
        .logit_softcap = c->logit_softcap,
        .is_local = m->is_local, .ffn_len = m->ffn_len, .head_dim = m->head_dim, .n_head_kv = m->n_head_kv,
    };
    const char *dev = getenv("LG_HIP_DEVICE");
    if (lg_hip_model_create(&hc, dev ? atoi(dev) : 0, &g_dev) != 0) die("model_create");
    const struct gguf_context *g = m->ctx;
    for (uint64_t i = 0; i < g->header.num_tensors; i++) {
        const struct gguf_tensor *t = &g->tensors[i];
        if (lg_hip_model_tensor(g_dev, t->name, t->type, t->n_dims, t->dims, t->data) < 0) die(t->name);
    }
    int rows = LG_MTP_N > LG_HIP_MAX_ROWS ? LG_HIP_MAX_ROWS : LG_MTP_N;
    const char *wide = getenv("LG_HIP_MAX_ROWS");        /* prefill uses the widest block the model was committed for */
    if (wide && atoi(wide) > rows) rows = atoi(wide);
    if (rows > LG_HIP_MAX_ROWS) rows = LG_HIP_MAX_ROWS;
    if (LG_MTP_N > LG_HIP_MAX_ROWS) { fprintf(stderr, "run-hip: LG_MTP_N=%d exceeds the %d rows the kernels are built for\n", LG_MTP_N, LG_HIP_MAX_ROWS); exit(1); }
    if (lg_hip_model_commit(g_dev, rows) != 0) die("model_commit");
    g_owner = m; g_owner_ctx = (const void *)m->ctx;
    g_logits_on = 0;
    return g_dev;
}

static lg_hip_kv *device_kv(const struct kvcache *kv) { return kv && kv->k ? (lg_hip_kv *)kv->k[0] : NULL; }

/* kvcache_init (include/model.h:79): per-layer geometry is mirrored into the public struct;
 * k[L]/v[L] of an owning layer hold the opaque device handle (layer 0 always owns), NULL marks
 * a sharing layer exactly as in the reference. */
int kvcache_init(struct kvcache *kv, const struct model *m, int max_seq) {
    lg_hip_model *d = device_model(m);
    const int nl = m->cfg.n_layer;
    memset(kv, 0, sizeof *kv);
    kv->n_layer = nl; kv->max_seq = max_seq;
    kv->kv_dim = calloc((size_t)nl, sizeof(int));
    kv->seq = calloc((size_t)nl, sizeof(int));
    kv->f16 = calloc((size_t)nl, sizeof(int));
    kv->k = calloc((size_t)nl, sizeof(void *));
    kv->v = calloc((size_t)nl, sizeof(void *));
    if (!kv->kv_dim || !kv->seq || !kv->f16 || !kv->k || !kv->v) return -1;
    lg_hip_kv *h = NULL;
    if (lg_hip_kv_create(d, max_seq, &h) != 0) die("kv_create");
    g_live++;
    for (int L = 0; L < nl; L++) {
        int rows = 0, width = 0;
        lg_hip_kv_layout(h, L, &rows, &width);
        kv->kv_dim[L] = m->n_head_kv[L] * m->head_dim[L];
        kv->seq[L] = rows;
        kv->f16[L] = rows > 0;
        if (rows > 0) { kv->k[L] = h; kv->v[L] = h; }
    }
    return 0;
}

void kvcache_free(struct kvcache *kv) {
    if (!kv) return;
    if (device_kv(kv)) { lg_hip_kv_destroy(device_kv(kv)); if (g_live > 0) g_live--; }
    free(kv->k); free(kv->v); free(kv->kv_dim); free(kv->seq); free(kv->f16);
    memset(kv, 0, sizeof *kv);
}

void kvcache_save_prefix(struct kvcache *kv, int n)    { if (lg_hip_kv_save_prefix(device_kv(kv), n) != 0) die("kv_save_prefix"); }
void kvcache_restore_prefix(struct kvcache *kv, int n) { if (lg_hip_kv_restore_prefix(device_kv(kv), n) != 0) die("kv_restore_prefix"); }

static void want_logits(lg_hip_model *d, int on) {
    if (g_logits_on == on) return;
    lg_hip_set_option(d, "store_logits", on);
    g_logits_on = on;
}

/* The block form with a run-time width; model_forward_spec below pins it to LG_MTP_N. */
int lg_model_forward_spec_n(struct model *m, struct kvcache *kv, const int *toks, int rows, int pos, int *out) {
    lg_hip_model *d = device_model(m);
    int adv = 0;
    want_logits(d, model_pick != NULL);
    if (lg_hip_forward_spec(d, device_kv(kv), toks, rows, pos, out, &adv) != 0) die("forward_spec");
    if (model_pick) {
        /* sampling hook: pick from every row's logits, accept while the pick agrees
         * (src/cuda/mtp-kernel.cuh:103-116) */
        float *row = malloc((size_t)m->cfg.n_vocab * sizeof(float));
        if (!row) { fprintf(stderr, "run-hip: out of memory\n"); exit(1); }
        for (int j = 0; j < rows; j++) {
            if (lg_hip_get_logits(d, j, row) != 0) die("get_logits");
            out[j] = model_pick(row, m->cfg.n_vocab);
        }
        free(row);
        adv = 1;
        while (adv < rows && out[adv - 1] == toks[adv]) adv++;
        if (lg_hip_set_hidden_row(d, adv - 1) != 0) die("set_hidden_row");
    }
    return adv;
}

int model_forward_spec(struct model *m, struct kvcache *kv, const int *toks, int pos, int *out) {
    return lg_model_forward_spec_n(m, kv, toks, LG_MTP_N, pos, out);
}

/* model_forward_next (include/model.h:103): the one-row block; the argmax stays on the device. */
int model_forward_next(struct model *m, struct kvcache *kv, int token, int pos) {
    int out = -1;
    lg_model_forward_spec_n(m, kv, &token, 1, pos, &out);
    return out;
}

/* model_forward (include/model.h:98): one row with the logits copied back; logits == NULL is
 * the cache-write-only form the reference uses for prompt tokens (src/cpu/model-cpu.c:482-487). */
void model_forward(struct model *m, struct kvcache *kv, int token, int pos, float *logits) {
    lg_hip_model *d = device_model(m);
    if (!logits) { if (lg_hip_prefill(d, device_kv(kv), &token, 1, pos) != 0) die("prefill"); return; }
    int out, adv;
    want_logits(d, 1);
    if (lg_hip_forward_spec(d, device_kv(kv), &token, 1, pos, &out, &adv) != 0) die("forward");
    if (lg_hip_get_logits(d, 0, logits) != 0) die("get_logits");
    if (m->last_hidden && lg_hip_get_hidden(d, m->last_hidden) != 0) die("get_hidden");
}

void model_prefill(struct model *m, struct kvcache *kv, const int *tokens, int n, int pos0) {
    if (lg_hip_prefill(device_model(m), device_kv(kv), tokens, n, pos0) != 0) die("prefill");
}

/* Media spans are outside this backend: it serves token ids only. */
void model_prefill_embd(struct model *m, struct kvcache *kv, const float *rows, int n, int pos0) {
    (void)m; (void)kv; (void)rows; (void)n; (void)pos0;
    fprintf(stderr, "run-hip: embedding-row prefill (media) is not supported by this backend\n");
    exit(1);
}
void model_prefill_mixed(struct model *m, struct kvcache *kv, const float *rows, const int *ids, int n, int pos0) {
    for (int i = 0; i < n; i++) if (ids[i] < 0) model_prefill_embd(m, kv, rows, n, pos0);
    model_prefill(m, kv, ids, n, pos0);
}
void model_prefill_reserve(void) { }

/* Post-norm hidden of the last valid verify row, for a draft head (src/cuda/mtp-kernel.cuh:117-118). */
int lg_model_last_hidden(struct model *m, float *dst) { return lg_hip_get_hidden(device_model(m), dst); }
lg_hip_model *lg_model_device(struct model *m) { return device_model(m); }
lg_hip_kv    *lg_model_device_kv(struct kvcache *kv) { return device_kv(kv); }
void lg_model_release(void) { if (g_dev) { lg_hip_model_destroy(g_dev); g_dev = NULL; g_owner = NULL; g_owner_ctx = NULL; g_live = 0; } }

/* ---- draft head on the device (src/cuda/mtp-kernel.cuh:272-402) --------------------------------
 * First use uploads the head (mtp_cuda_init there); a failure disables drafting for the process
 * ((void *)-1), and the caller pads the block (src/run.c:58-63). */
static lg_hip_model *draft_model(struct mtp *t, const struct model *m) {
    if (t->cuda == (void *)-1) return NULL;
    if (t->cuda) return (lg_hip_model *)t->cuda;
    lg_hip_model *target = device_model(m), *d = NULL;
    int32_t *geo = malloc((size_t)t->n_layer * 4 * sizeof *geo);
    if (!geo) { t->cuda = (void *)-1; return NULL; }
    int32_t *is_local = geo, *ffn = geo + t->n_layer, *hd = geo + 2 * t->n_layer, *nkv = geo + 3 * t->n_layer;
    for (int L = 0; L < t->n_layer; L++) {
        is_local[L] = m->is_local[t->l[L].src]; ffn[L] = t->n_ff; hd[L] = t->l[L].hd; nkv[L] = m->n_head_kv[t->l[L].src];
    }
    struct lg_hip_config hc = {
        .n_layer = t->n_layer, .n_embd = t->n_inner, .n_head = t->n_head, .n_vocab = t->n_vocab,
        .sliding_window = m->cfg.sliding_window, .n_embd_per_layer = 0, .n_kv_start = 0,
        .rms_eps = t->eps, .rope_freq_base = t->base_full, .rope_freq_base_swa = t->base_swa, .logit_softcap = t->softcap,
        .is_local = is_local, .ffn_len = ffn, .head_dim = hd, .n_head_kv = nkv,
    };
    int ok = lg_hip_draft_create(target, &hc, &d) == 0;
    free(geo);
    const struct gguf_context *g = t->ctx;
    for (uint64_t i = 0; ok && i < g->header.num_tensors; i++) {
        const struct gguf_tensor *w = &g->tensors[i];
        const char *name = w == t->pre ? "pre_projection.weight" : w == t->post ? "post_projection.weight" : w->name;
        ok = lg_hip_model_tensor(d, name, w->type, w->n_dims, w->dims, w->data) >= 0;
    }
    ok = ok && lg_hip_model_commit(d, 1) == 0;
    if (!ok) {
        fprintf(stderr, "mtp: device upload failed, drafting disabled: %s\n", lg_hip_last_error());
        if (d) lg_hip_model_destroy(d);
        t->cuda = (void *)-1;
        return NULL;
    }
    t->cuda = d;
    g_live++;
    return d;
}
static int draft_on_device(struct mtp *t, const struct model *m, const struct kvcache *kv, int token, int pos, int chain) {
    lg_hip_model *d = draft_model(t, m);
    int32_t tok = -1;
    if (!d) return -1;
    if (lg_hip_draft_step(d, device_kv(kv), token, pos, chain, &tok) != 0) {
        if (chain) return -1;                      /* e.g. no post-projection: the caller pads */
        die("draft_step");
    }
    return tok;
}
int  mtp_draft_device(struct mtp *t, const struct model *m, const struct kvcache *kv, int token, int pos) {
    return draft_on_device(t, m, kv, token, pos, 0);
}
int  mtp_draft_chain_device(struct mtp *t, const struct model *m, const struct kvcache *kv, int token, int pos) {
    return draft_on_device(t, m, kv, token, pos, 1);
}
/* n_rounds speculative rounds with no host round trip in between (draft, chained drafts, verify, accept, next
 * chosen token: the body of the reference's loop, src/run.c:54-71 and :559-574, kept on the device).  Returns 0,
 * or -1 when the head is unavailable or cannot chain: the caller then drives the loop itself. */
int lg_model_mtp_rounds(struct mtp *t, const struct model *m, struct kvcache *kv, int token, int pos, int rows,
                        int n_rounds, int *blocks, int *out, int *adv) {
    lg_hip_model *d = draft_model(t, m);
    if (!d) return -1;
    int rc = lg_hip_mtp_rounds(d, device_kv(kv), token, pos, rows, n_rounds, blocks, out, adv, NULL);
    if (rc == -4) return -1;                       /* no post-projection */
    if (rc != 0) die("mtp_rounds");
    return 0;
}
void mtp_free_device(struct mtp *t) {
    if (t->cuda && t->cuda != (void *)-1) { lg_hip_model_destroy((lg_hip_model *)t->cuda); if (g_live > 0) g_live--; }
    t->cuda = NULL;
}
/* the head's device handle, for callers that read its hidden state or logits */
lg_hip_model *lg_mtp_device(struct mtp *t, const struct model *m) { return draft_model(t, m); }
