/* model.h — the backend seam of the verify path.
 *
 * Same structs, field order and function signatures as the reference's
 * include/model.h:10-190, so that model-hip.c (this directory) is a third
 * interchangeable backend beside src/cpu/model-cpu.c and src/cuda/model-cuda-i8.cu:
 * the choice is made at link time (CMakeLists.txt:42-45,77-78).  What each
 * function must do is stated in model-hip.c next to its implementation.
 */
#ifndef MODEL_H
#define MODEL_H

#include "gguf.h"

struct config {
    char  arch[32];
    int   n_layer;
    int   n_embd;
    int   n_head;
    int   n_head_kv;
    int   head_dim_swa;        /* head size on sliding-window layers */
    int   head_dim_full;       /* head size on global layers */
    int   n_ff;                /* widest feed-forward layer */
    int   n_vocab;             /* length of tokenizer.ggml.tokens */
    int   n_ctx;
    int   sliding_window;
    int   n_embd_per_layer;    /* per-layer-embedding (PLE) width, 0 = none */
    int   n_kv_start;          /* layers >= this read an earlier layer's KV */
    float rms_eps;
    float rope_freq_base;
    float rope_freq_base_swa;
    float logit_softcap;       /* 0 = none */
};

int  config_load(struct config *c, const struct gguf_context *ctx);
void config_print(const struct config *c);

struct model {
    struct config              cfg;
    const struct gguf_context *ctx;        /* borrowed */
    int                       *is_local;   /* per layer: sliding-window attention */
    int                       *ffn_len;    /* per layer: feed-forward width */
    int                       *head_dim;   /* per layer */
    int                       *n_head_kv;  /* per layer */
    float                     *last_hidden; /* [n_embd] post-output-norm hidden of the last logits row */
};

int  model_init(struct model *m, const struct gguf_context *ctx);
void model_free(struct model *m);

/* Per owning layer: seq[L] rows of kv_dim[L] values; position p lives in row
 * p % seq[L] (identity on global layers).  Sharing layers hold NULL. */
struct kvcache {
    int     n_layer;
    int     max_seq;
    int    *kv_dim;
    int    *seq;
    int    *f16;
    void  **k;
    void  **v;
    void  **px_k;
    void  **px_v;
};

int  kvcache_init(struct kvcache *kv, const struct model *m, int max_seq);
void kvcache_free(struct kvcache *kv);
void kvcache_save_prefix(struct kvcache *kv, int n);
void kvcache_restore_prefix(struct kvcache *kv, int n);

void model_forward(struct model *m, struct kvcache *kv, int token, int pos, float *logits);
int  model_forward_next(struct model *m, struct kvcache *kv, int token, int pos);
extern int (*model_pick)(const float *logits, int n);
void model_prefill(struct model *m, struct kvcache *kv, const int *tokens, int n, int pos0);
void model_prefill_embd(struct model *m, struct kvcache *kv, const float *rows, int n, int pos0);
void model_prefill_mixed(struct model *m, struct kvcache *kv, const float *rows,
                         const int *ids, int n, int pos0);
void model_prefill_reserve(void);

#ifndef LG_MTP_N
#define LG_MTP_N 3
#endif

struct mtp;
struct mtp *mtp_open(const char *path, const struct model *m);
void        mtp_free(struct mtp *t);
int mtp_draft(struct mtp *t, const struct model *m, const struct kvcache *kv, int token, int pos);
int mtp_draft_chain(struct mtp *t, const struct model *m, const struct kvcache *kv, int token, int pos);

/* toks[0] = chosen token at pos, toks[1..] drafts; out[j] = greedy successor of
 * toks[j]; returns how many positions advanced (1..LG_MTP_N). */
int model_forward_spec(struct model *m, struct kvcache *kv, const int *toks, int pos, int *out);

extern const int model_kv_host;

#endif
