/* mtp-internal.h — the draft head as the backends see it.
 *
 * Same names and meaning as the reference's src/mtp-internal.h:11-37 (struct mtp_layer,
 * struct mtp, the three device entry points) so that model-hip.c compiles unchanged against
 * either header.  The host-draft scratch buffers of the reference's struct are not kept here:
 * this backend's cache lives on the device and every draft runs there; `cuda` holds the
 * backend's device state.
 */
#ifndef MTP_INTERNAL_H
#define MTP_INTERNAL_H

#include "gguf.h"
#include "model.h"

struct mtp_layer {
    const float *attn_norm, *q_norm, *post_attn, *ffn_norm, *post_ffw;
    const float *out_scale;                  /* scalar, may be NULL */
    const struct gguf_tensor *q, *o, *gate, *up, *down;
    int hd;            /* q head size = head size of the target cache layer it reads */
    int local;         /* 1: reads the target's sliding cache, 0: the global one */
    int src;           /* target layer whose cache the block attends */
};

struct mtp {
    struct gguf_context *ctx;
    int n_layer, n_inner, n_bb, n_vocab, n_head, n_ff;
    float eps, base_full, base_swa, softcap;
    const struct gguf_tensor *pre, *post, *head;
    const float *out_norm;
    struct mtp_layer *l;
    void *cuda;        /* device state of the backend, NULL before the first draft, (void *)-1 = unavailable */
};

int  mtp_draft_device(struct mtp *t, const struct model *m, const struct kvcache *kv, int token, int pos);
int  mtp_draft_chain_device(struct mtp *t, const struct model *m, const struct kvcache *kv, int token, int pos);
void mtp_free_device(struct mtp *t);

#endif
