/* session.h — one loaded model + one KV cache behind plain function calls.
 *
 * What the reference's generate() does around the backend seam (src/run.c:711-745: load,
 * model_init, kvcache_init, prefill, decode) for callers that hold token ids instead of text:
 * run-hip's command line and the Python tests.  Everything goes through model.h.
 */
#ifndef LG_SESSION_H
#define LG_SESSION_H
#include "model.h"

struct lg_session;
struct lg_session *lg_session_open(const char *gguf_path);
void lg_session_close(struct lg_session *s);
int  lg_session_kv(struct lg_session *s, int max_seq);              /* (re)creates the cache */
struct model   *lg_session_model(struct lg_session *s);
struct kvcache *lg_session_kvcache(struct lg_session *s);
/* n_layer, n_embd, n_head, n_vocab, ple, n_kv_start, window, n_ff, n_head_kv, head_dim_swa, head_dim_full, n_ctx */
int  lg_session_info(struct lg_session *s, int *out, int cap);
/* is_local, head_dim, n_head_kv, ffn_len of layer L */
int  lg_session_layer(struct lg_session *s, int L, int *out4);
void lg_session_prefill(struct lg_session *s, const int *tokens, int n, int pos0);
int  lg_session_forward_next(struct lg_session *s, int token, int pos);
void lg_session_forward(struct lg_session *s, int token, int pos, float *logits);
int  lg_session_forward_spec(struct lg_session *s, const int *toks, int rows, int pos, int *out);
/* Greedy generation of n_gen tokens after `prompt`, plain (rows = 1) or speculative with draft
 * blocks of `rows` tokens taken from `drafts` (what a draft head would propose for each emitted
 * position; NULL = repeat the last token, the reference's padding, src/run.c:58-63).
 * Returns tokens emitted; *steps = target forwards/verify steps run. */
int  lg_session_generate(struct lg_session *s, const int *prompt, int n_prompt, int n_gen, int rows,
                         const int *drafts, int *emitted, int *steps);
/* Draft head (include/model.h:156-178): open a gemma4-assistant file for this session's model,
 * one draft (chain = 0: from the target's hidden; 1: chained on the head's own), the head's
 * post-norm hidden, its logits (dst NULL: switch storing on/off), and the reference's
 * speculative loop with the head proposing every block. */
struct mtp *lg_session_mtp_open(struct lg_session *s, const char *path);
void lg_session_mtp_close(struct mtp *t);
int  lg_session_mtp_draft(struct lg_session *s, struct mtp *t, int token, int pos, int chain);
int  lg_session_mtp_hidden(struct lg_session *s, struct mtp *t, float *dst);
int  lg_session_mtp_logits(struct lg_session *s, struct mtp *t, int on, float *dst);
int  lg_session_generate_mtp(struct lg_session *s, struct mtp *t, const int *prompt, int n_prompt, int n_gen, int rows,
                             int *emitted, int *steps, int *n_draft, int *n_accept);
/* The same generation with `batch` rounds at a time kept on the device (lg_hip_mtp_rounds): the host
 * waits once per batch instead of once per draft and per verify step. */
int  lg_session_generate_mtp_rounds(struct lg_session *s, struct mtp *t, const int *prompt, int n_prompt, int n_gen, int rows,
                                    int batch, int *emitted, int *steps, int *n_draft, int *n_accept);
#endif
