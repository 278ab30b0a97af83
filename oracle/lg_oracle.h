/* lg_oracle.h — CPU oracle for the MTP speculative-verify path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product (the HIP library, the host
 * layer, run-hip) may include, link or call this; it exists so tests, the smoke
 * check and the benchmark's cpu_baseline leg have an independent statement of
 * what the path must compute.  Every function cites the reference lines it
 * restates; how each one is pinned is listed at the top of lg_oracle.c.
 */
#ifndef LG_ORACLE_H
#define LG_ORACLE_H

#include <stdint.h>
#include <stddef.h>

/* numerics classes of a whole forward */
enum lgo_mode {
    LGO_REF     = 0,  /* reference `run` (src/cpu/model-cpu.c): f32 activations, serial sums, libm,
                         f16 global KV + f32 window-exact sliding rings */
    LGO_I8      = 1,  /* reference `run-cuda-i8` class: q8 activations at the reference's quantization
                         points, exact int32 block dots, f16 KV everywhere; float orders and elementary
                         functions as this build defines them (include/lg_math.h) */
    LGO_I8_LIBM = 2,  /* LGO_I8 with libm elementary functions: measures what lg_math.h changes */
    LGO_I8_F32  = 3,  /* LGO_I8's op sequence, orders and functions with the activation quantization switched off
                         (f32 activations into a serial f32 dot): differs from LGO_REF by float reordering and
                         f16 sliding rings only, so the gap to LGO_REF pins the composition to reorder noise */
};

/* f32 combine order of the q4_0 x q8 matmul */
enum lgo_order {
    LGO_ORDER_SEG    = 0,  /* this build: lgo_segments(k) contiguous K segments, serial fma inside each,
                              adjacent-pair tree across them */
    LGO_ORDER_CUDA32 = 1,  /* reference: 32 lane-strided partials + shfl_down tree
                              (src/cuda/model-cuda-i8.cu:830-845,897-902) */
};

/* ---- primitives --------------------------------------------------------- */
void    lgo_quant_q8(const float *x, int n, int8_t *q, float *d, int32_t *sum);
int32_t lgo_block_dot(const unsigned char *block18, const int8_t *q32);
void    lgo_matmul_q4q8(const void *w, int k, int m, const int8_t *xq, const float *xd, int rows,
                        float *out, int32_t *dots, int order);
void    lgo_matmul_f32(const void *w, uint32_t ggml_type, int k, int m, const float *x, float *out);
/* f32 / f16 / bf16 weights x f32 activations in this build's order: lane (e/4)%64 partials, fma ascending, pair tree */
void    lgo_matmul_fw(const void *w, uint32_t ggml_type, int k, int m, const float *x, float *out);
void    lgo_rmsnorm(float *out, const float *x, const float *w, int n, float eps, int tree);
void    lgo_rope(float *v, int d, int pos, const float *freq_tab, const float *ff, int exact);
/* one (query head) attention over an f16 ring: keys start..pos, row of position p = p % seq */
void    lgo_attention_f16(float *out, const float *q, const uint16_t *kc, const uint16_t *vc,
                          int hd, int kv_dim, int kvh, int seq, int start, int pos, int tiled, int exact);
int     lgo_segments(int k);
int     lgo_accept(const int *toks, const int *out, int rows);
float   lgo_expf(float x); float lgo_tanhf(float x); void lgo_sincosf(float x, float *s, float *c);
float   lgo_gelu(float x, int exact);
uint16_t lgo_f32_to_f16(float f); float lgo_f16_to_f32(uint16_t h);
int     lgo_ring_rows(int window, int max_seq);

/* ---- whole model -------------------------------------------------------- */
struct lgo_model;
struct lgo_kv;
struct lgo_model *lgo_model_open(const char *gguf_path);
void  lgo_model_close(struct lgo_model *m);
int   lgo_model_info(const struct lgo_model *m, int32_t *out, int cap);  /* n_layer,n_embd,n_head,n_vocab,ple,n_kv_start,window,... */
int   lgo_layer_info(const struct lgo_model *m, int L, int32_t *out4);   /* is_local, head_dim, n_head_kv, ffn_len */
struct lgo_kv *lgo_kv_new(const struct lgo_model *m, int max_seq, int mode);
void  lgo_kv_free(struct lgo_kv *kv);
/* storage of layer L: *rows ring length, *width kv_dim, *is_f16; returns K (which=0) or V (1) base, NULL if shared */
void *lgo_kv_layer(struct lgo_kv *kv, int L, int which, int *rows, int *width, int *is_f16);
/* one position; logits/hidden may be NULL; returns the greedy token (first maximum) */
int   lgo_forward(struct lgo_model *m, struct lgo_kv *kv, int token, int pos, int mode,
                  float *logits, float *hidden);
void  lgo_prefill(struct lgo_model *m, struct lgo_kv *kv, const int *tokens, int n, int pos0, int mode);
/* sequential verify (src/cpu/model-cpu.c:51-58) over `rows` tokens; returns adv */
int   lgo_forward_spec(struct lgo_model *m, struct lgo_kv *kv, const int *toks, int rows, int pos,
                       int mode, int *out, float *hidden);
void  lgo_set_threads(int n);
/* the verify step as the device runs it: all rows forwarded (cache rows of rejected drafts
 * written), then the accept rule */
int   lgo_forward_spec_all(struct lgo_model *m, struct lgo_kv *kv, const int *toks, int rows, int pos,
                           int mode, int *out, float *hidden);

/* ---- draft head (src/mtp.c; device form src/cuda/mtp-kernel.cuh:272-402) -------------- */
struct lgo_mtp;
struct lgo_mtp *lgo_mtp_open(const char *gguf_path, const struct lgo_model *target);
void  lgo_mtp_close(struct lgo_mtp *t);
int   lgo_mtp_info(const struct lgo_mtp *t, int32_t *out, int cap);   /* n_layer,n_inner,n_bb,n_vocab,n_head,n_ff,has_post */
int   lgo_mtp_draft(struct lgo_mtp *t, struct lgo_model *target, struct lgo_kv *kv, int token, int pos,
                    const float *h_prev, int mode, float *hidden_out, float *logits_out);
int   lgo_mtp_post(struct lgo_mtp *t, const float *hidden, int mode, float *h_out);

#endif
