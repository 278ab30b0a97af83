/* synth.h — seeded random-init Gemma-4-style models written as GGUF.
 *
 * No reference counterpart (the reference ships no model files or generators);
 * the tensor names, shapes and metadata keys are the ones its loader reads
 * (src/model.c:67-196, src/cpu/model-cpu.c:267-448).  Output depends only on
 * the spec, not on the thread count.
 */
#ifndef LG_SYNTH_H
#define LG_SYNTH_H

#include <stdint.h>

struct lg_synth_spec {
    int32_t n_layer, n_embd, n_head, n_head_kv;
    int32_t head_dim;          /* sliding-window layers */
    int32_t head_dim_full;     /* global layers; 0 = same as head_dim */
    int32_t n_ff, n_vocab, n_ctx;
    int32_t sliding_window;
    int32_t local_period;      /* layer L is global iff L % period == period-1; 0 = every layer global */
    int32_t ple;               /* per-layer-embedding width, 0 = none */
    int32_t shared_kv_layers;  /* trailing layers that reuse an earlier layer's KV (their k/v tensors are omitted) */
    int32_t has_v;             /* 0: no attn_v tensors (V = un-normed K projection) */
    int32_t has_rope_freqs;
    int32_t ple_float;         /* type of per_layer_model_proj / inp_gate / proj: 0 = q4_0, 1 = f32, 2 = f16, 3 = bf16 (what
                                  QAT conversions keep at full precision, src/cuda/model-cuda-i8.cu:645-653) */
    float   w_std;             /* std of every matrix before q4_0 packing */
    float   qk_norm;           /* centre of attn_q_norm / attn_k_norm weights; 0 = sqrt(1.28/sqrt(head_dim)) */
    float   norm_jitter;       /* norm weights are centre * (1 + jitter*u), u uniform in [-1,1) */
    float   out_scale;         /* layer_output_scale value; 0 = tensor absent */
    float   rms_eps, rope_base, rope_base_swa, softcap;
    uint64_t seed;
};

/* 0 on success; a negative code and a message on stderr otherwise. */
int lg_synth_write(const char *path, const struct lg_synth_spec *spec);

/* A draft head ("gemma4-assistant", src/mtp.c:124-215) for a target of width n_backbone whose
 * sliding / global layers have heads of head_dim_swa / head_dim_full: the last n_full blocks
 * read the global cache, the others the sliding one. */
struct lg_synth_assistant_spec {
    int32_t n_layer, n_inner, n_backbone, n_head, n_ff, n_vocab;
    int32_t head_dim_swa, head_dim_full, n_full;
    int32_t has_post;          /* 0: no post-projection (drafts cannot chain) */
    float   w_std, qk_norm, norm_jitter, out_scale;
    float   rms_eps, rope_base, rope_base_swa, softcap;
    uint64_t seed;
};
int lg_synth_write_assistant(const char *path, const struct lg_synth_assistant_spec *spec);

#endif
