/* lg_hip.h — C ABI of liblg_hip.so, the gfx950 backend of little-gemma's MTP verify step.
 *
 * Plain C: opaque handles, pointers, sizes, int status codes (0 = ok, negative = error; the
 * message is kept per thread and read with lg_hip_last_error()).  No HIP, torch or GGUF types
 * cross this boundary, so the reference's C host code (or anything with an FFI) can bind it.
 * model-hip.c (little-gemma_amd/host/) implements the reference's include/model.h on top of
 * these calls; each entry point below cites the reference interface it stands behind.
 *
 * Threading: one caller thread per model, like the reference backends
 * (src/cuda/model-cuda.cuh:724-726); calls on one model are not re-entrant.
 * Device errors are returned, never exit(): the caller decides (model-hip.c prints and exits
 * like CUDA_CHECK, src/cuda/model-cuda.cuh:34-36).
 */
#ifndef LG_HIP_H
#define LG_HIP_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LG_HIP_MAX_ROWS 8          /* widest verify block (LG_MTP_N) the kernels are built for */

typedef struct lg_hip_model lg_hip_model;
typedef struct lg_hip_kv    lg_hip_kv;

/* Hyper-parameters and per-layer geometry: the fields of struct config / struct model the
 * forward reads (include/model.h:10-48).  Arrays have n_layer entries and are copied. */
struct lg_hip_config {
    int32_t n_layer, n_embd, n_head, n_vocab;
    int32_t sliding_window, n_embd_per_layer, n_kv_start;
    float   rms_eps, rope_freq_base, rope_freq_base_swa, logit_softcap;
    const int32_t *is_local, *ffn_len, *head_dim, *n_head_kv;
};

const char *lg_hip_last_error(void);
/* Number of usable devices (0 when there is none); never fails. */
int lg_hip_device_count(void);

/* ---- model: weights resident on the device ------------------------------------------------
 * Replaces ensure_weights/ensure_scratch (src/cuda/model-cuda.cuh:738-799,937-970) with an
 * explicit sequence: create, hand over every tensor once, commit. */
int  lg_hip_model_create(const struct lg_hip_config *cfg, int device, lg_hip_model **out);
/* One GGUF tensor by its GGUF name (e.g. "blk.3.attn_q.weight"): ggml type id, dims[0] = row
 * length, dims[1] = rows, data = host bytes in GGUF layout.  Matrices must be q4_0 with a row
 * length that is a multiple of 256 and a row count that is a multiple of 8 (the reference's
 * repack has the same k%256 rule, src/cuda/model-cuda-i8.cu:613-620); vectors must be f32.
 * Unknown names are ignored (returns 1) so a caller can simply walk the file. */
int  lg_hip_model_tensor(lg_hip_model *m, const char *name, uint32_t ggml_type, uint32_t n_dims,
                         const uint64_t *dims, const void *data);
/* Checks that every tensor the forward needs arrived, lays weights out for the kernels and
 * allocates scratch for blocks of up to max_rows (1..LG_HIP_MAX_ROWS) verify rows. */
int  lg_hip_model_commit(lg_hip_model *m, int max_rows);
void lg_hip_model_destroy(lg_hip_model *m);

/* ---- KV cache: f16 rings on the device (kvcache_init/free, include/model.h:79-80;
 * src/cuda/model-cuda.cuh:998-1051).  Global layers hold max_seq rows, sliding layers
 * lg_hip_ring_rows(window, max_seq); row of position p = p % rows. */
int  lg_hip_kv_create(lg_hip_model *m, int max_seq, lg_hip_kv **out);
void lg_hip_kv_destroy(lg_hip_kv *kv);
int  lg_hip_ring_rows(int window, int max_seq);
/* What lg_hip_kv_create asks for besides the rings (no counterpart in the reference, whose attention
 * keeps its partials per launch): bytes of attention partials, one slot of (max, sum, max_hd
 * accumulators) per (row of the cache's widest block, head, key tile a block can touch).  The widest
 * PROMPT block of a cache (*wide_rows: 512, 128, 32, or 0 = verify-width blocks only) is the largest
 * whose partials stay within 2 GiB; any_global = the model has a layer without a sliding window.
 * Arithmetic only: callable without a device. */
size_t lg_hip_kv_partials(int max_seq, int window, int any_global, int max_rows, int n_head, int max_hd,
                          int *wide_rows, int *tiles_max);
/* rows/width of an owning layer's K (== V) storage; *rows = 0 for a layer that shares. */
int  lg_hip_kv_layout(const lg_hip_kv *kv, int layer, int *rows, int *width);
/* Copy whole cache rows (binary16 bit patterns) from/to host memory: which = 0 K, 1 V. */
int  lg_hip_kv_write(lg_hip_kv *kv, int layer, int which, int row0, int n_rows, const uint16_t *src);
int  lg_hip_kv_read(const lg_hip_kv *kv, int layer, int which, int row0, int n_rows, uint16_t *dst);
/* kvcache_save_prefix / kvcache_restore_prefix (include/model.h:82-92): first min(n, rows)
 * rows of every owning layer, device to device. */
int  lg_hip_kv_save_prefix(lg_hip_kv *kv, int n);
int  lg_hip_kv_restore_prefix(lg_hip_kv *kv, int n);

/* ---- the verify step: model_forward_spec (include/model.h:179-186,
 * src/cuda/mtp-kernel.cuh:82-120).  toks[0] is the chosen token at position pos, toks[1..]
 * the drafts; out[j] = greedy successor of toks[j] (first maximum of the soft-capped logits);
 * *adv = 1 + number of leading drafts that held.  K/V rows pos..pos+n_rows-1 are written.
 * Embedding lookup, the whole decoder, lm_head, argmax and the accept rule run on the device
 * inside one captured graph; the host copies n_rows tokens in and n_rows+1 ints out. */
int  lg_hip_forward_spec(lg_hip_model *m, lg_hip_kv *kv, const int32_t *toks, int n_rows, int pos,
                         int32_t *out, int32_t *adv);
/* model_prefill (include/model.h:121): positions pos0..pos0+n-1, cache writes only, no head.
 * Runs as blocks of 512 rows (128 when the cache holds fewer than 1024 positions) whose matmuls use the int8
 * matrix cores (the reference's chunked prefill, src/cuda/prefill-kernel.cuh:631-675), then 128- and 32-row
 * blocks, then verify-width blocks for the tail; every block leaves the cache rows that position-by-position
 * decode would. */
int  lg_hip_prefill(lg_hip_model *m, lg_hip_kv *kv, const int32_t *toks, int n, int pos0);
/* Post-output-norm hidden state of the last valid row of the latest verify step (n_embd
 * floats): what the reference keeps in g_hidden / model.last_hidden for the draft head
 * (src/cuda/mtp-kernel.cuh:117-118). */
int  lg_hip_get_hidden(lg_hip_model *m, float *dst);
/* Re-point that hidden state at row `row` of the latest step: for callers that accept rows by
 * their own rule (the sampling hook, src/cuda/mtp-kernel.cuh:103-118). */
int  lg_hip_set_hidden_row(lg_hip_model *m, int row);
/* Soft-capped logits of row `row` of the latest step (n_vocab floats).  Only stored while the
 * "store_logits" option is on (model_forward, include/model.h:98, needs them; the verify does not). */
int  lg_hip_get_logits(lg_hip_model *m, int row, float *dst);
/* Options: "store_logits" (0/1, default 0), "use_graph" (0/1, default 1), "wide_prefill" (0/1,
 * default 1: 0 sends the whole prompt through verify-width blocks). */
int  lg_hip_set_option(lg_hip_model *m, const char *name, int value);
/* Measurement aid (no reference counterpart): with the option "xcd_tail_stamps" on, every unit of the
 * one-XCD launches of a layer writes the device wall clock (100 MHz) at its 8 phase boundaries; this
 * copies the stamps of the latest such launch, [64 units][8], and returns 64.  which = 0: the launch that
 * ends the layer (lg_k_ple_tail), 1: the one that ends its attention half (lg_k_attn_tail). */
int  lg_hip_tail_stamps(lg_hip_model *m, int which, unsigned long long *dst, int cap);

/* ---- draft head: the gemma4-assistant network on the device (mtp_draft_device,
 * mtp_draft_chain_device, mtp_free_device: src/mtp-internal.h:33-37, src/cuda/mtp-kernel.cuh:272-402).
 * A head is a model object whose blocks own no cache: block L cross-attends the target's last
 * sliding (n_kv_start-2) or last global (n_kv_start-1) cache layer (src/mtp.c:173-176,193-201).
 * cfg: n_embd = the head's inner width, n_head_kv[L] / head_dim[L] / is_local[L] = those of the
 * target layer the block reads, n_kv_start and n_embd_per_layer = 0, sliding_window ignored (the
 * target's is used).  Tensors go through lg_hip_model_tensor under their GGUF names, the two
 * next-token projections as "pre_projection.weight" (2*n_embd(target) -> inner) and
 * "post_projection.weight" (inner -> n_embd(target), optional: without it drafts cannot chain);
 * then lg_hip_model_commit(head, 1).  Destroy with lg_hip_model_destroy before the target. */
int  lg_hip_draft_create(lg_hip_model *target, const struct lg_hip_config *cfg, lg_hip_model **out);
/* One draft: the token the head expects after `token`, where `token` will sit at position pos
 * and the target cache holds the positions before it.  chain = 0: h_prev is the target's hidden
 * state of the last accepted row (lg_hip_get_hidden(target)); chain = 1: h_prev is the post-
 * projection of this head's own hidden from its previous draft.  One captured graph per call
 * and a 4-byte read-back, like the reference.  lg_hip_get_hidden(head) afterwards returns the
 * head's post-norm hidden (inner width); lg_hip_get_logits(head, 0) its logits when stored. */
int  lg_hip_draft_step(lg_hip_model *head, lg_hip_kv *target_kv, int token, int pos, int chain, int32_t *tok_out);

/* Whole speculative rounds on the device: the loop the reference drives from the host with one
 * synchronisation per draft and per verify step (mtp_step, src/run.c:54-71, inside the generation
 * loop :737-768).  Round r verifies the block [chosen, d1..d(n_rows-1)] whose drafts the head
 * proposes (d1 from the target's hidden state, the others chained), accepts, and takes the greedy
 * successor of the last accepted row as the next round's chosen token; tokens and positions move
 * between head and target in device memory, one captured graph per round, and the host waits
 * once, after n_rounds.  token = the first chosen token, to sit at position pos; the target's
 * hidden state must be that of the token before it (as for lg_hip_draft_step with chain = 0).
 * Out: blocks[n_rounds][n_rows] as verified, out[n_rounds][n_rows] greedy successors,
 * adv[n_rounds]; round r emitted blocks[r][0..adv[r]-1] and *final_pos = pos + sum(adv).
 * The cache must hold pos + n_rows*n_rounds positions (every block may be accepted whole). */
int  lg_hip_mtp_rounds(lg_hip_model *head, lg_hip_kv *target_kv, int token, int pos, int n_rows, int n_rounds,
                       int32_t *blocks, int32_t *out, int32_t *adv, int32_t *final_pos);

/* ---- device-resident stepping: the same step with no host round trip between steps.
 * A schedule is n_steps blocks of n_rows tokens built by the caller (drafts come from a draft
 * head or, in the benchmark, are prepared in advance); each step verifies block `step`, writes
 * its out[] and adv, then advances the device-resident position by adv and the step counter
 * by one.  No reference counterpart: the reference synchronises every step
 * (src/cuda/mtp-kernel.cuh:95,112). */
int  lg_hip_schedule_load(lg_hip_model *m, const int32_t *toks, int n_steps, int n_rows, int pos0);
int  lg_hip_schedule_run(lg_hip_model *m, lg_hip_kv *kv, int n_steps);   /* enqueues, does not wait */
int  lg_hip_schedule_wait(lg_hip_model *m, int32_t *out, int32_t *adv, int32_t *final_pos);
/* Times n_steps already-loaded steps with device events on the library's stream; *ms = total. */
int  lg_hip_schedule_time(lg_hip_model *m, lg_hip_kv *kv, int n_steps, float *ms);

/* ---- measurement: run one step un-captured, every kernel launched with a start and a stop event of its own
 * (hipExtLaunchKernelGGL: the kernel's begin-to-end time, without the packet handling around it), and sum
 * the durations per kernel class.  names/ms/launches/bytes are caller arrays of `cap` entries;
 * returns the number of classes filled.  bytes[i] = weight + KV bytes the class must read per
 * step (algorithmic, not measured). */
int  lg_hip_profile_step(lg_hip_model *m, lg_hip_kv *kv, const int32_t *toks, int n_rows, int pos,
                         int repeats, const char **names, float *ms, int32_t *launches,
                         double *bytes, int cap);

/* What a chain of dependent kernels costs on this machine before it does any work: a captured graph of
 * n_kernels launches in a row, each of grid x block threads, replayed `replays` times; mode 0 = empty kernels,
 * mode 1 = every kernel reads the 64 bytes its predecessor wrote and writes 64 for its successor.
 * *us_per_kernel = elapsed / (replays * n_kernels).  No reference counterpart (the reference's own measure of
 * the same thing is its graph-vs-launch comparison, src/cuda/mtp-kernel.cuh:63-80). */
int  lg_hip_launch_floor(int n_kernels, int mode, int grid, int block, int replays, float *us_per_kernel);

/* Where the workgroups of a launch run and what a hand-over between the workgroups of ONE XCD costs (the chip has 8
 * XCDs with an L2 each; no reference counterpart: the reference's decode graph overlaps independent matmuls on a second
 * stream instead, src/cuda/model-cuda.cuh:917-935).
 * lg_hip_xcd_map: XCC_ID and HW_ID registers of every workgroup of `launches` consecutive launches of grid x block
 * threads with lds_bytes of dynamic LDS; xcc / hwid = [launches][grid].
 * lg_hip_xcd_handover: n (2..32) workgroups of a 256-workgroup launch -- set_mode 0: the workgroups i with i % 8 == sel
 * (one XCD when workgroups are dealt to the XCDs in turn); set_mode 1: workgroups sel*n .. sel*n+n-1 (spread over all
 * XCDs) -- run `rounds` rounds of: store `bytes` each, wait for the stores, raise a flag, poll the n flags, read the
 * neighbour's bytes back and check them.  store_scope / load_scope: 0 plain, 1 sc0, 2 sc1, 3 sc0 sc1.  res = [n][4]:
 * { ticks of the device wall clock over the rounds, words that were not what the neighbour wrote, polls given up,
 * XCD id }; *tick_ns = nanoseconds per tick.  Every wait is bounded: a combination that is not coherent reports
 * mismatches or given-up polls, it does not hang. */
int  lg_hip_xcd_map(int grid, int block, int lds_bytes, int launches, int32_t *xcc, int32_t *hwid);
int  lg_hip_xcd_handover(int set_mode, int sel, int n, int store_scope, int load_scope, int bytes, int rounds,
                         int32_t *res, float *tick_ns);

/* ---- isolated kernels, host pointers in and out (parity tests of the parts) ----------------
 * q4_0 x q8_0 matmul (matmul_q_spec, src/cuda/model-cuda-i8.cu:1592-1602): w = m rows of k/32
 * 18-byte q4_0 blocks; x = rows x k floats, quantized on the device per 32 (d_quant_group,
 * src/cuda/model-cuda.cuh:84-92).  Outputs (each may be NULL): out[rows][m] f32;
 * dots[rows][m][k/32] int32 block dots; xq[rows][k] int8; xd[rows][k/32] f32 scales;
 * xsum[rows][k/32] int32 sums.  *kernel_ms (may be NULL) = mean device time of `repeats` launches
 * of the matmul kernel alone. */
int  lg_hip_matmul_q4q8(const void *w, int k, int m, const float *x, int rows, float *out,
                        int32_t *dots, int8_t *xq, float *xd, int32_t *xsum, int repeats, float *kernel_ms);
/* The row work between two matmuls of a verify block (add-norm + norm + q8: add_rmsnorm_kernel, rmsnorm_kernel and
 * d_quant_group, src/cuda/model-cuda.cuh:119-175, :84-110, one kernel here): x_out = (x + rmsnorm(dout) * w_post) *
 * out_scale (dout, out_scale may be NULL), h = rmsnorm(x_out) * w_pre (w_pre NULL: h = x_out), q8 of h per 32.
 * rows 1..8, E a multiple of 256 up to 4096.  Outputs (each may be NULL): x_out, h_out [rows][E] f32, xq [rows][E]
 * int8, xd / xsum [rows][E/32]. */
int  lg_hip_rows_norm_q8(const float *x, const float *dout, const float *w_post, const float *out_scale,
                         const float *w_pre, int rows, int E, float eps, float *x_out, float *h_out,
                         int8_t *xq, float *xd, int32_t *xsum);
/* The kernel a verify block runs between ffn_down and the per-layer projection, on its own: the FFN residual update
 * x_out = x + rmsnorm(dout) * w_post, the inp_gate matmul on the q8 of x_out, gelu(.) * ipl and the q8 of that
 * (rmsnorm_add_kernel, matmul_q(inp_gate) and geglu_kernel of the per-layer-input block,
 * src/cuda/model-cuda.cuh:1251-1258; src/cpu/model-cpu.c:413-420).  w_gate = ple plain q4_0 rows of E weights, ipl =
 * [rows][ple].  rows 1..8, E a multiple of 256 up to 4096, ple = 256 (the width model_commit accepts).  Outputs (each may be
 * NULL): x_out [rows][E] f32, pq [rows][ple] int8, pd / psum [rows][ple/32]. */
int  lg_hip_rows_ple_gate(const float *x, const float *dout, const float *w_post, const void *w_gate, const float *ipl,
                          int rows, int E, int ple, float eps, float *x_out, int8_t *pq, float *pd, int32_t *psum);
/* The per-layer inputs of a block, on their own (build_per_layer_n, src/cuda/model-cuda.cuh:1121-1147):
 * out = (rmsnorm(pmp / sqrt(E)) * proj_norm + tok_row * sqrt(ple)) / sqrt(2) per (row, layer), pmp = the raw
 * per_layer_model_proj output [rows][n_layer*ple], pte = n_tok plain q4_0 rows of n_layer*ple (per_layer_token_embd),
 * toks = the rows' token ids (< n_tok).  out [rows][n_layer*ple]. */
int  lg_hip_ple_inputs(const float *pmp, const float *proj_norm, const void *pte, int n_tok, const int32_t *toks,
                       int rows, int n_layer, int ple, int E, float eps, float *out);
/* The feed-forward half of a layer for a verify block of 4..8 rows as ONE launch partitioned over the 8 XCDs of the
 * chip (rmsnorm_add_n_kernel + rmsnorm_kernel with the q8 epilogue, matmul_q_spec(gate / up), geglu_n_kernel,
 * matmul_q_spec(down): src/cuda/prefill-kernel.cuh:452-497), on its own: x_out = x + rmsnorm(dout) * w_post,
 * h = rmsnorm(x_out) * w_pre, act = gelu(gate . q8(h)) * (up . q8(h)), out = down . q8(act).  gate / up = FF plain
 * q4_0 rows of E weights, down = E rows of FF.  Shapes: E a multiple of 256 up to 4096 and FF a multiple of 256 that one
 * of the built instantiations serves (E 512 / FF 2048, E 2560 / FF 10240, E 3840 / FF 15360); a device of 256 compute
 * units in 8 XCDs.  Outputs (each may be NULL): x_out [rows][E], act [rows][FF], out [rows][E]; *kernel_ms = mean
 * device time of `repeats` launches, each preceded by a fill of flush_mb MiB when flush_mb > 0 (so that the weights
 * come from HBM as in a step, not from the memory-side cache); delay_w = units of 64 clocks the compute wavefronts wait
 * before they request their weights; stamps (NULL or [256][2][16]) = device wall-clock ticks
 * of every workgroup at its phase boundaries in the last launch, seen by its first wavefront and by the one that serves
 * the hand-overs. */
int  lg_hip_ffn_xcd(const float *x, const float *dout, const float *w_post, const float *w_pre, const void *gate,
                    const void *up, const void *down, int rows, int E, int FF, float eps, float *x_out, float *act,
                    float *out, int repeats, float *kernel_ms, int flush_mb, int delay_w, int64_t *stamps);
/* Matmul against a matrix kept in f32 (the per-layer-embedding matrices of QAT conversions; the reference's int8
 * backend multiplies such weights by the f32 activations unquantized, src/cuda/model-cuda-i8.cu:645-653, :846-895):
 * w = m rows of k floats, x = rows x k floats, out = rows x m floats.  Any number of rows (8 per workgroup row). */
int  lg_hip_matmul_f32w(const float *w, int k, int m, const float *x, int rows, float *out);
/* Decode attention over an f16 ring (split_attn_kernel + combine_attn_kernel,
 * src/cuda/model-cuda.cuh:527-608) for a block of `rows` queries at pos..pos+rows-1:
 * q = rows x n_head x hd floats, already normed and rotated; kc/vc = seq rows of n_head_kv*hd
 * binary16; window = 0 for a global layer.  out = rows x n_head x hd floats. */
int  lg_hip_attention(const float *q, const uint16_t *kc, const uint16_t *vc, int rows, int n_head,
                      int n_head_kv, int hd, int seq, int window, int pos, float *out,
                      int repeats, float *kernel_ms);
/* The same attention for callers that cannot allocate (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  q, kc, vc and out
 * are DEVICE pointers on the current device; the kernels' working memory (step state, tile partials)
 * lives in a static device array of lg_hip_attention_noalloc_limit() bytes (8 MiB, held by every GPU
 * the library runs on until the process ends), so the call allocates and frees nothing.  Shapes whose
 * partials do not fit (rows * n_head * key tiles * hd * 4 bytes, plus small change) are refused with
 * -2.  The launches go to `stream` (a hipStream_t, NULL = the default stream) and the call returns
 * without waiting: out is valid once the stream has passed them.  All calls on one GPU share the
 * array, so two calls that overlap in time on one GPU race; calls on one stream are ordered.
 * The first call on a device asks the runtime for the array's address and raises the kernels' dynamic
 * LDS limits, which a stream under capture does not allow: a caller that captures calls
 * lg_hip_attention_noalloc_init() on that device beforehand (it allocates nothing either, does the same
 * two things for every shape the entry point accepts, and is a no-op from then on). */
int    lg_hip_attention_noalloc(const float *d_q, const uint16_t *d_kc, const uint16_t *d_vc, int rows, int n_head,
                                int n_head_kv, int hd, int seq, int window, int pos, float *d_out, void *stream);
int    lg_hip_attention_noalloc_init(void);
size_t lg_hip_attention_noalloc_limit(void);
/* ffn_down of a verify block of 4..8 rows on the matrix cores (lg_k_down_m), in isolation: act = rows x FF floats (quantized
 * to q8 on the device, as the gate/up kernel's epilogue does), down = FF-wide q4_0 rows of the E outputs; out = rows x E,
 * the four K-quarter slabs added by the four workgroups of a row group themselves (join = 1: a hand-over inside their XCD)
 * or here as the consumer kernel adds them (join = 0).  The model path is ffn_down of
 * src/cuda/model-cuda-i8.cu's q4_0 x q8 matmul; this entry exists for parity tests and timing. */
int    lg_hip_down_m(const float *act, const void *down_q4_0, int rows, int E, int FF, int join, float *out, int repeats, float *kernel_ms);
/* Gate/up + GeGLU of a verify block in isolation: x = rows x E floats (quantized to q8 on the device by the step's row
 * kernel), gate / up = FF plain q4_0 rows of E each; aq / ad / asum receive the q8 of gelu(gate) * up in natural order
 * (rows x FF values, rows x FF/32 scales and sums).  1..3 rows run lg_k_geglu_t, 4..8 rows lg_k_geglu_m.  The model path
 * is the FFN of src/cuda/model-cuda.cuh:663-698 on src/cuda/model-cuda-i8.cu's q4_0 x q8 matmul; this entry exists for
 * parity tests and timing. */
int    lg_hip_gate_up_geglu(const float *x, const void *gate_q4_0, const void *up_q4_0, int rows, int E, int FF,
                            int8_t *aq, float *ad, int32_t *asum, int repeats, float *kernel_ms);
/* Host-side weight layout transform used by lg_hip_model_tensor, exposed for tests: q4_0 rows
 * -> the kernels' tile order.  dst needs lg_hip_repacked_bytes(k, m) bytes. */
int    lg_hip_segments(int k);      /* K segments of a row of k weights: 8, or 32 when k/32 > 128 and a multiple of 32 */
size_t lg_hip_repacked_bytes(int k, int m);
int    lg_hip_repack_q4_0(const void *src, int k, int m, void *dst);

#ifdef __cplusplus
}
#endif
#endif /* LG_HIP_H */
