// lg_hip.hip — C ABI of the gfx950 verify-step backend (declared in include/lg_hip.h).
//
// Host side: weight layout, scratch, the launch sequence of one step, graph capture, the
// device-resident step schedule and the measurement helpers.  Device side: lg_kernels.h.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <map>
#include <mutex>
#include <string>
#include <type_traits>
#include <thread>
#include <vector>

#include "../../include/lg_hip.h"
#include "lg_kernels.h"
#include "lg_mfma.h"
#include "lg_fused.h"
#include "lg_xcd.h"
#include "lg_xffn.h"
#include "lg_xtail.h"
#include "lg_xrg.h"

static_assert(LG_HIP_MAX_ROWS == LG_HIP_MAX_ROWS_DEV, "row limits must agree");
#define LG_FUSE_ROWS_MAX 2         // widest block whose q/k/v matmul does the preceding row work itself

// ---- errors -----------------------------------------------------------------------------------
static thread_local char g_err[512] = "";
static int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}
#define HIP_TRY(expr) do { hipError_t e_ = (expr); if (e_ != hipSuccess) \
    return fail(-100 - (int)e_, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__); } while (0)

extern "C" const char *lg_hip_last_error(void) { return g_err; }
extern "C" int lg_hip_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) { (void)hipGetLastError(); return 0; }
    return n;
}
// The widest prompt block a cache of max_seq positions takes: LG_WIDE_ROWS for caches of 1024 positions and more,
// LG_WIDE_MID below (a short cache does not pay 512 spare rows per sliding ring and 512 rows of attention partials)
static int wide_rows_for(int max_seq) { return max_seq >= 1024 ? LG_WIDE_ROWS : LG_WIDE_MID; }
extern "C" int lg_hip_ring_rows(int window, int max_seq) {
    int r = (window + wide_rows_for(max_seq) + 31) / 32 * 32;   // window + spare for the widest block written before its queries run, tile multiple
    return r < max_seq ? r : max_seq;
}

// The attention partials of a cache: one (max, sum, hd accumulators) slot per (row of the widest block, head, key
// tile any block can touch).  A global layer's block late in a long cache touches every tile, so at the widest
// block the slots grow with rows x max_seq: the widest PROMPT block of a cache is stepped down (512, 128, 32 rows,
// then verify-width blocks only) until the partials fit LG_PARTIALS_BUDGET.  Pure arithmetic, no device needed.
#define LG_PARTIALS_BUDGET ((size_t)2 << 30)
extern "C" size_t lg_hip_kv_partials(int max_seq, int window, int any_global, int max_rows, int n_head, int max_hd,
                                     int *wide_rows, int *tiles_max) {
    const int steps[4] = { wide_rows_for(max_seq), LG_WIDE_MID, LG_WIDE, 0 };
    size_t bytes = 0;
    int wide = 0, tiles = 1;
    for (int i = 0; i < 4; ++i) {
        wide = steps[i];
        if (i > 0 && wide >= steps[i - 1]) continue;
        const int ring_span = window > 0 ? window + (wide > max_rows ? wide : max_rows) : max_seq;
        const int span = any_global || window <= 0 ? max_seq : ring_span;
        tiles = (span < max_seq ? span : max_seq) / 32 + 2;
        const size_t slots = (size_t)(max_rows > wide ? max_rows : wide) * n_head * tiles;
        bytes = slots * ((size_t)max_hd * 4 + 8);
        if (bytes <= LG_PARTIALS_BUDGET || wide == 0) break;
    }
    if (wide_rows) *wide_rows = wide;
    if (tiles_max) *tiles_max = tiles;
    return bytes;
}

// ---- weight layout ----------------------------------------------------------------------------
extern "C" int lg_hip_segments(int k) { return lg_segments(k); }

extern "C" size_t lg_hip_repacked_bytes(int k, int m) {
    if (k <= 0 || m <= 0 || k % 256 || m % 8) return 0;
    const int S = lg_segments(k);
    if ((k / 32) % S) return 0;
    return (size_t)(m / (64 / S)) * (size_t)(k / 32 / S) * LG_TILE;
}

// rows[i] points at virtual row i (k/32 blocks of 18 bytes each)
static void repack_rows(const uint8_t *const *rows, int k, int m, uint8_t *dst) {
    const int S = lg_segments(k), rw = 64 / S, nit = k / 32 / S, groups = m / rw;
    auto work = [&](int g0, int g1) {
        for (int g = g0; g < g1; ++g)
            for (int it = 0; it < nit; ++it) {
                uint8_t *tile = dst + ((size_t)g * nit + it) * LG_TILE;
                for (int r = 0; r < rw; ++r)
                    for (int c = 0; c < S; ++c) {
                        const uint8_t *blk = rows[g * rw + r] + (size_t)(c * nit + it) * 18;
                        memcpy(tile + (r * S + c) * 16, blk + 2, 16);
                        memcpy(tile + 1024 + (r * S + c) * 2, blk, 2);
                    }
            }
    };
    unsigned hw = std::thread::hardware_concurrency();
    int nt = (int)(hw ? (hw > 16 ? 16 : hw) : 4);
    if ((size_t)groups * nit < 4096 || nt < 2) { work(0, groups); return; }
    std::vector<std::thread> pool;
    for (int t = 0; t < nt; ++t) pool.emplace_back(work, (int)((long long)groups * t / nt), (int)((long long)groups * (t + 1) / nt));
    for (auto &th : pool) th.join();
}

// Row-block tiles (lg_k_geglu_t): tile (64-row block, kb) holds for lane r the 16 nibble bytes of block kb
// of row 64*block + r, then the 64 f16 scales; tiles ordered [block][kb].  Same size as the segment tiles.
static void repack_rowblocks(const uint8_t *const *rows, int k, int m, uint8_t *dst) {
    const int nb = k / 32, blocks = m / 64;
    auto work = [&](int b0, int b1) {
        for (int b = b0; b < b1; ++b)
            for (int kb = 0; kb < nb; ++kb) {
                uint8_t *tile = dst + ((size_t)b * nb + kb) * LG_TILE;
                for (int r = 0; r < 64; ++r) {
                    const uint8_t *blk = rows[b * 64 + r] + (size_t)kb * 18;
                    memcpy(tile + r * 16, blk + 2, 16);
                    memcpy(tile + 1024 + r * 2, blk, 2);
                }
            }
    };
    unsigned hw = std::thread::hardware_concurrency();
    int nt = (int)(hw ? (hw > 16 ? 16 : hw) : 4);
    if ((size_t)blocks * nb < 4096 || nt < 2) { work(0, blocks); return; }
    std::vector<std::thread> pool;
    for (int t = 0; t < nt; ++t) pool.emplace_back(work, (int)((long long)blocks * t / nt), (int)((long long)blocks * (t + 1) / nt));
    for (auto &th : pool) th.join();
}

extern "C" int lg_hip_repack_q4_0(const void *src, int k, int m, void *dst) {
    if (!lg_hip_repacked_bytes(k, m)) return fail(-2, "repack: k=%d must be a multiple of 256 (1024 above 4096) and m=%d of 8", k, m);
    std::vector<const uint8_t *> rows((size_t)m);
    for (int i = 0; i < m; ++i) rows[i] = (const uint8_t *)src + (size_t)i * (k / 32) * 18;
    repack_rows(rows.data(), k, m, (uint8_t *)dst);
    return 0;
}

// ---- objects ----------------------------------------------------------------------------------
struct HostTensor { uint32_t type, n_dims; uint64_t dims[4]; const void *data; };

struct Layer {
    uint8_t *wqkv = nullptr, *wo = nullptr, *wgu = nullptr, *wdown = nullptr, *winp = nullptr, *wproj = nullptr;
    float *winp_f = nullptr, *wproj_f = nullptr;   // inp_gate / proj when the file keeps them in a float type (then winp / wproj are null)
    uint8_t *wdn_m = nullptr;                      // ffn_down again as the per-workgroup streams of lg_k_down_m
    uint8_t *wo_ch = nullptr;                      // attn_output again as matrix-core chains [row block][segment]: lg_k_attn_tail
    uint8_t *wo_rb = nullptr;                      // attn_output again as row-block tiles: the chains of lg_k_merge_o
    uint8_t *xgu = nullptr, *xdn = nullptr;        // gate/up and ffn_down again as per-workgroup streams of the XCD-partitioned kernel (lg_xffn.h)
    float *attn_norm = nullptr, *q_norm = nullptr, *k_norm = nullptr, *post_attn = nullptr, *ffn_norm = nullptr,
          *post_ffw = nullptr, *post_norm = nullptr, *out_scale = nullptr;
    int is_local = 0, hd = 0, nkv = 0, nff = 0, qd = 0, kd = 0, qkv_m = 0, k_off = 0, v_off = 0, owns = 0, src = 0;
    const float *rope_tab = nullptr, *rope_ff = nullptr;
};

enum KClass { KC_ROWS, KC_PMP, KC_QKV, KC_QKVPOST, KC_ATTN, KC_MERGE, KC_O, KC_GATEUP, KC_DOWN, KC_PLEGATE, KC_PLEPROJ,
              KC_HEAD, KC_ACCEPT, KC_FFN, KC_TAIL, KC_ATAIL, KC_COUNT };
static const char *k_class_names[KC_COUNT] = { "rows_norm_quant", "ple_model_proj", "qkv", "qkv_post", "attn_tiles", "attn_merge",
    "attn_output", "gate_up_geglu", "ffn_down", "ple_gate", "ple_proj", "lm_head", "accept", "ffn_xcd", "ple_tail", "attn_tail" };

struct Profile {
    bool on = false;
    std::vector<hipEvent_t> ev;        // pairs
    std::vector<int> cls;
};

struct lg_hip_model {
    int device = 0;
    hipStream_t stream = nullptr;
    bool owns_stream = true;           // false for a draft head: it runs on its target's stream and never destroys it
    // a second stream and two events for the one branch of a step that is off the critical chain: the per-layer
    // inputs (per_layer_model_proj + lg_k_ipl), needed first by layer 0's per-layer gate, run beside layer 0's
    // attention and feed-forward (the reference forks its decode graph the same way, src/cuda/model-cuda.cuh:917-935)
    hipStream_t stream2 = nullptr;
    hipEvent_t ev_fork = nullptr, ev_join = nullptr;
    int fork_ple = 0;                  // option: use it.  Off: replayed as a graph with a second branch the step takes 2.77 ms instead of 2.26
    // config
    int n_layer = 0, E = 0, H = 0, n_vocab = 0, window = 0, ple = 0, n_kv_start = 0, max_rows = 0;
    float eps = 0, base = 0, base_swa = 0, softcap = 0;
    std::vector<int> is_local, ffn_len, head_dim, n_head_kv;
    std::map<std::string, HostTensor> host;
    bool committed = false;
    // weights
    std::vector<Layer> L;
    uint8_t *emb = nullptr, *pmp = nullptr, *pte = nullptr;
    float *pmp_f = nullptr;                        // per_layer_model_proj kept in a float type (then pmp is null)
    float *pgf = nullptr;                          // [rows][ple] f32 gate output, input of a float-typed proj
    uint8_t *emb_rb = nullptr;                     // token_embd again as row-block tiles: the lm_head of 4..8-row blocks (lg_k_head_m)
    float *output_norm = nullptr, *rope_freqs = nullptr, *proj_norm = nullptr;
    std::vector<void *> allocs;
    std::map<std::pair<int, int>, float *> rope_tabs;      // (is_local, hd) -> table
    size_t weight_bytes = 0;
    // scratch
    float *x[2] = { nullptr, nullptr }, *qkv = nullptr, *dout = nullptr, *pmp_raw = nullptr, *hidden_rows = nullptr,
          *g_hidden = nullptr, *logits = nullptr, *pval = nullptr, *q_rot = nullptr;
    int8_t *aq = nullptr, *gq = nullptr, *pq = nullptr, *hq = nullptr;     // q8 activation buffers (values + {scale,sum})
    int8_t *eq = nullptr;              // q8 of the block's embedding rows: input of per_layer_model_proj (kept apart from hq, which layer 0 rewrites meanwhile)
    int *pidx = nullptr;
    StepCtl *ctl = nullptr;
    int32_t *sched = nullptr, *out = nullptr, *adv = nullptr;
    int sched_cap = 0, sched_steps = 0, sched_rows = 0, sched_pos0 = 0, sched_loaded = 0;
    int32_t *pin = nullptr;            // pinned host staging
    int last_rows = 0, last_adv = 0;
    int store_logits = 0, use_graph = 1, wide_prefill = 1, fuse_rows = 1, attn_rows = 1, attn_rows_fq = 1, head_mfma = 1, down_kq = 1, tail_spread = 1, rows_geglu = 0;
    // the feed-forward half of a layer as one XCD-partitioned launch (lg_xffn.h): built when the shape and the chip fit
    int xcd_ffn = 0;                         // option: use it (verify blocks of 4..8 rows)
    int down_m = 1;                          // option: ffn_down of 4..8-row blocks on the matrix cores (lg_k_down_m): 1 = the row group's four workgroups add
                                             // their slabs themselves, 2 = four slabs for the consumer, 0 = the v_dot4 kernels; its streams are built
                                             // at commit unless LG_HIP_DOWN_M=0
    DownMSync *dmsync = nullptr;
    int xcd_attn_tail = 0;                   // option: attention merge, output projection and the row work after it as one launch on one XCD
                                             // (lg_k_attn_tail): 0 off (as measured it gains nothing), 1 from three rows up, 2 for every verify block;
                                             // the copy of the weights it reads is only built when LG_HIP_XCD_ATTN_TAIL is set at commit
    int merge_o = 0;                         // option: attention merge and output projection as one launch (lg_k_merge_o): 0 off (as measured it loses
                                             // as much in the row kernel that adds its 8 slabs as it gains), 1 from three rows up, 2 always; the second
                                             // copy of the weights it reads is only built when LG_HIP_MERGE_O is set at commit
    int merge_o_slices = 0;                  // option: slices of the output rows per (head, row), 0 = chosen by the launcher
    // the per-layer-input block and the next row work as one launch on one XCD (lg_xtail.h)
    int xcd_tail = 1;                        // option: 0 off, 1 for blocks that do not fold the row work into q/k/v, 2 for every verify block
    XtailSync *tsync = nullptr;
    float *tgf = nullptr;                    // [LG_HIP_MAX_ROWS][ple] gated values of lg_k_ple_tail_s
    RgSync *rgsync = nullptr;                // flags and epoch base of lg_k_rows_geglu
    unsigned long long *tstamps = nullptr;   // [LG_XTAIL_UNITS][8] phase stamps of the last such launch (option xcd_tail_stamps)
    int tail_stamps = 0;
    bool xffn_built = false;                 // streams and working memory exist
    int xffn_cls = -1;                       // which instantiation serves the shape
    int xffn_delay = 0;                      // option: units of 64 clocks its compute wavefronts wait before they request their weights
    float *slabs = nullptr, *xact = nullptr; // [8][max_rows][E] partial sums of ffn_down; [8][max_rows][max FF/8] gelu(gate)*up per XCD
    uint32_t *xq8 = nullptr;                 // [8][E/32][80] q8 rows per XCD
    XcdSync *xsync = nullptr;
    std::map<std::string, hipGraphExec_t> graphs;
    Profile prof;
    // a draft head (src/mtp.c) is a model whose layers own no cache: they read `target`'s
    lg_hip_model *target = nullptr;
    std::vector<lg_hip_model *> drafts;      // heads attached to this (target) model
    uint8_t *w_pre = nullptr, *w_post = nullptr;         // next-token pre / post projections, tiled
    int8_t *catq = nullptr;                  // q8 of [embedding(token) * sqrt(nb), h_prev], width 2*nb
    float *hprev = nullptr;                  // post-projection of the previous draft's hidden (chained drafts)
    bool draft_chain = false;
};

struct lg_hip_kv {
    lg_hip_model *m = nullptr;
    int max_seq = 0, tiles_max = 0, wide_rows = 0;      // wide_rows: the widest prompt block (sliding rings and partials are sized for it)
    std::vector<int> seq, kv_dim;
    std::vector<uint16_t *> k, v, px_k, px_v;
    float *pm = nullptr, *pl = nullptr, *pacc = nullptr;
    unsigned id = 0;
};
static unsigned g_kv_ids = 0;

template <typename T>
static int dev_alloc(lg_hip_model *m, T **p, size_t n) {
    HIP_TRY(hipMalloc((void **)p, n * sizeof(T) ? n * sizeof(T) : 16));
    m->allocs.push_back((void *)*p);
    return 0;
}

extern "C" int lg_hip_model_create(const struct lg_hip_config *c, int device, lg_hip_model **out) {
    if (!c || !out) return fail(-1, "model_create: null argument");
    if (c->n_layer <= 0 || c->n_embd <= 0 || c->n_embd % 256 || c->n_embd > 256 * LG_MAXV || c->n_head <= 0 ||
        c->n_vocab <= 0 || c->n_vocab % 32)
        return fail(-2, "model_create: unsupported shape (n_embd %d must be a multiple of 256 and <= %d, n_vocab %d a multiple of 32)",
                    c->n_embd, 256 * LG_MAXV, c->n_vocab);
    if (c->n_embd_per_layer % 32) return fail(-2, "model_create: per-layer embedding width %d must be a multiple of 256 or 0", c->n_embd_per_layer);
    if (lg_hip_device_count() <= device) return fail(-3, "model_create: no HIP device %d (the verify step has no CPU path)", device);
    HIP_TRY(hipSetDevice(device));
    lg_hip_model *m = new lg_hip_model();
    m->device = device;
    m->n_layer = c->n_layer; m->E = c->n_embd; m->H = c->n_head; m->n_vocab = c->n_vocab;
    m->window = c->sliding_window; m->ple = c->n_embd_per_layer; m->n_kv_start = c->n_kv_start;
    m->eps = c->rms_eps; m->base = c->rope_freq_base; m->base_swa = c->rope_freq_base_swa; m->softcap = c->logit_softcap;
    m->is_local.assign(c->is_local, c->is_local + c->n_layer);
    m->ffn_len.assign(c->ffn_len, c->ffn_len + c->n_layer);
    m->head_dim.assign(c->head_dim, c->head_dim + c->n_layer);
    m->n_head_kv.assign(c->n_head_kv, c->n_head_kv + c->n_layer);
    if (getenv("LG_HIP_NO_GRAPH")) m->use_graph = 0;       // un-captured launches (kernel tracing tools)
    if (getenv("LG_HIP_NO_FUSE")) m->fuse_rows = 0;        // row work in kernels of its own (comparison runs)
    if (getenv("LG_HIP_NO_ATTN_ROWS")) m->attn_rows = 0;   // attention tiles per row everywhere (comparison runs)
    if (const char *e = getenv("LG_HIP_ATTN_ROWS_FQ")) m->attn_rows_fq = atoi(e) != 0;
    if (const char *e = getenv("LG_HIP_ROWS_GEGLU")) m->rows_geglu = atoi(e) != 0;     // the row work ahead of gate/up inside the gate/up launch
    if (const char *e = getenv("LG_HIP_XCD_TAIL_SPREAD")) m->tail_spread = atoi(e);   // 0: the one-XCD tail as ple/32 x rows units of 4 wavefronts only; 2: as 8-wavefront units at 3 and 4 rows too
    if (getenv("LG_HIP_NO_DOWN_KQ")) m->down_kq = 0;       // ffn_down of verify blocks by whole rows everywhere (comparison runs)
    hipError_t e = hipStreamCreateWithFlags(&m->stream, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipStreamCreateWithFlags(&m->stream2, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&m->ev_fork, hipEventDisableTiming);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&m->ev_join, hipEventDisableTiming);
    if (e != hipSuccess) { delete m; return fail(-100 - (int)e, "hipStreamCreate: %s", hipGetErrorString(e)); }
    if (getenv("LG_HIP_FORK")) m->fork_ple = atoi(getenv("LG_HIP_FORK")) != 0;   // the per-layer inputs as a second branch (comparison runs)
    *out = m;
    return 0;
}

extern "C" int lg_hip_model_tensor(lg_hip_model *m, const char *name, uint32_t type, uint32_t n_dims,
                                   const uint64_t *dims, const void *data) {
    if (!m || !name || !dims || !data || n_dims < 1 || n_dims > 4) return fail(-1, "model_tensor: bad argument");
    if (m->committed) return fail(-4, "model_tensor: model already committed");
    static const char *top[] = { "token_embd.weight", "output_norm.weight", "rope_freqs.weight",
                                 "per_layer_token_embd.weight", "per_layer_model_proj.weight", "per_layer_proj_norm.weight",
                                 "pre_projection.weight", "post_projection.weight" };
    bool known = !strncmp(name, "blk.", 4);
    for (const char *t : top) known = known || !strcmp(name, t);
    if (!known) return 1;
    HostTensor h;
    h.type = type; h.n_dims = n_dims; h.data = data;
    for (int i = 0; i < 4; ++i) h.dims[i] = i < (int)n_dims ? dims[i] : 1;
    m->host[name] = h;
    return 0;
}

static const HostTensor *find(lg_hip_model *m, const std::string &name) {
    auto it = m->host.find(name);
    return it == m->host.end() ? nullptr : &it->second;
}
static std::string lname(int L, const char *leaf) { return "blk." + std::to_string(L) + "." + leaf; }

static int upload_vec(lg_hip_model *m, const std::string &name, size_t n, bool required, float **out) {
    const HostTensor *t = find(m, name);
    *out = nullptr;
    if (!t) return required ? fail(-5, "model_commit: tensor %s is missing", name.c_str()) : 0;
    size_t have = 1;
    for (uint32_t i = 0; i < t->n_dims; ++i) have *= t->dims[i];
    if (t->type != 0 || have != n) return fail(-6, "model_commit: %s must be f32 with %zu elements", name.c_str(), n);
    if (dev_alloc(m, out, n)) return -7;
    HIP_TRY(hipMemcpy(*out, t->data, n * 4, hipMemcpyHostToDevice));
    m->weight_bytes += n * 4;
    return 0;
}

struct RowSrc { const HostTensor *t; };
static int check_mat(const HostTensor *t, const std::string &name, uint64_t k, uint64_t mrows) {
    if (!t) return fail(-5, "model_commit: tensor %s is missing", name.c_str());
    if (t->type != 2) return fail(-6, "model_commit: %s has ggml type %u; the verify path takes q4_0 matrices only", name.c_str(), t->type);
    if (t->dims[0] != k || t->dims[1] != mrows) return fail(-6, "model_commit: %s is %llu x %llu, expected %llu x %llu", name.c_str(),
        (unsigned long long)t->dims[0], (unsigned long long)t->dims[1], (unsigned long long)k, (unsigned long long)mrows);
    if (k % 256 || mrows % 8) return fail(-6, "model_commit: %s needs row length %% 256 == 0 and rows %% 8 == 0", name.c_str());
    return 0;
}
// f32 / f16 / bf16 (ggml types 0 / 1 / 30): matrices a QAT conversion keeps at full precision
static bool float_typed(const HostTensor *t) { return t && (t->type == 0 || t->type == 1 || t->type == 30); }
static int upload_float_mat(lg_hip_model *m, const HostTensor *t, const std::string &name, uint64_t k, uint64_t mrows, float **out) {
    if (t->dims[0] != k || t->dims[1] != mrows) return fail(-6, "model_commit: %s is %llu x %llu, expected %llu x %llu", name.c_str(),
        (unsigned long long)t->dims[0], (unsigned long long)t->dims[1], (unsigned long long)k, (unsigned long long)mrows);
    if (k % 256) return fail(-6, "model_commit: %s needs row length %% 256 == 0", name.c_str());
    const size_t n = (size_t)k * mrows;
    std::vector<float> wide;
    const float *src = (const float *)t->data;
    if (t->type != 0) {                                       // widening f16 / bf16 to f32 is exact
        wide.resize(n);
        const uint16_t *h = (const uint16_t *)t->data;
        for (size_t i = 0; i < n; ++i) {
            if (t->type == 1) wide[i] = lg_f16_to_f32(h[i]);
            else { const uint32_t u = (uint32_t)h[i] << 16; memcpy(&wide[i], &u, 4); }
        }
        src = wide.data();
    }
    if (dev_alloc(m, out, n)) return -7;
    HIP_TRY(hipMemcpy(*out, src, n * 4, hipMemcpyHostToDevice));
    m->weight_bytes += n * 4;
    return 0;
}
// upload a tiled matrix whose virtual rows are given by `rows`
static int upload_tiled(lg_hip_model *m, const std::vector<const uint8_t *> &rows, int k, uint8_t **out,
                        std::vector<uint8_t> &stage, bool rowblocks = false) {
    const size_t bytes = lg_hip_repacked_bytes(k, (int)rows.size());
    if (!bytes || (rowblocks && (rows.size() % 64 || lg_segments(k) != 8))) return fail(-6, "model_commit: cannot tile a %zu x %d matrix", rows.size(), k);
    stage.resize(bytes);
    if (rowblocks) repack_rowblocks(rows.data(), k, (int)rows.size(), stage.data());
    else repack_rows(rows.data(), k, (int)rows.size(), stage.data());
    if (dev_alloc(m, out, bytes)) return -7;
    HIP_TRY(hipMemcpy(*out, stage.data(), bytes, hipMemcpyHostToDevice));
    m->weight_bytes += bytes;
    return 0;
}
static void push_rows(std::vector<const uint8_t *> &rows, const HostTensor *t, uint64_t r0, uint64_t n) {
    const size_t rb = (size_t)(t->dims[0] / 32) * 18;
    for (uint64_t r = r0; r < r0 + n; ++r) rows.push_back((const uint8_t *)t->data + r * rb);
}

static int cu_count();

// ---- weight streams of the XCD-partitioned feed-forward kernel (lg_xffn.h) --------------------------
// Shapes it is instantiated for: { gate/up operands per workgroup, blocks per gate/up segment (capacity), ffn_down
// chains per wavefront, blocks per ffn_down segment (capacity), q8 blocks of an XCD's activations (capacity) }.
struct XffnClass { int ops, nc, uw, ndc, cbc; };
static const XffnClass k_xffn_classes[] = { { 1, 2, 1, 8, 8 },       // E <= 512, FF <= 2048 (the small test models)
                                            { 3, 10, 2, 10, 40 },    // E4B shape: E 2560, FF 10240
                                            { 4, 15, 2, 15, 60 } };  // 12B shape: E 3840, FF 15360
static size_t xffn_lds(const XffnGeo &g, int M) { return g.lds(M); }
static int xffn_class_of(const XffnGeo &g) {
    if (!g.ok || (g.SX != 1 && g.SX != 4) || g.lds(LG_HIP_MAX_ROWS) + 256 > 160 * 1024) return -1;
    for (int c = 0; c < (int)(sizeof k_xffn_classes / sizeof k_xffn_classes[0]); ++c) {
        const XffnClass &k = k_xffn_classes[c];
        if (g.ops == k.ops && g.nit <= k.nc && (g.units + 7) / 8 <= k.uw && g.nitd <= k.ndc && g.CB <= k.cbc) return c;
    }
    return -1;
}
template <typename F>
static void for_workgroups(F work) {                  // the 256 workgroup streams, on a few host threads
    unsigned hw = std::thread::hardware_concurrency();
    const int nt = (int)(hw ? (hw > 16 ? 16 : hw) : 4);
    std::vector<std::thread> pool;
    for (int t = 0; t < nt; ++t) pool.emplace_back([=]() { for (int wg = 256 * t / nt; wg < 256 * (t + 1) / nt; ++wg) work(wg); });
    for (auto &th : pool) th.join();
}
// gate/up: workgroup (XCD x = wg % 8, rank r = wg / 8) owns the FFN columns x*C + r*CW .. + CW-1; its weight rows are
// those columns' gate rows followed by their up rows, cut into operands of 32; per K segment and operand: the nibble
// bytes as [pair of blocks][half h][row n] 8 + 8 bytes, then the f16 scales as [pair][row n] 2 + 2 bytes (an odd count
// of blocks is padded with a zero block)
static void xffn_pack_gu(const uint8_t *gate, const uint8_t *up, const XffnGeo &g, uint8_t *dst) {
    const size_t rowb = (size_t)g.nb * 18;
    memset(dst, 0, 256 * g.gu_bytes);
    for_workgroups([&](int wg) {
        const int x = wg & 7, r = wg >> 3, c0 = x * g.C + r * g.CW;
        for (int sg = 0; sg < 8; ++sg)
            for (int o = 0; o < g.ops; ++o) {
                const int vr = g.R2 - 32 * o < 32 ? g.R2 - 32 * o : 32;
                uint8_t *ob = dst + (size_t)wg * g.gu_bytes + (size_t)sg * g.gu_seg + (size_t)32 * o * g.rb;
                for (int n = 0; n < vr; ++n) {
                    const int li = 32 * o + n;
                    const uint8_t *row = li < g.CW ? gate + (size_t)(c0 + li) * rowb : up + (size_t)(c0 + li - g.CW) * rowb;
                    for (int it = 0; it < g.nit; ++it) {
                        const uint8_t *blk = row + (size_t)(sg * g.nit + it) * 18;
                        for (int h = 0; h < 2; ++h) memcpy(ob + (size_t)(((it >> 1) * 2 + h) * vr + n) * 16 + (it & 1) * 8, blk + 2 + 8 * h, 8);
                        memcpy(ob + (size_t)g.nitp * vr * 16 + (size_t)((it >> 1) * vr + n) * 4 + (it & 1) * 2, blk, 2);
                    }
                }
            }
    });
}
// ffn_down: workgroup (x, r) owns the output rows r*RW .. + RW-1 and the K segments x*SX .. + SX-1 of them; per
// (operand of 32 rows, segment): nibble bytes [pair of blocks][half][row], then scales [pair][row]
static void xffn_pack_dn(const uint8_t *down, const XffnGeo &g, uint8_t *dst) {
    const size_t rowb = (size_t)(g.FF >> 5) * 18;
    memset(dst, 0, 256 * g.dn_bytes);
    for_workgroups([&](int wg) {
        const int x = wg & 7, r = wg >> 3;
        for (int gr = 0; gr < g.groups; ++gr) {
            const int vr = g.RW - 32 * gr < 32 ? g.RW - 32 * gr : 32;
            for (int sx = 0; sx < g.SX; ++sx) {
                uint8_t *ub = dst + (size_t)wg * g.dn_bytes + (size_t)(gr * g.SX * 32 + sx * vr) * g.rbd;
                for (int n = 0; n < vr; ++n) {
                    const uint8_t *row = down + (size_t)(r * g.RW + 32 * gr + n) * rowb;
                    for (int it = 0; it < g.nitd; ++it) {
                        const uint8_t *blk = row + (size_t)((x * g.SX + sx) * g.nitd + it) * 18;
                        for (int h = 0; h < 2; ++h) memcpy(ub + (size_t)(((it >> 1) * 2 + h) * vr + n) * 16 + (it & 1) * 8, blk + 2 + 8 * h, 8);
                        memcpy(ub + (size_t)g.nitdp * vr * 16 + (size_t)((it >> 1) * vr + n) * 4 + (it & 1) * 2, blk, 2);
                    }
                }
            }
        }
    });
}

// ffn_down as the streams of lg_k_down_m: workgroup (row group r of 64, K quarter q), per segment 8q + s and operand of up to
// 32 rows the pair layout of the streams above
static void pack_down_m(const uint8_t *down, const DownMGeo &g, uint8_t *dst) {
    const size_t rowb = (size_t)(g.FF >> 5) * 18;
    memset(dst, 0, 256 * g.wg_bytes);
    for_workgroups([&](int wg) {
        const int r = wg >> 2, q = wg & 3;
        for (int s = 0; s < 8; ++s)
            for (int o = 0; o < g.ops; ++o) {
                const int vr = g.RW - 32 * o < 32 ? g.RW - 32 * o : 32;
                uint8_t *ob = dst + (size_t)wg * g.wg_bytes + (size_t)s * g.seg_bytes + (size_t)32 * o * g.nitdp * 18;
                for (int n = 0; n < vr; ++n) {
                    const uint8_t *row = down + (size_t)(r * g.RW + 32 * o + n) * rowb;
                    for (int it = 0; it < g.nitd; ++it) {
                        const uint8_t *blk = row + (size_t)((8 * q + s) * g.nitd + it) * 18;
                        for (int h = 0; h < 2; ++h) memcpy(ob + (size_t)(((it >> 1) * 2 + h) * vr + n) * 16 + (it & 1) * 8, blk + 2 + 8 * h, 8);
                        memcpy(ob + (size_t)g.nitdp * vr * 16 + (size_t)((it >> 1) * vr + n) * 4 + (it & 1) * 2, blk, 2);
                    }
                }
            }
    });
}
// shapes lg_k_down_m is instantiated for: operands per workgroup, pairs of blocks per segment
static bool down_m_shape(const DownMGeo &g) {
    return g.ok && ((g.ops == 1 && g.npairs <= 3) || (g.ops == 2 && g.npairs <= 5) || (g.ops == 2 && g.npairs <= 8));
}

// attn_output as the chains of lg_k_attn_tail: chain (row block rb of 32 rows, K segment c of 8) = the segment's nit blocks
// of the 32 rows in the pair layout of the streams above; chains ordered [rb][c], nit * 576 bytes each
static void pack_o_chains(const uint8_t *const *rows, int k, int m, uint8_t *dst) {
    const int nit = k / 32 / 8;
    const size_t cb = (size_t)nit * 576;
    for (int rb = 0; rb < m / 32; ++rb)
        for (int c = 0; c < 8; ++c) {
            uint8_t *ub = dst + ((size_t)rb * 8 + c) * cb;
            for (int n = 0; n < 32; ++n)
                for (int it = 0; it < nit; ++it) {
                    const uint8_t *blk = rows[rb * 32 + n] + (size_t)(c * nit + it) * 18;
                    for (int h = 0; h < 2; ++h) memcpy(ub + (size_t)(((it >> 1) * 2 + h) * 32 + n) * 16 + (it & 1) * 8, blk + 2 + 8 * h, 8);
                    memcpy(ub + (size_t)nit * 512 + (size_t)((it >> 1) * 32 + n) * 4 + (it & 1) * 2, blk, 2);
                }
        }
}
// shapes lg_k_attn_tail is instantiated for: pairs of blocks per chain, row blocks per unit
static bool attn_tail_shape(int qd, int E, int *np, int *rbs) {
    if (qd % 512 || lg_segments(qd) != 8 || E % 256 || E > 4096) return false;
    const int p = qd / 512, r = (E / 32 + LG_XCD_WGS - 1) / LG_XCD_WGS;
    if (np) *np = p;
    if (rbs) *rbs = r;
    return (p == 1 && r == 1) || (p == 2 && r == 1) || (p == 4 && r == 3);
}

static const float *rope_table(lg_hip_model *m, int is_local, int hd, int *rc) {
    auto key = std::make_pair(is_local, hd);
    auto it = m->rope_tabs.find(key);
    if (it != m->rope_tabs.end()) return it->second;
    std::vector<float> tab((size_t)hd / 2);
    const float base = is_local ? m->base_swa : m->base;
    for (int i = 0; i < hd / 2; ++i) tab[i] = powf(base, -2.0f * (float)i / (float)hd);   // src/cpu/model-cpu.c:90
    float *d = nullptr;
    if (hipMalloc((void **)&d, tab.size() * 4) != hipSuccess || hipMemcpy(d, tab.data(), tab.size() * 4, hipMemcpyHostToDevice) != hipSuccess) {
        *rc = fail(-7, "model_commit: rope table upload failed");
        return nullptr;
    }
    m->allocs.push_back(d);
    m->rope_tabs[key] = d;
    return d;
}

extern "C" int lg_hip_model_commit(lg_hip_model *m, int max_rows) {
    if (!m) return fail(-1, "model_commit: null model");
    if (m->committed) return fail(-4, "model_commit: already committed");
    if (max_rows < 1 || max_rows > LG_HIP_MAX_ROWS) return fail(-2, "model_commit: max_rows %d outside 1..%d", max_rows, LG_HIP_MAX_ROWS);
    HIP_TRY(hipSetDevice(m->device));
    m->max_rows = max_rows;
    const int E = m->E, H = m->H, nl = m->n_layer;
    std::vector<uint8_t> stage;
    int rc = 0;
    {
        const HostTensor *t = find(m, "token_embd.weight");
        if ((rc = check_mat(t, "token_embd.weight", E, m->n_vocab))) return rc;
        std::vector<const uint8_t *> rows;
        push_rows(rows, t, 0, m->n_vocab);
        if ((rc = upload_tiled(m, rows, E, &m->emb, stage))) return rc;
        // a second copy in the order the matrix-core lm_head reads (the first also serves the embedding lookup);
        // it is not counted into weight_bytes, which says what a step streams
        if (max_rows >= 4 && m->n_vocab % 64 == 0 && lg_segments(E) == 8 && !getenv("LG_HIP_NO_HEAD_MFMA")) {
            const size_t wb = m->weight_bytes;
            if ((rc = upload_tiled(m, rows, E, &m->emb_rb, stage, true))) return rc;
            m->weight_bytes = wb;
        }
    }
    if ((rc = upload_vec(m, "output_norm.weight", E, true, &m->output_norm))) return rc;
    int hd_global = 0;
    for (int L = 0; L < nl; ++L) if (!m->is_local[L]) hd_global = m->head_dim[L];
    if (find(m, "rope_freqs.weight") && hd_global)
        if ((rc = upload_vec(m, "rope_freqs.weight", hd_global / 2, true, &m->rope_freqs))) return rc;
    if (m->ple > 0 && find(m, "per_layer_token_embd.weight")) {
        if (m->ple % 32) return fail(-2, "model_commit: per-layer width %d", m->ple);
        const HostTensor *t = find(m, "per_layer_token_embd.weight");
        const uint64_t total = (uint64_t)m->ple * nl;
        if (t->type != 2 || t->dims[0] != total || t->dims[1] != (uint64_t)m->n_vocab)
            return fail(-6, "model_commit: per_layer_token_embd.weight must be q4_0 %llu x %d", (unsigned long long)total, m->n_vocab);
        const size_t bytes = (size_t)m->n_vocab * (total / 32) * 18;
        if (dev_alloc(m, &m->pte, bytes)) return -7;
        HIP_TRY(hipMemcpy(m->pte, t->data, bytes, hipMemcpyHostToDevice));
        const HostTensor *p = find(m, "per_layer_model_proj.weight");
        if (float_typed(p)) {
            if ((rc = upload_float_mat(m, p, "per_layer_model_proj.weight", E, total, &m->pmp_f))) return rc;
        } else {
            if ((rc = check_mat(p, "per_layer_model_proj.weight", E, total))) return rc;
            std::vector<const uint8_t *> rows;
            push_rows(rows, p, 0, total);
            if ((rc = upload_tiled(m, rows, E, &m->pmp, stage))) return rc;
        }
        if ((rc = upload_vec(m, "per_layer_proj_norm.weight", m->ple, true, &m->proj_norm))) return rc;
    } else m->ple = 0;

    m->L.resize(nl);
    int max_qkv = 0, max_ff = 0, max_qd = 0;
    // the XCD-partitioned feed-forward kernel: one shape for all layers, a chip of 256 CUs in 8 XCDs, blocks of 4+ rows
    XffnGeo xg = lg_xffn_geo(E, m->ffn_len[0]);
    // (its weight streams are second copies of the FFN matrices: built only when the option is asked for at commit)
    bool xffn = max_rows >= 4 && !m->target && cu_count() == LG_XCDS * LG_XCD_WGS && xffn_class_of(xg) >= 0 &&
                getenv("LG_HIP_XCD_FFN") && atoi(getenv("LG_HIP_XCD_FFN")) != 0;
    for (int L = 1; L < nl && xffn; ++L) xffn = m->ffn_len[L] == m->ffn_len[0];
    std::vector<uint8_t> xstage;
    for (int L = 0; L < nl; ++L) {
        Layer &y = m->L[L];
        y.is_local = m->is_local[L]; y.hd = m->head_dim[L]; y.nkv = m->n_head_kv[L]; y.nff = m->ffn_len[L];
        if (y.hd != 64 && y.hd != 128 && y.hd != 256 && y.hd != 512) return fail(-2, "model_commit: layer %d head size %d (64/128/256/512 are built)", L, y.hd);
        if (y.nkv <= 0 || H % y.nkv || H / y.nkv > 8) return fail(-2, "model_commit: layer %d: %d query heads per kv head (at most 8 are built)", L, H / y.nkv);
        if (y.nff % 32) return fail(-2, "model_commit: layer %d feed-forward width %d must be a multiple of 32", L, y.nff);
        y.qd = H * y.hd; y.kd = y.nkv * y.hd;
        y.owns = !m->target && L < m->n_kv_start;
        const int kv_start = m->target ? m->target->n_kv_start : m->n_kv_start;
        y.src = y.owns ? L : kv_start - (y.is_local ? 2 : 1);               // src/cpu/model-cpu.c:175-179, src/mtp.c:173-176
        if (y.src < 0) return fail(-2, "model_commit: layer %d has no layer to share KV with", L);
        if (m->target) {
            const Layer &t = m->target->L[y.src];
            if (t.hd != y.hd || t.nkv != y.nkv || (t.is_local != 0) != (y.is_local != 0))
                return fail(-2, "model_commit: draft block %d (head size %d, %d kv heads, %s) does not match the target layer %d it reads",
                            L, y.hd, y.nkv, y.is_local ? "sliding" : "global", y.src);
        }
        const HostTensor *q = find(m, lname(L, "attn_q.weight")), *k = find(m, lname(L, "attn_k.weight")),
                         *v = find(m, lname(L, "attn_v.weight"));
        if ((rc = check_mat(q, lname(L, "attn_q.weight"), E, y.qd))) return rc;
        std::vector<const uint8_t *> rows;
        push_rows(rows, q, 0, y.qd);
        y.qkv_m = y.qd;
        if (y.owns) {
            if ((rc = check_mat(k, lname(L, "attn_k.weight"), E, y.kd))) return rc;
            push_rows(rows, k, 0, y.kd);
            y.k_off = y.qd; y.v_off = y.qd; y.qkv_m += y.kd;                // no attn_v: V = raw K projection
            if (v) {
                if ((rc = check_mat(v, lname(L, "attn_v.weight"), E, y.kd))) return rc;
                push_rows(rows, v, 0, y.kd);
                y.v_off = y.qd + y.kd; y.qkv_m += y.kd;
            }
        }
        if ((rc = upload_tiled(m, rows, E, &y.wqkv, stage))) return rc;
        rows.clear();
        const HostTensor *o = find(m, lname(L, "attn_output.weight"));
        if ((rc = check_mat(o, lname(L, "attn_output.weight"), y.qd, E))) return rc;
        push_rows(rows, o, 0, E);
        if ((rc = upload_tiled(m, rows, y.qd, &y.wo, stage))) return rc;
        // (8 query heads: the K segments of this projection are the heads, and the merge can run their chains itself)
        if (getenv("LG_HIP_XCD_ATTN_TAIL") && atoi(getenv("LG_HIP_XCD_ATTN_TAIL")) > 0 && !m->target && attn_tail_shape(y.qd, E, nullptr, nullptr) &&
            cu_count() == LG_XCDS * LG_XCD_WGS) {
            stage.resize((size_t)E * (y.qd / 32) * 18);
            pack_o_chains(rows.data(), y.qd, E, stage.data());
            if (dev_alloc(m, &y.wo_ch, stage.size())) return -7;
            HIP_TRY(hipMemcpy(y.wo_ch, stage.data(), stage.size(), hipMemcpyHostToDevice));
            m->weight_bytes += stage.size();
        }
        if (getenv("LG_HIP_MERGE_O") && atoi(getenv("LG_HIP_MERGE_O")) > 0 && !m->target && m->H == 8 && lg_segments(y.qd) == 8 && E % 64 == 0 && y.hd % 32 == 0 && y.hd <= 512 &&
            (rc = upload_tiled(m, rows, y.qd, &y.wo_rb, stage, true))) return rc;
        rows.clear();
        const HostTensor *g = find(m, lname(L, "ffn_gate.weight")), *u = find(m, lname(L, "ffn_up.weight")),
                         *d = find(m, lname(L, "ffn_down.weight"));
        if ((rc = check_mat(g, lname(L, "ffn_gate.weight"), E, y.nff))) return rc;
        if ((rc = check_mat(u, lname(L, "ffn_up.weight"), E, y.nff))) return rc;
        if ((rc = check_mat(d, lname(L, "ffn_down.weight"), y.nff, E))) return rc;
        for (int t = 0; t < y.nff / 32; ++t) { push_rows(rows, g, (uint64_t)t * 32, 32); push_rows(rows, u, (uint64_t)t * 32, 32); }
        if ((rc = upload_tiled(m, rows, E, &y.wgu, stage, true))) return rc;    // row-block tiles (lg_k_geglu_t)
        rows.clear();
        push_rows(rows, d, 0, E);
        if ((rc = upload_tiled(m, rows, y.nff, &y.wdown, stage))) return rc;
        rows.clear();
        if (!(getenv("LG_HIP_DOWN_M") && atoi(getenv("LG_HIP_DOWN_M")) <= 0) && !m->target && max_rows >= 4 && cu_count() == LG_XCDS * LG_XCD_WGS) {
            const DownMGeo dg = lg_down_m_geo(E, y.nff);
            if (down_m_shape(dg)) {
                xstage.resize(256 * dg.wg_bytes);
                pack_down_m((const uint8_t *)d->data, dg, xstage.data());
                if (dev_alloc(m, &y.wdn_m, 256 * dg.wg_bytes)) return -7;
                HIP_TRY(hipMemcpy(y.wdn_m, xstage.data(), 256 * dg.wg_bytes, hipMemcpyHostToDevice));
                if (!m->dmsync) {
                    if (dev_alloc(m, &m->dmsync, (size_t)1)) return -7;
                    HIP_TRY(hipMemset(m->dmsync, 0, sizeof(DownMSync)));
                }
            }
        }
        if (xffn) {                                               // (second copies: not counted into weight_bytes, which says what a step streams)
            xstage.resize(256 * (xg.gu_bytes > xg.dn_bytes ? xg.gu_bytes : xg.dn_bytes));
            xffn_pack_gu((const uint8_t *)g->data, (const uint8_t *)u->data, xg, xstage.data());
            if (dev_alloc(m, &y.xgu, 256 * xg.gu_bytes)) return -7;
            HIP_TRY(hipMemcpy(y.xgu, xstage.data(), 256 * xg.gu_bytes, hipMemcpyHostToDevice));
            xffn_pack_dn((const uint8_t *)d->data, xg, xstage.data());
            if (dev_alloc(m, &y.xdn, 256 * xg.dn_bytes)) return -7;
            HIP_TRY(hipMemcpy(y.xdn, xstage.data(), 256 * xg.dn_bytes, hipMemcpyHostToDevice));
        }
        if (m->ple) {
            if (m->ple != 256) return fail(-2, "model_commit: per-layer width %d (256 is built)", m->ple);
            const HostTensor *ig = find(m, lname(L, "inp_gate.weight")), *pj = find(m, lname(L, "proj.weight"));
            if (float_typed(ig) != float_typed(pj))
                return fail(-6, "model_commit: blk.%d inp_gate and proj must both be q4_0 or both f32/f16/bf16", L);
            if (float_typed(ig)) {
                if ((rc = upload_float_mat(m, ig, lname(L, "inp_gate.weight"), E, m->ple, &y.winp_f))) return rc;
                if ((rc = upload_float_mat(m, pj, lname(L, "proj.weight"), m->ple, E, &y.wproj_f))) return rc;
            } else {
            if ((rc = check_mat(ig, lname(L, "inp_gate.weight"), E, m->ple))) return rc;
            if ((rc = check_mat(pj, lname(L, "proj.weight"), m->ple, E))) return rc;
            push_rows(rows, ig, 0, m->ple);
            if ((rc = upload_tiled(m, rows, E, &y.winp, stage))) return rc;
            rows.clear();
            push_rows(rows, pj, 0, E);
            if ((rc = upload_tiled(m, rows, m->ple, &y.wproj, stage))) return rc;
            }
            if ((rc = upload_vec(m, lname(L, "post_norm.weight"), E, true, &y.post_norm))) return rc;
        }
        if ((rc = upload_vec(m, lname(L, "attn_norm.weight"), E, true, &y.attn_norm))) return rc;
        if ((rc = upload_vec(m, lname(L, "attn_q_norm.weight"), y.hd, true, &y.q_norm))) return rc;
        if ((rc = upload_vec(m, lname(L, "attn_k_norm.weight"), y.hd, y.owns, &y.k_norm))) return rc;
        if ((rc = upload_vec(m, lname(L, "post_attention_norm.weight"), E, true, &y.post_attn))) return rc;
        if ((rc = upload_vec(m, lname(L, "ffn_norm.weight"), E, true, &y.ffn_norm))) return rc;
        if ((rc = upload_vec(m, lname(L, "post_ffw_norm.weight"), E, true, &y.post_ffw))) return rc;
        if ((rc = upload_vec(m, lname(L, "layer_output_scale.weight"), 1, false, &y.out_scale))) return rc;
        y.rope_tab = rope_table(m, y.is_local, y.hd, &rc);
        if (!y.rope_tab) return rc;
        y.rope_ff = y.is_local ? nullptr : m->rope_freqs;
        if (y.qkv_m > max_qkv) max_qkv = y.qkv_m;
        if (y.nff > max_ff) max_ff = y.nff;
        if (y.qd > max_qd) max_qd = y.qd;
    }
    if (m->target) {
        const int nb = m->target->E;
        const HostTensor *pre = find(m, "pre_projection.weight"), *post = find(m, "post_projection.weight");
        if ((rc = check_mat(pre, "pre_projection.weight", 2 * (uint64_t)nb, E))) return rc;
        std::vector<const uint8_t *> rows;
        push_rows(rows, pre, 0, E);
        if ((rc = upload_tiled(m, rows, 2 * nb, &m->w_pre, stage))) return rc;
        if (post) {                                                 // optional: without it drafts cannot chain
            if ((rc = check_mat(post, "post_projection.weight", E, nb))) return rc;
            rows.clear();
            push_rows(rows, post, 0, nb);
            if ((rc = upload_tiled(m, rows, E, &m->w_post, stage))) return rc;
        }
        if (dev_alloc(m, &m->catq, (size_t)2 * nb * 5 / 4) || dev_alloc(m, &m->hprev, (size_t)nb)) return -7;
        if (max_rows != 1) return fail(-2, "model_commit: a draft head runs one row at a time");
    }
    m->host.clear();
    // Layer scratch holds the widest block that can run: LG_WIDE_ROWS for a model that takes prompts, max_rows for a
    // draft head (it is never prefilled).  What only the head touches (final-norm rows, per-workgroup maxima, logits)
    // holds max_rows: a prompt block has no head.
    const size_t R = (size_t)(m->target || max_rows > LG_WIDE_ROWS ? max_rows : LG_WIDE_ROWS), HR = (size_t)max_rows;
    if (dev_alloc(m, &m->x[0], R * E) || dev_alloc(m, &m->x[1], R * E) || dev_alloc(m, &m->qkv, R * max_qkv) ||
        dev_alloc(m, &m->dout, 4 * R * E) || dev_alloc(m, &m->q_rot, R * max_qd) || dev_alloc(m, &m->hidden_rows, HR * E) || dev_alloc(m, &m->g_hidden, (size_t)E) ||
        dev_alloc(m, &m->aq, R * max_qd * 5 / 4) || dev_alloc(m, &m->gq, R * max_ff * 5 / 4) || dev_alloc(m, &m->hq, R * E * 5 / 4 + (size_t)12 * E) ||
        dev_alloc(m, &m->pval, HR * (m->n_vocab / 32)) || dev_alloc(m, &m->pidx, HR * (m->n_vocab / 32)) ||
        dev_alloc(m, &m->logits, HR * m->n_vocab) || dev_alloc(m, &m->ctl, (size_t)1))
        return -7;
    if (m->ple && dev_alloc(m, &m->eq, R * E * 5 / 4 + (size_t)12 * E)) return -7;
    if (!m->target) {                        // hand-over state of the one-XCD kernels (lg_xtail.h)
        if (dev_alloc(m, &m->tsync, (size_t)1) || dev_alloc(m, &m->tstamps, (size_t)2 * LG_XTAIL_UNITS * 8) ||
            dev_alloc(m, &m->tgf, (size_t)LG_HIP_MAX_ROWS * (m->ple > 0 ? m->ple : 1))) return -7;
        HIP_TRY(hipMemset(m->tstamps, 0, (size_t)2 * LG_XTAIL_UNITS * 8 * 8));
        HIP_TRY(hipMemset(m->tsync, 0, sizeof(XtailSync)));
        if (dev_alloc(m, &m->rgsync, (size_t)1)) return -7;
        HIP_TRY(hipMemset(m->rgsync, 0, sizeof(RgSync)));
        HIP_TRY(hipMemset(m->aq, 0, R * max_qd * 5 / 4));       // (row slots past the block are read as operand rows of the matrix cores)
        if (getenv("LG_HIP_XCD_TAIL")) m->xcd_tail = atoi(getenv("LG_HIP_XCD_TAIL"));
    }
    if (getenv("LG_HIP_XCD_ATTN_TAIL")) m->xcd_attn_tail = atoi(getenv("LG_HIP_XCD_ATTN_TAIL"));
    if (getenv("LG_HIP_DOWN_M")) m->down_m = atoi(getenv("LG_HIP_DOWN_M"));
    if (getenv("LG_HIP_MERGE_O")) m->merge_o = atoi(getenv("LG_HIP_MERGE_O"));
    if (getenv("LG_HIP_MERGE_O_SLICES")) m->merge_o_slices = atoi(getenv("LG_HIP_MERGE_O_SLICES"));
    if (m->ple && (dev_alloc(m, &m->pmp_raw, R * m->ple * nl) || dev_alloc(m, &m->pq, R * m->ple * 5 / 4) || dev_alloc(m, &m->pgf, R * m->ple)))
        return -7;
    if (xffn) {
        if (dev_alloc(m, &m->slabs, (size_t)LG_XCDS * max_rows * E) || dev_alloc(m, &m->xact, (size_t)LG_XCDS * max_rows * xg.C) ||
            dev_alloc(m, &m->xq8, (size_t)LG_XCDS * xg.nb * LG_MU_DWORDS) || dev_alloc(m, &m->xsync, (size_t)1)) return -7;
        HIP_TRY(hipMemset(m->xsync, 0, sizeof(XcdSync)));
        HIP_TRY(hipMemset(m->xq8, 0, (size_t)LG_XCDS * xg.nb * LG_MU_DWORDS * 4));        // row slots past the block are read as operand rows
        m->xffn_built = true; m->xffn_cls = xffn_class_of(xg);
        m->xcd_ffn = getenv("LG_HIP_XCD_FFN") && atoi(getenv("LG_HIP_XCD_FFN")) != 0;     // off unless asked for: the separate kernels are faster (see lg_xffn.h)
        m->xffn_delay = 0x100;
    }
    HIP_TRY(hipMemset(m->ctl, 0, sizeof(StepCtl)));
    HIP_TRY(hipMemset(m->g_hidden, 0, (size_t)E * 4));
    m->sched_cap = 4096;
    if (dev_alloc(m, &m->sched, (size_t)m->sched_cap * LG_HIP_MAX_ROWS + LG_WIDE_ROWS) || dev_alloc(m, &m->out, (size_t)m->sched_cap * LG_HIP_MAX_ROWS) ||
        dev_alloc(m, &m->adv, (size_t)m->sched_cap))
        return -7;
    // pinned staging: step state at 0, a verify block's successors at 32 and accept count at 48, a block's tokens from 64
    HIP_TRY(hipHostMalloc((void **)&m->pin, (64 + LG_WIDE_ROWS) * sizeof(int32_t), hipHostMallocDefault));
    HIP_TRY(hipDeviceSynchronize());
    m->committed = true;
    return 0;
}

extern "C" void lg_hip_model_destroy(lg_hip_model *m) {
    if (!m) return;
    (void)hipSetDevice(m->device);
    (void)hipDeviceSynchronize();
    for (auto &g : m->graphs) (void)hipGraphExecDestroy(g.second);
    for (void *p : m->allocs) (void)hipFree(p);
    for (hipEvent_t e : m->prof.ev) (void)hipEventDestroy(e);
    if (m->pin) (void)hipHostFree(m->pin);
    if (m->target) {
        auto &v = m->target->drafts;
        for (size_t i = 0; i < v.size(); ++i) if (v[i] == m) { v.erase(v.begin() + i); break; }
    }
    if (m->owns_stream && m->stream) (void)hipStreamDestroy(m->stream);
    if (m->stream2) (void)hipStreamDestroy(m->stream2);
    if (m->ev_fork) (void)hipEventDestroy(m->ev_fork);
    if (m->ev_join) (void)hipEventDestroy(m->ev_join);
    for (lg_hip_model *d : m->drafts) { d->target = nullptr; d->stream = nullptr; }        // orphaned heads refuse to run
    delete m;
}

// ---- KV cache ---------------------------------------------------------------------------------
extern "C" int lg_hip_kv_create(lg_hip_model *m, int max_seq, lg_hip_kv **out) {
    if (!m || !out || !m->committed) return fail(-1, "kv_create: model not committed");
    if (max_seq < 1) return fail(-2, "kv_create: max_seq %d", max_seq);
    HIP_TRY(hipSetDevice(m->device));
    lg_hip_kv *kv = new lg_hip_kv();
    kv->m = m; kv->max_seq = max_seq; kv->id = ++g_kv_ids;
    const int nl = m->n_layer;
    kv->seq.assign(nl, 0); kv->kv_dim.assign(nl, 0);
    kv->k.assign(nl, nullptr); kv->v.assign(nl, nullptr); kv->px_k.assign(nl, nullptr); kv->px_v.assign(nl, nullptr);
    int max_hd = 0, any_global = 0;
    for (int L = 0; L < nl; ++L) {
        const Layer &y = m->L[L];
        if (y.hd > max_hd) max_hd = y.hd;
        if (!(y.is_local && m->window > 0)) any_global = 1;
    }
    const size_t pbytes = lg_hip_kv_partials(max_seq, m->window, any_global, m->max_rows, m->H, max_hd, &kv->wide_rows, &kv->tiles_max);
    for (int L = 0; L < nl; ++L) {
        const Layer &y = m->L[L];
        kv->kv_dim[L] = y.kd;
        if (!y.owns) continue;
        const bool ring = y.is_local && m->window > 0;
        kv->seq[L] = ring ? lg_hip_ring_rows(m->window, max_seq) : max_seq;
        const size_t bytes = (size_t)kv->seq[L] * y.kd * 2;
        hipError_t e1 = hipMalloc((void **)&kv->k[L], bytes), e2 = hipMalloc((void **)&kv->v[L], bytes);
        if (e1 != hipSuccess || e2 != hipSuccess) { lg_hip_kv_destroy(kv); return fail(-7, "kv_create: out of device memory at layer %d", L); }
        (void)hipMemset(kv->k[L], 0, bytes); (void)hipMemset(kv->v[L], 0, bytes);
    }
    const size_t slots = pbytes / ((size_t)max_hd * 4 + 8);
    if (hipMalloc((void **)&kv->pm, slots * 4) != hipSuccess || hipMalloc((void **)&kv->pl, slots * 4) != hipSuccess ||
        hipMalloc((void **)&kv->pacc, slots * max_hd * 4) != hipSuccess) { lg_hip_kv_destroy(kv); return fail(-7, "kv_create: out of device memory for attention partials"); }
    HIP_TRY(hipDeviceSynchronize());
    *out = kv;
    return 0;
}

extern "C" void lg_hip_kv_destroy(lg_hip_kv *kv) {
    if (!kv) return;
    (void)hipSetDevice(kv->m->device);
    (void)hipDeviceSynchronize();
    // graphs captured for this cache hold its pointers
    const std::string tag = "kv" + std::to_string(kv->id) + ":";
    std::vector<lg_hip_model *> holders(kv->m->drafts);
    holders.push_back(kv->m);
    for (lg_hip_model *h : holders)
        for (auto it = h->graphs.begin(); it != h->graphs.end();) {
            if (it->first.compare(0, tag.size(), tag) == 0) { (void)hipGraphExecDestroy(it->second); it = h->graphs.erase(it); }
            else ++it;
        }
    for (size_t L = 0; L < kv->k.size(); ++L) {
        (void)hipFree(kv->k[L]); (void)hipFree(kv->v[L]); (void)hipFree(kv->px_k[L]); (void)hipFree(kv->px_v[L]);
    }
    (void)hipFree(kv->pm); (void)hipFree(kv->pl); (void)hipFree(kv->pacc);
    delete kv;
}

extern "C" int lg_hip_kv_layout(const lg_hip_kv *kv, int layer, int *rows, int *width) {
    if (!kv || layer < 0 || layer >= (int)kv->seq.size()) return fail(-1, "kv_layout: bad layer %d", layer);
    if (rows) *rows = kv->seq[layer];
    if (width) *width = kv->kv_dim[layer];
    return 0;
}
static int kv_span(const lg_hip_kv *kv, int layer, int which, int row0, int n, size_t *off, size_t *bytes, uint16_t **base) {
    if (!kv || layer < 0 || layer >= (int)kv->seq.size() || !kv->k[layer]) return fail(-1, "kv copy: layer %d owns no cache", layer);
    if (row0 < 0 || n < 0 || row0 + n > kv->seq[layer]) return fail(-2, "kv copy: rows %d..%d outside 0..%d", row0, row0 + n, kv->seq[layer]);
    *off = (size_t)row0 * kv->kv_dim[layer];
    *bytes = (size_t)n * kv->kv_dim[layer] * 2;
    *base = which ? kv->v[layer] : kv->k[layer];
    return 0;
}
extern "C" int lg_hip_kv_write(lg_hip_kv *kv, int layer, int which, int row0, int n, const uint16_t *src) {
    size_t off, bytes; uint16_t *base;
    int rc = kv_span(kv, layer, which, row0, n, &off, &bytes, &base);
    if (rc) return rc;
    HIP_TRY(hipSetDevice(kv->m->device));
    HIP_TRY(hipStreamSynchronize(kv->m->stream));
    HIP_TRY(hipMemcpy(base + off, src, bytes, hipMemcpyHostToDevice));
    return 0;
}
extern "C" int lg_hip_kv_read(const lg_hip_kv *kv, int layer, int which, int row0, int n, uint16_t *dst) {
    size_t off, bytes; uint16_t *base;
    int rc = kv_span(kv, layer, which, row0, n, &off, &bytes, &base);
    if (rc) return rc;
    HIP_TRY(hipSetDevice(kv->m->device));
    HIP_TRY(hipStreamSynchronize(kv->m->stream));
    HIP_TRY(hipMemcpy(dst, base + off, bytes, hipMemcpyDeviceToHost));
    return 0;
}
extern "C" int lg_hip_kv_save_prefix(lg_hip_kv *kv, int n) {
    if (!kv || n < 0) return fail(-1, "kv_save_prefix: bad argument");
    HIP_TRY(hipSetDevice(kv->m->device));
    HIP_TRY(hipStreamSynchronize(kv->m->stream));
    for (size_t L = 0; L < kv->k.size(); ++L) {
        if (!kv->k[L]) continue;
        const int rows = n < kv->seq[L] ? n : kv->seq[L];
        const size_t bytes = (size_t)rows * kv->kv_dim[L] * 2;
        (void)hipFree(kv->px_k[L]); (void)hipFree(kv->px_v[L]);
        kv->px_k[L] = kv->px_v[L] = nullptr;
        if (!bytes) continue;
        HIP_TRY(hipMalloc((void **)&kv->px_k[L], bytes));
        HIP_TRY(hipMalloc((void **)&kv->px_v[L], bytes));
        HIP_TRY(hipMemcpy(kv->px_k[L], kv->k[L], bytes, hipMemcpyDeviceToDevice));
        HIP_TRY(hipMemcpy(kv->px_v[L], kv->v[L], bytes, hipMemcpyDeviceToDevice));
    }
    return 0;
}
extern "C" int lg_hip_kv_restore_prefix(lg_hip_kv *kv, int n) {
    if (!kv || n < 0) return fail(-1, "kv_restore_prefix: bad argument");
    HIP_TRY(hipSetDevice(kv->m->device));
    for (size_t L = 0; L < kv->k.size(); ++L) {
        if (!kv->px_k[L]) continue;
        const int rows = n < kv->seq[L] ? n : kv->seq[L];
        const size_t bytes = (size_t)rows * kv->kv_dim[L] * 2;
        HIP_TRY(hipMemcpyAsync(kv->k[L], kv->px_k[L], bytes, hipMemcpyDeviceToDevice, kv->m->stream));
        HIP_TRY(hipMemcpyAsync(kv->v[L], kv->px_v[L], bytes, hipMemcpyDeviceToDevice, kv->m->stream));
    }
    return 0;
}

// ---- launching --------------------------------------------------------------------------------
static size_t lds_mm(int M, int k) { return (size_t)M * k + (size_t)M * (k / 32) * 8; }
// lg_k_attn: queries of the G heads, K and V tiles, exponentials; with the q/k/v preparation fused in, a head
// vector of staging per wavefront (16-byte aligned)
static size_t attn_lds(int G, int hd, bool fused_post) {
    const size_t b = (size_t)G * hd * 4 + (size_t)2 * 32 * (hd + 8) * 2 + (size_t)G * 32 * 4 + (size_t)G * 4;
    return fused_post ? ((b + 15) & ~(size_t)15) + (size_t)(LG_WG / 64) * hd * 4 : b;
}

// Kernels that want more than the default dynamic LDS limit have it raised once per (device, kernel, size).  What
// has been raised is kept in a fixed table (open addressing on the kernel's address; nothing is allocated, so a
// look-up is safe on a path that promises not to allocate); a kernel that finds no free slot has its limit set on
// every call, which costs time and nothing else.
struct LdsRaised { const void *fn; int dev; size_t bytes; };
static LdsRaised g_lds_raised[1024];
static std::mutex g_lds_mu;
template <typename K>
static int set_lds(K kernel, size_t bytes) {
    if (bytes <= 48 * 1024) return 0;
    if (bytes > 160 * 1024) return fail(-8, "kernel needs %zu bytes of LDS (160 KiB per workgroup)", bytes);
    const void *fn = reinterpret_cast<const void *>(kernel);
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(g_lds_mu);
    const size_t n = sizeof(g_lds_raised) / sizeof(g_lds_raised[0]);
    size_t at = ((uintptr_t)fn >> 4) * 0x9E3779B97F4A7C15ull >> 54;          // 10 bits
    LdsRaised *slot = nullptr;
    for (size_t probe = 0; probe < 32; ++probe, at = (at + 1) % n) {
        LdsRaised &e = g_lds_raised[at];
        if (!e.fn || (e.fn == fn && e.dev == dev)) { slot = &e; break; }
    }
    if (slot && slot->fn && slot->bytes >= bytes) return 0;
    HIP_TRY(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
    if (slot) { slot->fn = fn; slot->dev = dev; slot->bytes = bytes; }
    return 0;
}

struct Launcher {
    lg_hip_model *m;
    bool dry;              // only raise LDS limits, launch nothing (done once before a capture)
    int rc = 0;
    bool side = false;     // launches go to the model's second stream (the forked branch of a step)
    hipStream_t stream() const { return side ? m->stream2 : m->stream; }
    // per-class timing: an event pair that the launch itself fills in (begin and end of the kernel's own execution,
    // what a kernel trace reports; a pair recorded around the launch also counts the packet handling, ~1.5 us)
    bool events(int cls, hipEvent_t *a, hipEvent_t *b) {
        if (rc) return false;
        if (hipEventCreate(a) != hipSuccess || hipEventCreate(b) != hipSuccess) { rc = fail(-9, "event create failed"); return false; }
        m->prof.ev.push_back(*a); m->prof.ev.push_back(*b); m->prof.cls.push_back(cls);
        return true;
    }
    void end() {
        if (!rc) { hipError_t e = hipGetLastError(); if (e != hipSuccess) rc = fail(-100 - (int)e, "kernel launch failed: %s", hipGetErrorString(e)); }
    }
};
// (the kernel's parameter types come from the kernel, the arguments are converted to them one by one)
template <typename... P, typename... A>
static void launch_timed(void (*kernel)(P...), dim3 grid, dim3 block, size_t lds, hipStream_t st, hipEvent_t e0, hipEvent_t e1, A &&...a) {
    hipExtLaunchKernelGGL(kernel, grid, block, (uint32_t)lds, st, e0, e1, 0, static_cast<P>(a)...);
}

#define LAUNCH(cls, kernel, grid, block, lds, ...) do { if (!lx.rc) { lx.rc = set_lds(kernel, lds); } if (!lx.rc && !lx.dry) { \
    if (lx.m->prof.on) { hipEvent_t e0_, e1_; if (lx.events(cls, &e0_, &e1_)) launch_timed(kernel, grid, block, lds, lx.stream(), e0_, e1_, __VA_ARGS__); } \
    else hipLaunchKernelGGL(kernel, grid, block, lds, lx.stream(), __VA_ARGS__); \
    lx.end(); } } while (0)

// Compute units of the current device (asked once).
static int cu_count() {
    static int n = -1;
    if (n < 0) {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) v = 0;
        n = v;
    }
    return n;
}

// Plain matmul launch: picks the segment count from k and the workgroup shape from the row count
// (small matrices get one wavefront per workgroup so that every CU has work).
template <int M, bool DUMP>
static int launch_mm(Launcher &lx, int cls, const MmArgs &a_in, bool slabs_ok = false) {
    MmArgs a = a_in;                                      // (+ the workgroup size of the launch, set below)
    const int S = lg_segments(a.k), rw = 64 / S, ngroups = a.m / rw;
    if constexpr (M > LG_HIP_MAX_ROWS) {                 // wide (prefill) block: matrix-core kernels, 32 weight rows per workgroup
        if (a.m % 32) { lx.rc = fail(-2, "wide matmul: %d rows is not a multiple of 32", a.m); return 1; }
        // S = 32: four workgroups per row block, each a quarter of the K segments, writing its own slab of a.out
        const dim3 grid(a.m / 32, (M + LG_WIDE - 1) / LG_WIDE, S == 32 ? 4 : 1);
        if (S == 32) LAUNCH(cls, (lg_k_mm_wide<M, 32, DUMP>), grid, dim3(LG_WIDE_WG), MfmaGeo::lds_bytes, a, M);
        else         LAUNCH(cls, (lg_k_mm_wide<M, 8, DUMP>), grid, dim3(LG_WIDE_WG), MfmaGeo::lds_bytes, a, M);
        return S == 32 ? 4 : 1;
    } else {
    const size_t lds = lds_mm(M, a.k);
    if (S == 32 && M >= 4 && slabs_ok && !DUMP) {
        // blocks of four and more rows whose consumer adds four slabs: cut by K quarter (a quarter of the activations
        // per workgroup, several workgroups per CU).  12B shape, 5 rows: ffn_down 16.9 -> 14.3 us, the rows kernel that
        // adds the slabs 6.6 -> 7.5 us, the step 3.814 -> 3.775 ms (2 and 5 wavefronts per workgroup: 3.827, 3.924)
        if constexpr (M >= 4 && M <= LG_HIP_MAX_ROWS) {
            const int oct = (a.m + 7) / 8, W = 4;
            a.nthreads = 64 * W;
            LAUNCH(cls, (lg_k_mm_kq<M>), dim3((oct + W - 1) / W, 4), dim3(64 * W), (size_t)M * (a.k / 1024) * 320, LG_MM_FIELDS(LG_XA, a) 0);
        }
        return 4;
    } else if (S == 32) {
        // 4 wavefronts (8 rows) per workgroup, or 5 when that makes exactly one workgroup per CU (2560 rows on 256 CUs):
        // with 320 workgroups a quarter of the CUs would hold two of them and the kernel would wait for those
        const int cus = cu_count();
        const int W = (ngroups % 5 == 0 && ngroups / 5 <= cus && ngroups / 4 > cus) ? 5 : 4;
        // chunks of four tiles for the longest rows (15 tiles per lane at k = 15360: 3.96 against 4.00 ms per step at
        // the 12B shape), of two otherwise (10 tiles at k = 10240: 2.602 against 2.618 ms at the E4B shape)
        a.nthreads = 64 * W;
        if ((a.k >> 5) / 32 >= 12) LAUNCH(cls, (lg_k_mm<M, 32, 1, DUMP, 4>), dim3((ngroups + W - 1) / W), dim3(64 * W), lds, LG_MM_FIELDS(LG_XA, a) 0);
        else                       LAUNCH(cls, (lg_k_mm<M, 32, 1, DUMP>), dim3((ngroups + W - 1) / W), dim3(64 * W), lds, LG_MM_FIELDS(LG_XA, a) 0);
    } else if (ngroups >= 4096) {
        const int W = 4;
        a.nthreads = 64 * W;
        LAUNCH(cls, (lg_k_mm<M, 8, 2, DUMP>), dim3((ngroups + 2 * W - 1) / (2 * W)), dim3(64 * W), lds, LG_MM_FIELDS(LG_XA, a) 0);
    } else if (M >= 4 && a.k >= 2048 && !DUMP) {
        // blocks of four and more rows: two row groups per workgroup, the tiles of each cut over two wavefronts
        // (over four was no faster at 8 and 10 tiles per group)
        if constexpr (M >= 4 && M <= LG_HIP_MAX_ROWS) {
            const size_t l2 = ((lds + 15) & ~(size_t)15) + (size_t)2 * M * 64 * 4;
            // (over four wavefronts from 12 tiles per group on: 12B shape, k = 3840 and 4096, 3.662 -> 3.645 ms per step)
            a.nthreads = (a.k >> 8) >= 12 ? 512 : 256;
            if ((a.k >> 8) >= 12) LAUNCH(cls, (lg_k_mm_ks<M, 4>), dim3((ngroups + 1) / 2), dim3(512), l2, LG_MM_FIELDS(LG_XA, a) 0);
            else                  LAUNCH(cls, (lg_k_mm_ks<M, 2>), dim3((ngroups + 1) / 2), dim3(256), l2, LG_MM_FIELDS(LG_XA, a) 0);
        }
    } else {
        // Two row groups per workgroup when there are very many groups, and for blocks of 4+ rows when one group per
        // workgroup would leave some CUs with two of them: their activations (16 KB at M = 5) are then staged twice
        // on the CUs that set the kernel's time.  (Short rows, k < 1024, have too little to stage for that to matter.)
        const int W = (ngroups >= 1024 || (M >= 4 && a.k >= 1024 && ngroups > cu_count())) ? 2 : 1;
        a.nthreads = 64 * W;
        LAUNCH(cls, (lg_k_mm<M, 8, 1, DUMP>), dim3((ngroups + W - 1) / W), dim3(64 * W), lds, LG_MM_FIELDS(LG_XA, a) 0);
    }
    }
    (void)rw; (void)ngroups;
    return 1;
}

// one block of M rows through the decoder (and the head when with_head)
// f32-weight matmul of a block of M rows: one wavefront per weight row, 8 block rows per workgroup row
template <int M>
static void launch_mmf(Launcher &lx, int cls, const MmfArgs &a) {
    constexpr int MC = M < 8 ? M : 8;
    LAUNCH(cls, (lg_k_mmf<MC>), dim3((a.m + LG_WG / 64 - 1) / (LG_WG / 64), (a.rows + MC - 1) / MC), dim3(LG_WG), 0, a);
}
static bool attention_rows_shared(int rows, int tiles, int nkv, int hd, int seq) {
    return rows > 1 && rows <= LG_HIP_MAX_ROWS && hd <= 256 && seq >= 32 && tiles * nkv >= 256;
}
// tiles per workgroup of lg_k_attn_rows: one, until the grid would exceed the three workgroups per CU that the
// staged tile's LDS lets a CU hold; then as many as bring it back under that (at most four), each tile's rows in
// flight while the tile before it is computed
static int attention_rows_tp(int tiles, int nkv) {
    const int tp = (tiles * nkv + 3 * 256 - 1) / (3 * 256);
    return tp < 1 ? 1 : tp > 4 ? 4 : tp;
}

// lg_k_attn_u (prompt blocks, queries in registers, a wavefront per (row, head) unit, 8 units per workgroup): rows of
// the block per workgroup, 0 when the shape does not fit
static int attention_u_rows(int rows, int G, int hd, int seq) {
    if (rows <= LG_HIP_MAX_ROWS || seq < 32 || (hd != 64 && hd != 128 && hd != 256 && hd != 512)) return 0;
    if (G < 1 || G > 8 || 8 % G) return 0;
    const int rw = 8 / G;
    return rows % rw == 0 ? rw : 0;
}
// launch geometry: tiles a row group can touch, tiles per workgroup (so that the grid has about two workgroups per CU)
template <typename L>
static int attention_u_launch(L &&launch, int rows, int rw, int nkv, int hd, int window, int block_tiles) {
    int nt = block_tiles;
    if (window > 0) { const int t = (window + rw - 1 + 31) / 32 + 1; if (t < nt) nt = t; }
    const int groups = rows / rw;
    int tp = (int)(((long long)nt * nkv * groups + 511) / 512);
    if (tp < 1) tp = 1;
    if (tp > nt) tp = nt;
    const dim3 grid((nt + tp - 1) / tp, nkv, groups);
    switch (hd) {
        case 512: return launch(lg_k_attn_u<512>, grid, AttnUGeo<512>::bytes(8), tp);
        case 256: return launch(lg_k_attn_u<256>, grid, AttnUGeo<256>::bytes(8), tp);
        case 128: return launch(lg_k_attn_u<128>, grid, AttnUGeo<128>::bytes(8), tp);
        default:  return launch(lg_k_attn_u<64>, grid, AttnUGeo<64>::bytes(8), tp);
    }
}

// the XCD-partitioned feed-forward launch: 256 workgroups of 512 threads, the instantiation of the shape's class
template <int M>
static void launch_xffn(Launcher &lx, const XffnArgs &a, int cls) {
    if constexpr (M >= 4 && M <= LG_HIP_MAX_ROWS) {
        const size_t lds = xffn_lds(lg_xffn_geo(a.E, a.FF), M);
        switch (cls) {
            case 0: LAUNCH(KC_FFN, (lg_k_ffn_xcd<M, 1, 2, 1, 8, 8>), dim3(256), dim3(LG_XFFN_THREADS), lds, LG_XFFN_FIELDS(LG_XA, a) 0); break;
            case 1: LAUNCH(KC_FFN, (lg_k_ffn_xcd<M, 3, 10, 2, 10, 40>), dim3(256), dim3(LG_XFFN_THREADS), lds, LG_XFFN_FIELDS(LG_XA, a) 0); break;
            case 2: LAUNCH(KC_FFN, (lg_k_ffn_xcd<M, 4, 15, 2, 15, 60>), dim3(256), dim3(LG_XFFN_THREADS), lds, LG_XFFN_FIELDS(LG_XA, a) 0); break;
            default: lx.rc = fail(-2, "ffn_xcd: no instantiation for this shape");
        }
    }
}

// The per-layer-input block of a verify block of `rows` rows as the one-XCD launch lg_k_ple_tail: q4_0 matrices of the
// 256-wide per-layer input, at most LG_XTAIL_UNITS (gate block, row) units, a chip whose workgroups are dealt over 8 XCDs
static bool use_ple_tail(const lg_hip_model *m, int rows) {
    if (!m->ple || !m->tsync || m->xcd_tail <= 0 || m->target || rows < 1 || rows > LG_HIP_MAX_ROWS) return false;
    if (m->ple != 256 || (m->ple / 32) * rows > LG_XTAIL_UNITS || m->E % 256 || m->E > 4096 || (m->E + 1023) / 1024 > m->ple / 32) return false;
    const int U = (m->ple / 32) * rows;
    const bool spread = m->tail_spread && (rows >= 5 || rows <= 2);   // (lg_k_ple_tail_s: 8 wavefronts per unit, enough of them at every width)
    // blocks of one and two rows: with lg_k_ple_tail_s the tail beats folding the next layer's row work into its q/k/v
    // matmul (E4B shape: 1.994 -> 1.958 ms at one row, 2.127 -> 2.032 at two); with lg_k_ple_tail alone it does not
    if (m->xcd_tail == 1 && rows <= LG_FUSE_ROWS_MAX && m->fuse_rows && !spread) return false;
    if (!spread && (m->E / 8 + 4 * U - 1) / (4 * U) > 4) return false;       // (few rows of a wide model: too few wavefronts for the projection)
    return cu_count() == LG_XCDS * LG_XCD_WGS;
}
// Slices of the E output rows per (head, row) of lg_k_merge_o: a divisor of the E/64 chunks that leaves at most two
// chunks per wavefront, the largest that keeps the launch within one workgroup per CU (else the smallest)
static int merge_o_slices(const lg_hip_model *m, int rows) {
    const int chunks = m->E / 64;
    int best = 0, least = 0;
    for (int d = 1; d <= chunks; ++d) {
        if (chunks % d || (chunks / d + 3) / 4 > 2) continue;
        if (!least) least = d;
        if (8 * rows * d <= cu_count()) best = d;
    }
    const int pick = best ? best : least;
    if (m->merge_o_slices > 0 && chunks % m->merge_o_slices == 0 && (chunks / m->merge_o_slices + 3) / 4 <= 2) return m->merge_o_slices;
    return pick;
}
static bool use_merge_o(const lg_hip_model *m, const Layer &y, int rows, int tiles) {
    if (!y.wo_rb || m->merge_o <= 0 || rows > LG_HIP_MAX_ROWS || (m->merge_o == 1 && rows < 3)) return false;
    return tiles < 128 && merge_o_slices(m, rows) > 0;
}
static void launch_merge_o(Launcher &lx, const MergeOArgs &a) {
    const int nit = a.g.hd / 32, rpl = ((a.E / 64) / a.slices + 3) / 4;
    const dim3 grid(a.rows * a.g.H * a.slices);
#define CASE(N, R) if (nit == N && rpl == R) { LAUNCH(KC_MERGE, (lg_k_merge_o<N, R>), grid, dim3(LG_WG), 0, lx.m->ctl, LG_MERGEO_FIELDS(LG_XA, a) 0); return; }
    CASE(2, 1) CASE(2, 2) CASE(4, 1) CASE(4, 2) CASE(8, 1) CASE(8, 2) CASE(16, 1) CASE(16, 2)
#undef CASE
    lx.rc = fail(-2, "merge_o: no instantiation for head_dim %d with %d chunks per wavefront", a.g.hd, rpl);
}

template <int M>
static void launch_down_m(Launcher &lx, const DownMArgs &a) {
    if constexpr (M >= 4 && M <= LG_HIP_MAX_ROWS) {
        const DownMGeo g = lg_down_m_geo(a.E, a.FF);
        const size_t lds = (size_t)8 * g.nitd * (LG_MU_DWORDS * 4) + (size_t)8 * g.ops * 8 * 32 * 4;
        if (g.ops == 1 && g.npairs <= 3) LAUNCH(KC_DOWN, (lg_k_down_m<M, 1, 3>), dim3(256), dim3(512), lds, LG_DOWNM_FIELDS(LG_XA, a) 0);
        else if (g.ops == 2 && g.npairs <= 5) LAUNCH(KC_DOWN, (lg_k_down_m<M, 2, 5>), dim3(256), dim3(512), lds, LG_DOWNM_FIELDS(LG_XA, a) 0);
        else if (g.ops == 2 && g.npairs <= 8) LAUNCH(KC_DOWN, (lg_k_down_m<M, 2, 8>), dim3(256), dim3(512), lds, LG_DOWNM_FIELDS(LG_XA, a) 0);
        else lx.rc = fail(-2, "down_m: no instantiation for this shape");
    }
}
static bool use_attn_tail(const lg_hip_model *m, const Layer &y, int rows, int tiles) {
    if (!y.wo_ch || !m->tsync || m->xcd_attn_tail <= 0 || rows > LG_HIP_MAX_ROWS || (m->xcd_attn_tail == 1 && rows < 3)) return false;
    const int slices = (m->E + 1023) / 1024;
    return tiles < 128 && m->H * rows <= 2 * LG_XCD_WGS && slices * rows <= LG_XCD_WGS && y.hd % 32 == 0 && y.hd <= 256;
}
template <int M>
static void launch_attn_tail(Launcher &lx, const XattnTailArgs &a) {
    if constexpr (M <= LG_HIP_MAX_ROWS) {
        lg_hip_model *m = lx.m;
        int np = 0, rb = 0;
        if (!attn_tail_shape(a.g.H * a.g.hd, a.E, &np, &rb)) { lx.rc = fail(-2, "attn_tail: no instantiation for this shape"); return; }
        const size_t lds = (size_t)(16 * np) * LG_MU_DWORDS * 4 + (size_t)8 * rb * 8 * 32 * 4;
        const dim3 grid(LG_XCDS * LG_XCD_WGS);
        if (np == 1 && rb == 1) LAUNCH(KC_ATAIL, (lg_k_attn_tail<M, 1, 1>), grid, dim3(512), lds, m->ctl, LG_XATTN_FIELDS(LG_XA, a) 0);
        else if (np == 2 && rb == 1) LAUNCH(KC_ATAIL, (lg_k_attn_tail<M, 2, 1>), grid, dim3(512), lds, m->ctl, LG_XATTN_FIELDS(LG_XA, a) 0);
        else LAUNCH(KC_ATAIL, (lg_k_attn_tail<M, 4, 3>), grid, dim3(512), lds, m->ctl, LG_XATTN_FIELDS(LG_XA, a) 0);
    }
}

template <int M>
static void launch_ple_tail(Launcher &lx, const XtailArgs &a) {
    if constexpr (M <= LG_HIP_MAX_ROWS) {
        // 5..8 rows: the form whose units fit one per CU (row j by 32 / M workgroups of 8 wavefronts); 1 and 2 rows: the
        // form that has enough wavefronts for the projection
        lg_hip_model *m = lx.m;
        const int E = a.r.g.k, W = M * (32 / M), G = (E / 8 + 8 * W - 1) / (8 * W);
        if ((m->tail_spread == 2 || (m->tail_spread && (M >= 5 || M <= 2))) && a.gf && a.r.g.ple == 256 && G >= 1 && G <= 3) {
            const size_t lds = (size_t)E * 5 / 4 + (size_t)M * a.r.g.ple * 5 / 4;
            const dim3 grid(LG_XCDS * W);
            static int fits[4] = { 0, 0, 0, 0 };              // per G: 0 unknown, 1 yes, -1 no (asked once, outside any capture)
            if (!fits[G]) {
                int per_cu = 0;
                hipError_t e = hipErrorInvalidValue;
                switch (G) {
                    case 1: e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, lg_k_ple_tail_s<M, 1>, 512, lds); break;
                    case 2: e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, lg_k_ple_tail_s<M, 2>, 512, lds); break;
                    case 3: e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, lg_k_ple_tail_s<M, 3>, 512, lds); break;
                }
                fits[G] = (e == hipSuccess && per_cu * LG_XCD_WGS >= W) ? 1 : -1;
            }
            if (fits[G] > 0) {
                switch (G) {
                    case 1: LAUNCH(KC_TAIL, (lg_k_ple_tail_s<M, 1>), grid, dim3(512), lds, m->ctl, LG_XTAIL_FIELDS(LG_XA, a) 0); break;
                    case 2: LAUNCH(KC_TAIL, (lg_k_ple_tail_s<M, 2>), grid, dim3(512), lds, m->ctl, LG_XTAIL_FIELDS(LG_XA, a) 0); break;
                    case 3: LAUNCH(KC_TAIL, (lg_k_ple_tail_s<M, 3>), grid, dim3(512), lds, m->ctl, LG_XTAIL_FIELDS(LG_XA, a) 0); break;
                }
                return;
            }
        }
    }
    if constexpr (M <= LG_HIP_MAX_ROWS) {
        lg_hip_model *m = lx.m;
        const int E = a.r.g.k, U = (a.r.g.ple / 32) * M;
        const int G = (E / 8 + 4 * U - 1) / (4 * U);
        const size_t lds = (size_t)E * 5 / 4 + (size_t)M * a.r.g.ple * 5 / 4;
        const dim3 grid(LG_XCDS * U);
        // the U units wait for each other: all of them must be resident on the 32 CUs of one XCD at once
        static int fits[5] = { 0, 0, 0, 0, 0 };              // per G: 0 unknown, 1 yes, -1 no (asked once, outside any capture)
        if (G >= 1 && G <= 4 && !fits[G]) {
            int per_cu = 0;
            hipError_t e = hipErrorInvalidValue;
            switch (G) {
                case 1: e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, lg_k_ple_tail<M, 1>, LG_WG, lds); break;
                case 2: e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, lg_k_ple_tail<M, 2>, LG_WG, lds); break;
                case 3: e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, lg_k_ple_tail<M, 3>, LG_WG, lds); break;
                case 4: e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, lg_k_ple_tail<M, 4>, LG_WG, lds); break;
            }
            fits[G] = (e == hipSuccess && per_cu * LG_XCD_WGS >= U) ? 1 : -1;
        }
        if (G < 1 || G > 4 || fits[G] < 0) { lx.rc = fail(-2, "ple_tail: %d units of %d row groups per wavefront do not fit one XCD", U, G); return; }
        switch (G) {
            case 1: LAUNCH(KC_TAIL, (lg_k_ple_tail<M, 1>), grid, dim3(LG_WG), lds, m->ctl, LG_XTAIL_FIELDS(LG_XA, a) 0); break;
            case 2: LAUNCH(KC_TAIL, (lg_k_ple_tail<M, 2>), grid, dim3(LG_WG), lds, m->ctl, LG_XTAIL_FIELDS(LG_XA, a) 0); break;
            case 3: LAUNCH(KC_TAIL, (lg_k_ple_tail<M, 3>), grid, dim3(LG_WG), lds, m->ctl, LG_XTAIL_FIELDS(LG_XA, a) 0); break;
            case 4: LAUNCH(KC_TAIL, (lg_k_ple_tail<M, 4>), grid, dim3(LG_WG), lds, m->ctl, LG_XTAIL_FIELDS(LG_XA, a) 0); break;
            default: lx.rc = fail(-2, "ple_tail: %d row groups per wavefront", G);
        }
    }
}

template <int M>
static int enqueue_step(lg_hip_model *m, lg_hip_kv *kv, bool with_head, bool dry) {
    Launcher lx{ m, dry };
    const int E = m->E, H = m->H, nl = m->n_layer;
    int cur = 0;                                   // x[cur] holds the residual
    bool have_x = false;                           // false: rows are still token ids
    const float *pend_dout = nullptr, *pend_w = nullptr, *pend_os = nullptr;   // sub-layer output waiting to be added
    int pend_parts = 1;                            // 4 when that output is four slabs of partial sums (wide ffn_down)
    const bool draft = m->target != nullptr;
    const int pos_off = draft ? -1 : 0;            // a draft at pos sees the cache as a query at pos-1 (src/cuda/mtp-kernel.cuh:170-182)
    if (draft) {
        // x = pre . [embedding(token)*sqrt(nb), h_prev] (src/mtp.c:268-278); h_prev is the target's hidden of the
        // accepted row, or for a chained draft post . (this head's previous hidden) (src/cuda/mtp-kernel.cuh:372-389)
        const lg_hip_model *t = m->target;
        const int nb = t->E;
        if (m->draft_chain) {
            MmArgs a{ m->w_post, E, nb, m->hprev, m->hq, nullptr };
            launch_mm<M, false>(lx, KC_PMP, a);
        }
        DraftInArgs d{};
        d.emb = t->emb; d.emb_seg = lg_segments(nb); d.emb_nit = nb / 32 / d.emb_seg; d.emb_scale = sqrtf((float)nb);
        d.toks = m->sched; d.h_prev = m->draft_chain ? m->hprev : t->g_hidden; d.nb = nb; d.q = m->catq;
        LAUNCH(KC_ROWS, lg_k_draft_input, dim3((2 * nb / 4 + LG_WG - 1) / LG_WG), dim3(LG_WG), 0, d, m->ctl);
        MmArgs p{ m->w_pre, 2 * nb, E, m->x[0], m->catq, nullptr };
        launch_mm<M, false>(lx, KC_PMP, p);
        have_x = true;
    }

    // rows kernel: fold the pending sub-layer output into the residual, norm with w_pre, quantize
    auto rows = [&](const float *w_pre, float *h_out, int units = 0, int8_t *q_out = nullptr) {
        RowArgs s{};
        s.q_units = M <= LG_HIP_MAX_ROWS ? units : 0;
        s.E = E; s.eps = m->eps; s.toks = m->sched; s.q = q_out ? q_out : m->hq;
        if (!have_x) {
            s.emb = m->emb; s.emb_seg = lg_segments(E); s.emb_nit = E / 32 / s.emb_seg; s.emb_scale = sqrtf((float)E);
            if (m->rgsync) s.bump = &m->rgsync->base;          // the step's first kernel: a new range of epochs for lg_k_rows_geglu
        } else s.x = m->x[cur];
        s.dout = pend_dout; s.w_post = pend_w; s.os = pend_os; s.dparts = pend_parts;
        s.w_pre = w_pre; s.h_out = h_out;
        if (pend_dout || !have_x) s.x_out = m->x[cur ^ 1];
        // verify blocks: the tail of the row work (store, norm weight, q8) cut over one workgroup per float4 of a lane
        const int slices = M <= LG_HIP_MAX_ROWS ? (E + 1023) / 1024 : 1;
        s.slices = slices;
        LAUNCH(KC_ROWS, (lg_k_rows<M>), dim3(M, slices), dim3(LG_WG), 0, m->ctl, LG_ROW_FIELDS(LG_XA, s) 0);
        if (s.x_out) cur ^= 1;
        have_x = true; pend_dout = pend_w = pend_os = nullptr; pend_parts = 1;
    };

    // The same row work done by the workgroups of the matmul that consumes it (lg_fused.h): verify-width blocks
    // whose residual is already in memory.  NV = float4 per lane of a row.
    const int NVr = (E + 1023) / 1024;
    // (blocks of one or two rows: wider ones pay more for the repeated row work than for the launch, see lg_fused.h)
    auto can_fuse = [&]() { return M <= LG_FUSE_ROWS_MAX && have_x && m->fuse_rows && pend_parts == 1; };
    auto row_work = [&](const float *w_pre) {
        RowWork r{ m->x[cur], pend_dout, pend_w, pend_os, m->x[cur ^ 1], w_pre, E, m->eps };
        return r;
    };
    auto row_work_done = [&]() {
        if (pend_dout) cur ^= 1;
        pend_dout = pend_w = pend_os = nullptr; pend_parts = 1;
    };
    auto rows_mm = [&](const float *w_pre, const MmArgs &a, int cls) {      // rows(w_pre) then an 8-segment matmul of the result
        if constexpr (M <= LG_FUSE_ROWS_MAX) {
            constexpr int NW = 1;
            RowsMmArgs f{ a, row_work(w_pre) };
            const dim3 grid((a.m / 8 + NW - 1) / NW);
            const size_t lds = lds_mm(M, a.k);
            switch (NVr) {
                case 1: LAUNCH(cls, (lg_k_rows_mm<M, 1, NW>), grid, dim3(LG_WG), lds, LG_ROWSMM_FIELDS(LG_XA, f) 0); break;
                case 2: LAUNCH(cls, (lg_k_rows_mm<M, 2, NW>), grid, dim3(LG_WG), lds, LG_ROWSMM_FIELDS(LG_XA, f) 0); break;
                case 3: LAUNCH(cls, (lg_k_rows_mm<M, 3, NW>), grid, dim3(LG_WG), lds, LG_ROWSMM_FIELDS(LG_XA, f) 0); break;
                default: LAUNCH(cls, (lg_k_rows_mm<M, 4, NW>), grid, dim3(LG_WG), lds, LG_ROWSMM_FIELDS(LG_XA, f) 0); break;
            }
            row_work_done();
        }
    };

    const bool tail = use_ple_tail(m, M);
    bool rows_done = false;                        // the row work ahead of the next matmul has been done by the launch before it
    bool join_ple = false;                         // the forked branch has to be waited for before its result is used
    if (m->ple) {
        rows(nullptr, nullptr, 0, m->eq);
        // the per-layer inputs are not needed before layer 0's per-layer gate: they run on the second stream, beside
        // layer 0's attention and feed-forward (captured, the graph gets a second branch)
        const bool fork = m->fork_ple && !dry && !m->prof.on && m->stream2 && !lx.rc;
        if (fork) {
            hipError_t e = hipEventRecord(m->ev_fork, m->stream);
            if (e == hipSuccess) e = hipStreamWaitEvent(m->stream2, m->ev_fork, 0);
            if (e != hipSuccess) lx.rc = fail(-100 - (int)e, "fork of the per-layer input branch: %s", hipGetErrorString(e));
            lx.side = true;
        }
        if (m->pmp_f) {                                       // kept in a float type: the f32 rows themselves are the input
            MmfArgs f{ m->pmp_f, E, m->ple * nl, m->x[cur], E, M, m->pmp_raw, m->ple * nl, nullptr, 0 };
            launch_mmf<M>(lx, KC_PMP, f);
        } else {
        MmArgs a{ m->pmp, E, m->ple * nl, m->pmp_raw, m->eq, nullptr };
        launch_mm<M, false>(lx, KC_PMP, a);
        }
        IplArgs i{ m->pmp_raw, m->ple, nl, M, m->proj_norm, m->pte, m->sched,
                   1.0f / sqrtf((float)E), sqrtf((float)m->ple), 1.0f / sqrtf(2.0f), m->eps };
        LAUNCH(KC_PMP, lg_k_ipl, dim3(nl, M), dim3(64), 0, i, m->ctl);
        if (fork) {
            lx.side = false;
            hipError_t e = hipEventRecord(m->ev_join, m->stream2);
            if (e != hipSuccess && !lx.rc) lx.rc = fail(-100 - (int)e, "fork of the per-layer input branch: %s", hipGetErrorString(e));
            join_ple = true;
        }
    }
    auto join = [&]() {
        if (!join_ple) return;
        join_ple = false;
        hipError_t e = hipStreamWaitEvent(m->stream, m->ev_join, 0);
        if (e != hipSuccess && !lx.rc) lx.rc = fail(-100 - (int)e, "join of the per-layer input branch: %s", hipGetErrorString(e));
    };
    // tiles a block of layer L can touch (a sliding layer needs only its window's, not the cache's), and whether the
    // layer takes the kernel that serves all rows of a block per (tile, kv head)
    auto layer_tiles = [&](int L) {
        const Layer &y = m->L[L];
        const int window = (y.is_local && m->window > 0) ? m->window + pos_off : 0;
        int tiles = kv->tiles_max;
        if (window > 0) { const int t = (window + M - 1 + 31) / 32 + 1; if (t < tiles) tiles = t; }
        return tiles;
    };
    auto rows_shared = [&](int L) {
        const Layer &y = m->L[L];
        return pos_off == 0 && m->attn_rows && attention_rows_shared(M, layer_tiles(L), y.nkv, y.hd, kv->seq[y.src]);
    };
    for (int L = 0; L < nl && !lx.rc; ++L) {
        const Layer &y = m->L[L];
        const int window = (y.is_local && m->window > 0) ? m->window + pos_off : 0;
        bool fused_post = false, merged_o = false, ffn_rows_done = false;
        {   // q/k/v projections, then per-head norm, rotary and the K/V rows of this block
            MmArgs a{ y.wqkv, E, y.qkv_m, m->qkv, m->hq, nullptr };
            if (rows_done) { launch_mm<M, false>(lx, KC_QKV, a); rows_done = false; }      // (the previous layer's tail did this layer's row work)
            else if (can_fuse()) rows_mm(y.attn_norm, a, KC_QKV);
            else { rows(y.attn_norm, nullptr); launch_mm<M, false>(lx, KC_QKV, a); }
            // blocks of the model itself, up to LG_HIP_MAX_ROWS rows: the attention kernel does this part as well
            fused_post = M <= LG_HIP_MAX_ROWS && (pos_off == 0 || !y.owns);    // (a draft head's layers own no cache: queries only)
            // ... unless the layer has so many (tile, kv head) pairs that one workgroup per pair can serve all rows of
            // the block against one staged tile (long global contexts, wide windows): the rows then arrive prepared
            // (that kernel prepares them itself while it has few workgroups: each of them repeats the preparation of its kv
            // head's queries, which a layer of many hundred workgroups pays for with more than the launch it saves: 12B
            // shape, 8192 keys, 688 workgroups: 36 -> 43 us; a 1024-key window, 272 workgroups: 11 -> 13.5 us against 4.2)
            if (rows_shared(L)) {
                const int tiles = layer_tiles(L), tp = attention_rows_tp(tiles, y.nkv);
                if (!m->attn_rows_fq || ((tiles + tp - 1) / tp) * y.nkv > 2 * cu_count()) fused_post = false;
            }
            QkvPostArgs p{};
            p.qkv = m->qkv; p.ld = y.qkv_m; p.k_off = y.k_off; p.v_off = y.v_off;
            p.H = H; p.nkv = y.nkv; p.hd = y.hd;
            p.q_norm = y.q_norm; p.k_norm = y.k_norm; p.rope_tab = y.rope_tab; p.rope_ff = y.rope_ff;
            p.q_rot = m->q_rot;
            p.kc = y.owns ? kv->k[L] : nullptr; p.vc = y.owns ? kv->v[L] : nullptr;
            p.seq = kv->seq[y.src]; p.kv_dim = y.kd; p.eps = m->eps;
            if (!fused_post) LAUNCH(KC_QKVPOST, lg_k_qkv_post, dim3(H + (y.owns ? 2 * y.nkv : 0), M), dim3(64), 0, p, m->ctl);
        }
        {   // attention tiles + merge
            const int G = H / y.nkv;
            AttnArgs a{};
            a.q = m->q_rot; a.H = H; a.nkv = y.nkv; a.hd = y.hd;
            a.kc = kv->k[y.src]; a.vc = kv->v[y.src]; a.seq = kv->seq[y.src]; a.kv_dim = y.kd; a.window = window;
            a.pm = kv->pm; a.pl = kv->pl; a.pacc = kv->pacc; a.tiles_max = kv->tiles_max; a.pos_off = pos_off;
            const int tiles = layer_tiles(L);
            a.gx = tiles; a.gz = M;
            const bool shared = rows_shared(L);
            // prompt blocks (the queries arrive prepared: lg_k_qkv_post ran): eight (row, head) units per workgroup with the
            // queries in registers
            const int urows = (!fused_post && pos_off == 0 && m->attn_rows) ? attention_u_rows(M, G, y.hd, kv->seq[y.src]) : 0;
            if (urows) {
                attention_u_launch([&](auto kernel, dim3 grid, size_t lds, int tp) {
                    LAUNCH(KC_ATTN, kernel, grid, dim3(512), lds, a, m->ctl, urows, tp);
                    return 0;
                }, M, urows, y.nkv, y.hd, window, tiles);
            } else
            if (shared) {
                if constexpr (M > 1 && M <= LG_HIP_MAX_ROWS) {
                    const size_t lds = y.hd == 256 ? AttnRowsGeo<256>::bytes(M * G, fused_post) : y.hd == 128 ? AttnRowsGeo<128>::bytes(M * G, fused_post) : AttnRowsGeo<64>::bytes(M * G, fused_post);
                    const int tp = attention_rows_tp(tiles, y.nkv);
                    const dim3 grid((tiles + tp - 1) / tp, y.nkv);
                    if (fused_post) {
                        a.qkv = m->qkv; a.ld = y.qkv_m; a.k_off = y.k_off; a.v_off = y.v_off;
                        a.q_norm = y.q_norm; a.k_norm = y.k_norm; a.rope_tab = y.rope_tab; a.rope_ff = y.rope_ff;
                        a.kcw = y.owns ? kv->k[L] : nullptr; a.vcw = y.owns ? kv->v[L] : nullptr; a.eps = m->eps;
                        if (y.hd == 256)      LAUNCH(KC_ATTN, (lg_k_attn_rows<M, 256, true>), grid, dim3(LG_WG), lds, m->ctl, tp, LG_ATTN_FIELDS(LG_XA, a) 0);
                        else if (y.hd == 128) LAUNCH(KC_ATTN, (lg_k_attn_rows<M, 128, true>), grid, dim3(LG_WG), lds, m->ctl, tp, LG_ATTN_FIELDS(LG_XA, a) 0);
                        else                  LAUNCH(KC_ATTN, (lg_k_attn_rows<M, 64, true>), grid, dim3(LG_WG), lds, m->ctl, tp, LG_ATTN_FIELDS(LG_XA, a) 0);
                    } else
                    if (y.hd == 256)      LAUNCH(KC_ATTN, (lg_k_attn_rows<M, 256>), grid, dim3(LG_WG), lds, m->ctl, tp, LG_ATTN_FIELDS(LG_XA, a) 0);
                    else if (y.hd == 128) LAUNCH(KC_ATTN, (lg_k_attn_rows<M, 128>), grid, dim3(LG_WG), lds, m->ctl, tp, LG_ATTN_FIELDS(LG_XA, a) 0);
                    else                  LAUNCH(KC_ATTN, (lg_k_attn_rows<M, 64>), grid, dim3(LG_WG), lds, m->ctl, tp, LG_ATTN_FIELDS(LG_XA, a) 0);
                }
            } else
            if (fused_post) {
                a.qkv = m->qkv; a.ld = y.qkv_m; a.k_off = y.k_off; a.v_off = y.v_off;
                a.q_norm = y.q_norm; a.k_norm = y.k_norm; a.rope_tab = y.rope_tab; a.rope_ff = y.rope_ff;
                a.kcw = y.owns ? kv->k[L] : nullptr; a.vcw = y.owns ? kv->v[L] : nullptr; a.eps = m->eps;
                if (y.hd <= 256) LAUNCH(KC_ATTN, (lg_k_attn<true, 1>), dim3(tiles, y.nkv, M), dim3(LG_WG), attn_lds(G, y.hd, true), m->ctl, LG_ATTN_FIELDS(LG_XA, a) 0);
                else             LAUNCH(KC_ATTN, (lg_k_attn<true, 2>), dim3(tiles, y.nkv, M), dim3(LG_WG), attn_lds(G, y.hd, true), m->ctl, LG_ATTN_FIELDS(LG_XA, a) 0);
            } else {
                LAUNCH(KC_ATTN, (lg_k_attn<false, 1>), dim3(tiles, y.nkv, M), dim3(LG_WG), attn_lds(G, y.hd, false), m->ctl, LG_ATTN_FIELDS(LG_XA, a) 0);
            }
            MergeArgs g{ kv->pm, kv->pl, kv->pacc, kv->tiles_max, H, y.hd, window, pos_off, m->aq, nullptr };
            merged_o = pos_off == 0 && use_merge_o(m, y, M, tiles);
            if (pos_off == 0 && have_x && use_attn_tail(m, y, M, tiles)) {
                // merge, output projection and the row work ahead of gate/up as one launch on one XCD
                XattnTailArgs f{};
                f.g = g; f.wo = y.wo_ch; f.aq = (uint32_t *)m->aq; f.pout = m->dout;
                f.x = m->x[cur]; f.w_post = y.post_attn; f.w_pre = y.ffn_norm; f.x_out = m->x[cur ^ 1];
                f.q = m->hq; f.q_units = (M >= 4) ? 2 : 1; f.E = E; f.eps = m->eps;
                f.sync = m->tsync; f.spin_limit = 1 << 16; f.stamps = m->tail_stamps ? m->tstamps + LG_XTAIL_UNITS * 8 : nullptr;
                launch_attn_tail<M>(lx, f);
                cur ^= 1;
                pend_dout = pend_w = pend_os = nullptr; pend_parts = 1;
                merged_o = true; ffn_rows_done = true;
            } else
            if (merged_o) {
                // the merge of (head, row) runs that head's chain of the output projection itself: eight slabs for the row kernel
                MergeOArgs f{ g, y.wo_rb, m->dout, E, merge_o_slices(m, M), M };
                launch_merge_o(lx, f);
                pend_dout = m->dout; pend_w = y.post_attn; pend_os = nullptr; pend_parts = 8;
            } else
            if (M <= LG_HIP_MAX_ROWS && tiles >= 128 && y.hd % 64 == 0) LAUNCH(KC_MERGE, (lg_k_attn_merge_split<M>), dim3(H, M, y.hd / 64), dim3(LG_WG), 0, m->ctl, LG_MERGE_FIELDS(LG_XA, g) 0);
            else LAUNCH(KC_MERGE, (lg_k_attn_merge<M>), dim3(H, M), dim3(LG_WG), 0, m->ctl, LG_MERGE_FIELDS(LG_XA, g) 0);
        }
        if (!merged_o) {   // attention output projection
            MmArgs a{ y.wo, y.qd, E, m->dout, m->aq, nullptr };
            pend_parts = launch_mm<M, false>(lx, KC_O, a);      // (four slabs for a wide block when n_head * head_dim > 4096)
            pend_dout = m->dout; pend_w = y.post_attn; pend_os = nullptr;
        }
        {   // feed-forward: gate/up + GeGLU, then down
            // verify blocks: 1..3 rows through v_dot4 with scalar operands, 4..8 rows through the matrix cores
            // (its float work per tile does not grow with the row count); each has its own activation order
            constexpr bool mfma = M >= 4 && M <= LG_HIP_MAX_ROWS;
            if (mfma && m->xffn_built && m->xcd_ffn && y.xgu && have_x && pend_dout && pend_parts == 1 && !pend_os) {
                // the whole half as one launch partitioned by XCD: row work, gate/up + GeGLU and the XCD's K share of
                // ffn_down; the consumer adds the 8 slabs (the top of the segment tree)
                XffnArgs f{ y.xgu, y.xdn, m->x[cur], pend_dout, pend_w, y.ffn_norm, m->x[cur ^ 1], m->slabs, m->xq8, m->xact,
                            m->xsync, m->ctl, E, y.nff, m->eps, 1 << 18, m->xffn_delay, nullptr };
                launch_xffn<M>(lx, f, m->xffn_cls);
                cur ^= 1;
                pend_dout = m->slabs; pend_parts = LG_XCDS; pend_w = y.post_ffw; pend_os = m->ple ? nullptr : y.out_scale;
            } else {
            const bool dn_m = mfma && m->down_m && y.wdn_m;       // ffn_down on the matrix cores: the activations as 80-dword blocks
            GegluArgs a{ y.wgu, E, y.nff, m->hq, m->gq, dn_m ? 2 : 0 };
            bool rows_in_geglu = false;
            if constexpr (mfma) {
                // the row work as the first workgroups of the gate/up launch, whose other workgroups request their weights
                // while it runs (lg_xrg.h); shapes whose K segment of E/256 tiles has a build
                const int slices = (E + 1023) / 1024;
                if (m->rows_geglu && m->rgsync && !ffn_rows_done && have_x && pend_dout && !pend_os && (pend_parts == 1 || pend_parts == 4) && (E == 2560 || E == 3840 || E == 512) &&
                    M * slices <= LG_RG_MAXP && L < LG_RG_STEP - 1) {
                    RowsGegluArgs f{ m->x[cur], pend_dout, pend_w, y.ffn_norm, m->x[cur ^ 1], m->hq, E, pend_parts, slices, m->eps,
                                     y.wgu, y.nff, m->gq, dn_m ? 2 : 0, m->rgsync, L, 1 << 16, m->tail_stamps ? m->tstamps + LG_XTAIL_UNITS * 8 : nullptr };
                    const dim3 grid(M * slices + y.nff / 32);
                    const size_t lds = (size_t)(E / 32) * LG_MU_DWORDS * 4;
                    if (E == 512)  LAUNCH(KC_GATEUP, (lg_k_rows_geglu<M, 2>), grid, dim3(512), lds, m->ctl, LG_RG_FIELDS(LG_XA, f) 0);
                    else if (E == 2560) LAUNCH(KC_GATEUP, (lg_k_rows_geglu<M, 10>), grid, dim3(512), lds, m->ctl, LG_RG_FIELDS(LG_XA, f) 0);
                    else           LAUNCH(KC_GATEUP, (lg_k_rows_geglu<M, 15>), grid, dim3(512), lds, m->ctl, LG_RG_FIELDS(LG_XA, f) 0);
                    cur ^= 1;
                    pend_dout = pend_w = pend_os = nullptr; pend_parts = 1;
                    rows_in_geglu = true;
                }
            }
            if (rows_in_geglu) {
            } else {
            if (!ffn_rows_done) rows(y.ffn_norm, nullptr, mfma ? 2 : 1);
            if constexpr (M > LG_HIP_MAX_ROWS)
                LAUNCH(KC_GATEUP, (lg_k_mm_geglu_wide<M>), dim3(y.nff / 32, (M + LG_WIDE - 1) / LG_WIDE), dim3(LG_WIDE_WG), MfmaGeo::lds_bytes, a, M);
            else if constexpr (mfma)
                LAUNCH(KC_GATEUP, (lg_k_geglu_m<M>), dim3(y.nff / 32), dim3(512), (size_t)(E / 32) * LG_MU_DWORDS * 4, LG_GEGLU_FIELDS(LG_XA, a) 0);
            else
                LAUNCH(KC_GATEUP, (lg_k_geglu_t<M>), dim3(y.nff / 32), dim3(512), 0, LG_GEGLU_FIELDS(LG_XA, a) 0);
            }
            MmArgs d{ y.wdown, y.nff, E, m->dout, m->gq, nullptr };
            if (dn_m) {
                DownMArgs dm{ y.wdn_m, (const uint32_t *)m->gq, m->dout, E, y.nff, m->down_m == 1 ? m->dmsync : nullptr, m->ctl, 1 << 16 };
                launch_down_m<M>(lx, dm);
                pend_parts = dm.sync ? 1 : 4;
            } else
            // (the rows kernel adds four slabs; the fused rows + PLE gate kernel of verify blocks takes whole sums)
            pend_parts = launch_mm<M, false>(lx, KC_DOWN, d, !m->ple && m->down_kq);
            pend_dout = m->dout; pend_w = y.post_ffw; pend_os = m->ple ? nullptr : y.out_scale;
            }
        }
        if (m->ple) join();
        if (m->ple && y.winp_f) {   // per-layer embedding block, matrices kept in a float type: residual update, then the
            // gate on the f32 rows (gelu(.) * ipl in its epilogue), then the projection of the f32 gate rows
            rows(nullptr, nullptr);
            MmfArgs g{ y.winp_f, E, m->ple, m->x[cur], E, M, m->pgf, m->ple, m->pmp_raw + (size_t)L * m->ple, m->ple * nl };
            launch_mmf<M>(lx, KC_PLEGATE, g);
            MmfArgs p{ y.wproj_f, m->ple, E, m->pgf, m->ple, M, m->dout, E, nullptr, 0 };
            launch_mmf<M>(lx, KC_PLEPROJ, p);
            pend_dout = m->dout; pend_w = y.post_norm; pend_os = y.out_scale;
        } else
        if (m->ple) {   // per-layer embedding block
            PleGateArgs a{ y.winp, E, m->ple, m->hq, m->pmp_raw, L, nl, m->pq };
            if constexpr (M > LG_HIP_MAX_ROWS) {
                rows(nullptr, nullptr);
                LAUNCH(KC_PLEGATE, (lg_k_mm_plegate_wide<M>), dim3(m->ple / 32, (M + LG_WIDE - 1) / LG_WIDE), dim3(LG_WIDE_WG), MfmaGeo::lds_bytes, a, M);
            } else if (tail && (L + 1 < nl || with_head) && pend_dout && have_x && !pend_os) {
                // the whole block and the row work that follows it (the next layer's, or the head's) in one launch on one XCD
                const bool last = L + 1 == nl;
                const bool head_m = M >= 4 && m->emb_rb && m->head_mfma;
                XtailArgs f{};
                f.r = RowsPleGateArgs{ a, m->x[cur], pend_dout, pend_w, nullptr, m->eps, pend_parts };
                f.pw = y.wproj; f.pout = m->dout; f.w_post2 = y.post_norm; f.os = y.out_scale;
                f.w_pre = last ? m->output_norm : m->L[L + 1].attn_norm;
                f.x_out = m->x[cur ^ 1]; f.h_out = last ? m->hidden_rows : nullptr;
                f.q = m->hq; f.q_units = last && head_m ? 2 : 0;
                f.sync = m->tsync; f.spin_limit = 1 << 16; f.stamps = m->tail_stamps ? m->tstamps : nullptr;
                f.gf = m->tgf;
                launch_ple_tail<M>(lx, f);
                cur ^= 1;
                pend_dout = pend_w = pend_os = nullptr; pend_parts = 1;
                rows_done = true;
                continue;
            } else {
                // the residual update after ffn_down and its q8 happen inside the gate kernel (no rows kernel here)
                RowsPleGateArgs r{ a, m->x[cur], pend_dout, pend_w, m->x[cur ^ 1], m->eps, pend_parts };
                LAUNCH(KC_PLEGATE, (lg_k_rows_plegate<M>), dim3(m->ple / 32, M), dim3(LG_WG), lds_mm(1, E), LG_RPG_FIELDS(LG_XA, r) 0);
                cur ^= 1;
                pend_dout = pend_w = pend_os = nullptr; pend_parts = 1;
            }
            MmArgs p{ y.wproj, m->ple, E, m->dout, m->pq, nullptr };
            launch_mm<M, false>(lx, KC_PLEPROJ, p);
            pend_dout = m->dout; pend_w = y.post_norm; pend_os = y.out_scale;
        }
    }
    join();
    if constexpr (M > LG_HIP_MAX_ROWS) {
        if (with_head) return fail(-2, "a wide block has no head: verify blocks hold at most %d rows", LG_HIP_MAX_ROWS);
        if (!lx.rc && !dry) hipLaunchKernelGGL(lg_k_advance, dim3(1), dim3(1), 0, m->stream, m->ctl, M);
        return lx.rc;
    } else
    if (with_head && !lx.rc) {
        const bool head_m = M >= 4 && m->emb_rb && m->head_mfma;
        if (!rows_done) rows(m->output_norm, m->hidden_rows, head_m ? 2 : 0);
        int grid = 512;                                  // two workgroups per CU, each walks `passes` blocks of 64 rows
        int passes = (m->n_vocab / 64 + grid - 1) / grid;
        if (passes < 1) passes = 1;
        grid = (m->n_vocab / 64 + passes - 1) / passes;
        HeadArgs h{ head_m ? m->emb_rb : m->emb, E, m->n_vocab, passes, m->hq, m->softcap, m->store_logits ? m->logits : nullptr, m->pval, m->pidx };
        if (head_m) {
            if constexpr (M >= 4 && M <= LG_HIP_MAX_ROWS)
                LAUNCH(KC_HEAD, (lg_k_head_m<M>), dim3(grid), dim3(512), (size_t)(E / 32) * LG_MU_DWORDS * 4, LG_HEAD_FIELDS(LG_XA, h) 0);
        } else
        LAUNCH(KC_HEAD, (lg_k_mm_head<M>), dim3(grid), dim3(LG_WG), lds_mm(M, E), LG_HEAD_FIELDS(LG_XA, h) 0);
        AcceptArgs c{ m->pval, m->pidx, grid, m->sched, m->out, m->adv, m->hidden_rows, m->g_hidden, E };
        LAUNCH(KC_ACCEPT, (lg_k_accept<M>), dim3(1), dim3(LG_WG), 0, m->ctl, LG_ACCEPT_FIELDS(LG_XA, c) 0);
    } else if (!lx.rc && !dry) {
        hipLaunchKernelGGL(lg_k_advance, dim3(1), dim3(1), 0, m->stream, m->ctl, M);
    }
    return lx.rc;
}

static int enqueue_step_rows(lg_hip_model *m, lg_hip_kv *kv, int rows, bool with_head, bool dry = false) {
    switch (rows) {
        case 1: return enqueue_step<1>(m, kv, with_head, dry);
        case 2: return enqueue_step<2>(m, kv, with_head, dry);
        case 3: return enqueue_step<3>(m, kv, with_head, dry);
        case 4: return enqueue_step<4>(m, kv, with_head, dry);
        case 5: return enqueue_step<5>(m, kv, with_head, dry);
        case 6: return enqueue_step<6>(m, kv, with_head, dry);
        case 7: return enqueue_step<7>(m, kv, with_head, dry);
        case 8: return enqueue_step<8>(m, kv, with_head, dry);
        case LG_WIDE: return enqueue_step<LG_WIDE>(m, kv, with_head, dry);
        case LG_WIDE_MID: return enqueue_step<LG_WIDE_MID>(m, kv, with_head, dry);
        case LG_WIDE_ROWS: return enqueue_step<LG_WIDE_ROWS>(m, kv, with_head, dry);
    }
    return fail(-2, "rows %d outside 1..%d", rows, LG_HIP_MAX_ROWS);
}

// launch one step, through a captured graph when enabled
static int launch_step(lg_hip_model *m, lg_hip_kv *kv, int rows, bool with_head) {
    if (!m->use_graph || m->prof.on) return enqueue_step_rows(m, kv, rows, with_head);
    const std::string key = "kv" + std::to_string(kv->id) + ":" + std::to_string(rows) + (with_head ? "h" : "p") + (m->store_logits ? "l" : "") + (m->draft_chain ? "c" : "") + (m->fuse_rows ? "" : "u") + (m->attn_rows ? "" : "r") + (m->attn_rows_fq ? "" : "q") + (m->head_mfma ? "" : "s") + (m->down_kq ? "" : "d") + (m->xcd_ffn ? "x" + std::to_string(m->xffn_delay) : "") + (m->fork_ple ? "" : "f") + "t" + std::to_string(m->xcd_tail) + (m->tail_spread == 1 ? "" : m->tail_spread ? "N" : "n") + (m->rows_geglu ? "g" : "") + (m->tail_stamps ? "s" : "") + (m->down_m ? "D" + std::to_string(m->down_m) : "") + "a" + std::to_string(m->xcd_attn_tail) + "o" + std::to_string(m->merge_o) + "." + std::to_string(m->merge_o_slices);
    auto it = m->graphs.find(key);
    if (it == m->graphs.end()) {
        hipGraph_t graph = nullptr;
        hipGraphExec_t exec = nullptr;
        int rc = enqueue_step_rows(m, kv, rows, with_head, true);
        if (rc) return rc;
        HIP_TRY(hipStreamBeginCapture(m->stream, hipStreamCaptureModeThreadLocal));
        rc = enqueue_step_rows(m, kv, rows, with_head);
        hipError_t e = hipStreamEndCapture(m->stream, &graph);
        if (rc) { if (graph) (void)hipGraphDestroy(graph); return rc; }
        if (e != hipSuccess) return fail(-100 - (int)e, "hipStreamEndCapture: %s", hipGetErrorString(e));
        e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
        (void)hipGraphDestroy(graph);
        if (e != hipSuccess) return fail(-100 - (int)e, "hipGraphInstantiate: %s", hipGetErrorString(e));
        it = m->graphs.emplace(key, exec).first;
    }
    HIP_TRY(hipGraphLaunch(it->second, m->stream));
    return 0;
}

static int check_block(lg_hip_model *m, lg_hip_kv *kv, const int32_t *toks, int n, int rows, int pos, bool wide = false) {
    if (!m || !kv || !toks || kv->m != m) return fail(-1, "bad model / cache / token pointer");
    if (rows < 1 || (rows > m->max_rows && !(wide && (rows == LG_WIDE || rows == LG_WIDE_MID || rows == LG_WIDE_ROWS)))) return fail(-2, "block of %d rows; the model was committed for 1..%d", rows, m->max_rows);
    if (pos < 0 || pos + rows > kv->max_seq) return fail(-2, "positions %d..%d do not fit a cache of %d", pos, pos + rows - 1, kv->max_seq);
    for (int i = 0; i < n; ++i) if (toks[i] < 0 || toks[i] >= m->n_vocab) return fail(-2, "token id %d outside the vocabulary of %d", toks[i], m->n_vocab);
    return 0;
}

extern "C" int lg_hip_set_option(lg_hip_model *m, const char *name, int value) {
    if (!m || !name) return fail(-1, "set_option: null argument");
    if (!strcmp(name, "store_logits")) m->store_logits = value != 0;
    else if (!strcmp(name, "head_mfma")) m->head_mfma = value != 0;
    else if (!strcmp(name, "use_graph")) m->use_graph = value != 0;
    else if (!strcmp(name, "wide_prefill")) m->wide_prefill = value != 0;
    else if (!strcmp(name, "fuse_rows")) m->fuse_rows = value != 0;
    else if (!strcmp(name, "attn_rows")) m->attn_rows = value != 0;
    else if (!strcmp(name, "attn_rows_fq")) m->attn_rows_fq = value != 0;
    else if (!strcmp(name, "xcd_tail_spread")) m->tail_spread = value;
    else if (!strcmp(name, "rows_geglu")) m->rows_geglu = value != 0;
    else if (!strcmp(name, "down_kq")) m->down_kq = value != 0;
    else if (!strcmp(name, "xcd_ffn")) m->xcd_ffn = value != 0 && m->xffn_built;
    else if (!strcmp(name, "fork_ple")) m->fork_ple = value != 0;
    else if (!strcmp(name, "down_m")) m->down_m = value < 0 ? 0 : value > 2 ? 2 : value;
    else if (!strcmp(name, "xcd_attn_tail")) m->xcd_attn_tail = value < 0 ? 0 : value > 2 ? 2 : value;
    else if (!strcmp(name, "merge_o")) m->merge_o = value < 0 ? 0 : value > 2 ? 2 : value;
    else if (!strcmp(name, "merge_o_slices")) m->merge_o_slices = value < 0 ? 0 : value;
    else if (!strcmp(name, "xcd_tail")) m->xcd_tail = value < 0 ? 0 : value > 2 ? 2 : value;
    else if (!strcmp(name, "xcd_tail_stamps")) m->tail_stamps = value != 0;
    else if (!strcmp(name, "xcd_ffn_delay")) m->xffn_delay = value < 0 ? 0 : value > 0x3FF ? 0x3FF : value;
    else return fail(-2, "set_option: unknown option %s", name);
    return 0;
}

// What a kernel of a step left in StepCtl.err (a hand-over inside an XCD that was given up, or whose workgroups were not
// on one XCD): the step's results are not to be used.
static int step_err(const char *who, int err) {
    if (!err) return 0;
    return fail(-9, "%s: a kernel of the step reported %s%s(err 0x%x); its results are void", who,
                (err & LG_XFFN_ERR_PLACE) ? "workgroups of one group on different XCDs " : "",
                (err & LG_XFFN_ERR_WAIT) ? "a hand-over that was given up " : "", err);
}

static int load_block(lg_hip_model *m, const int32_t *toks, int rows, int pos) {
    StepCtl c{ pos, 0, 0, 0 };
    memcpy(m->pin, &c, sizeof c);
    memcpy(m->pin + 64, toks, (size_t)rows * 4);
    HIP_TRY(hipMemcpyAsync(m->ctl, m->pin, sizeof c, hipMemcpyHostToDevice, m->stream));
    HIP_TRY(hipMemcpyAsync(m->sched, m->pin + 64, (size_t)rows * 4, hipMemcpyHostToDevice, m->stream));
    return 0;
}

extern "C" int lg_hip_forward_spec(lg_hip_model *m, lg_hip_kv *kv, const int32_t *toks, int rows, int pos,
                                   int32_t *out, int32_t *adv) {
    int rc = check_block(m, kv, toks, rows, rows, pos);
    if (rc) return rc;
    if (!out || !adv) return fail(-1, "forward_spec: null output");
    HIP_TRY(hipSetDevice(m->device));
    if ((rc = load_block(m, toks, rows, pos))) return rc;
    if ((rc = launch_step(m, kv, rows, true))) return rc;
    HIP_TRY(hipMemcpyAsync(m->pin + 32, m->out, (size_t)rows * 4, hipMemcpyDeviceToHost, m->stream));
    HIP_TRY(hipMemcpyAsync(m->pin + 48, m->adv, 4, hipMemcpyDeviceToHost, m->stream));
    HIP_TRY(hipMemcpyAsync(m->pin + 56, m->ctl, sizeof(StepCtl), hipMemcpyDeviceToHost, m->stream));
    HIP_TRY(hipStreamSynchronize(m->stream));
    if ((rc = step_err("forward_spec", m->pin[58]))) return rc;
    memcpy(out, m->pin + 32, (size_t)rows * 4);
    *adv = m->pin[48];
    m->last_rows = rows; m->last_adv = *adv;
    return 0;
}

// ---- draft head ---------------------------------------------------------------------------------
extern "C" int lg_hip_draft_create(lg_hip_model *target, const struct lg_hip_config *c, lg_hip_model **out) {
    if (!target || !c || !out || !target->committed) return fail(-1, "draft_create: the target model must be committed first");
    if (target->target) return fail(-2, "draft_create: the target is itself a draft head");
    if (target->n_kv_start < 2) return fail(-2, "draft_create: the target needs a sliding and a global cache layer to read");
    if (c->n_embd_per_layer) return fail(-2, "draft_create: a draft head has no per-layer embedding");
    // the rounds kept on the device copy the head's tokens straight into the target's blocks: same vocabulary or none
    if (c->n_vocab != target->n_vocab) return fail(-2, "draft_create: the head's vocabulary (%d) is not the target's (%d)", c->n_vocab, target->n_vocab);
    lg_hip_model *m = nullptr;
    int rc = lg_hip_model_create(c, target->device, &m);
    if (rc) return rc;
    (void)hipStreamDestroy(m->stream);
    m->stream = target->stream;                    // same queue: a draft reads what the last verify step wrote
    m->owns_stream = false;
    m->target = target;
    m->window = target->window;
    m->n_kv_start = 0;
    target->drafts.push_back(m);
    *out = m;
    return 0;
}

extern "C" int lg_hip_draft_step(lg_hip_model *d, lg_hip_kv *kv, int token, int pos, int chain, int32_t *tok_out) {
    if (!d || !kv || !tok_out || !d->target || !d->committed || kv->m != d->target) return fail(-1, "draft_step: bad draft / cache pointer");
    const lg_hip_model *t = d->target;
    if (token < 0 || token >= t->n_vocab) return fail(-2, "draft_step: token id %d outside the target vocabulary of %d", token, t->n_vocab);
    if (pos < 1 || pos > kv->max_seq) return fail(-2, "draft_step: position %d (the cache must hold 1..%d positions before it)", pos, kv->max_seq);
    if (chain && !d->w_post) return fail(-4, "draft_step: this head has no post-projection, drafts cannot chain");
    if (d->H > t->max_rows * t->H) return fail(-2, "draft_step: %d draft heads do not fit the target's attention scratch", d->H);
    HIP_TRY(hipSetDevice(d->device));
    int rc;
    int32_t tk = token;
    if ((rc = load_block(d, &tk, 1, pos))) return rc;
    d->draft_chain = chain != 0;
    rc = launch_step(d, kv, 1, true);
    d->draft_chain = false;
    if (rc) return rc;
    HIP_TRY(hipMemcpyAsync(d->pin + 32, d->out, 4, hipMemcpyDeviceToHost, d->stream));
    HIP_TRY(hipStreamSynchronize(d->stream));
    *tok_out = d->pin[32];
    d->last_rows = 1; d->last_adv = 1;
    return 0;
}

// One speculative round with no host involvement: K = rows-1 drafts (the first from the target's hidden state, the
// others chained), the link kernels that move their tokens, and the verify step.
static int enqueue_round(lg_hip_model *d, lg_hip_kv *kv, int rows, bool dry) {
    lg_hip_model *t = d->target;
    LinkArgs a{ d->ctl, t->ctl, d->sched, d->out, t->sched, t->out, t->adv, rows, 0 };
    int rc = 0;
    for (int j = 1; j <= rows && !rc; ++j) {
        a.phase = j;
        if (!dry) hipLaunchKernelGGL(lg_k_link, dim3(1), dim3(1), 0, t->stream, a);
        if (j == rows) break;
        d->draft_chain = j > 1;
        rc = enqueue_step_rows(d, kv, 1, true, dry);
        d->draft_chain = false;
    }
    if (!rc) rc = enqueue_step_rows(t, kv, rows, true, dry);
    a.phase = 0;
    if (!rc && !dry) hipLaunchKernelGGL(lg_k_link, dim3(1), dim3(1), 0, t->stream, a);
    if (!rc && !dry) { hipError_t e = hipGetLastError(); if (e != hipSuccess) rc = fail(-100 - (int)e, "mtp_rounds: launch failed: %s", hipGetErrorString(e)); }
    return rc;
}

extern "C" int lg_hip_mtp_rounds(lg_hip_model *d, lg_hip_kv *kv, int token, int pos, int rows, int n_rounds,
                                 int32_t *blocks, int32_t *out, int32_t *adv, int32_t *final_pos) {
    if (!d || !kv || !d->target || !d->committed || kv->m != d->target) return fail(-1, "mtp_rounds: bad draft / cache pointer");
    lg_hip_model *t = d->target;
    if (!blocks || !out || !adv) return fail(-1, "mtp_rounds: null output");
    if (rows < 2 || rows > t->max_rows) return fail(-2, "mtp_rounds: blocks of %d rows; the target was committed for 2..%d", rows, t->max_rows);
    if (rows > 2 && !d->w_post) return fail(-4, "mtp_rounds: this head has no post-projection, drafts cannot chain");
    if (n_rounds < 1 || n_rounds + 1 > t->sched_cap) return fail(-2, "mtp_rounds: %d rounds (limit %d)", n_rounds, t->sched_cap - 1);
    if (token < 0 || token >= t->n_vocab) return fail(-2, "mtp_rounds: token id %d outside the target vocabulary of %d", token, t->n_vocab);
    // every round may accept its whole block, so the last one may start rows*(n_rounds-1) positions on
    if (pos < 1 || (long long)pos + (long long)rows * n_rounds > kv->max_seq) return fail(-2, "mtp_rounds: positions %d..%lld do not fit a cache of %d", pos, (long long)pos + (long long)rows * n_rounds - 1, kv->max_seq);
    if (d->H > t->max_rows * t->H) return fail(-2, "mtp_rounds: %d draft heads do not fit the target's attention scratch", d->H);
    HIP_TRY(hipSetDevice(t->device));
    int rc;
    int32_t tk = token;
    if ((rc = load_block(t, &tk, 1, pos))) return rc;
    if (!t->use_graph || t->prof.on || d->prof.on) {
        for (int r = 0; r < n_rounds; ++r) if ((rc = enqueue_round(d, kv, rows, false))) return rc;
    } else {
        const std::string key = "kv" + std::to_string(kv->id) + ":round" + std::to_string(rows) + (t->store_logits ? "l" : "") + (d->store_logits ? "L" : "") + (t->fuse_rows ? "" : "u") + (d->fuse_rows ? "" : "v") + (t->attn_rows ? "" : "r") + (t->attn_rows_fq ? "" : "q") + (t->head_mfma ? "" : "s") + (t->down_kq ? "" : "d") + (t->xcd_ffn ? "x" : "") + (t->fork_ple ? "" : "f") + "t" + std::to_string(t->xcd_tail) + (t->tail_spread == 1 ? "" : t->tail_spread ? "N" : "n") + (t->rows_geglu ? "g" : "") + (t->down_m ? "D" + std::to_string(t->down_m) : "") + "a" + std::to_string(t->xcd_attn_tail) + "o" + std::to_string(t->merge_o) + "." + std::to_string(t->merge_o_slices);
        auto it = d->graphs.find(key);            // kept by the head: the graph dies with it or with the cache
        if (it == d->graphs.end()) {
            hipGraph_t graph = nullptr;
            hipGraphExec_t exec = nullptr;
            if ((rc = enqueue_round(d, kv, rows, true))) return rc;
            HIP_TRY(hipStreamBeginCapture(t->stream, hipStreamCaptureModeThreadLocal));
            rc = enqueue_round(d, kv, rows, false);
            hipError_t e = hipStreamEndCapture(t->stream, &graph);
            if (rc) { if (graph) (void)hipGraphDestroy(graph); return rc; }
            if (e != hipSuccess) return fail(-100 - (int)e, "hipStreamEndCapture: %s", hipGetErrorString(e));
            e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
            (void)hipGraphDestroy(graph);
            if (e != hipSuccess) return fail(-100 - (int)e, "hipGraphInstantiate: %s", hipGetErrorString(e));
            it = d->graphs.emplace(key, exec).first;
        }
        for (int r = 0; r < n_rounds; ++r) HIP_TRY(hipGraphLaunch(it->second, t->stream));
    }
    HIP_TRY(hipStreamSynchronize(t->stream));
    StepCtl c;
    HIP_TRY(hipMemcpy(&c, t->ctl, sizeof c, hipMemcpyDeviceToHost));
    if (c.step != n_rounds) return fail(-9, "mtp_rounds: %d of %d rounds ran", c.step, n_rounds);
    { const int erc = step_err("mtp_rounds", c.err); if (erc) return erc; }
    HIP_TRY(hipMemcpy(blocks, t->sched, (size_t)n_rounds * rows * 4, hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(out, t->out, (size_t)n_rounds * rows * 4, hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(adv, t->adv, (size_t)n_rounds * 4, hipMemcpyDeviceToHost));
    if (final_pos) *final_pos = c.pos;
    t->last_rows = rows; t->last_adv = adv[n_rounds - 1];
    t->sched_steps = 0;
    d->last_rows = 1; d->last_adv = 1;
    return 0;
}

extern "C" int lg_hip_prefill(lg_hip_model *m, lg_hip_kv *kv, const int32_t *toks, int n, int pos0) {
    if (n <= 0) return 0;
    if (!m) return fail(-1, "prefill: null model");
    HIP_TRY(hipSetDevice(m->device));
    bool wide_ok = !m->target && m->wide_prefill;
    for (int L = 0; L < m->n_layer && wide_ok; ++L) {
        const Layer &y = m->L[L];
        wide_ok = y.qkv_m % 32 == 0 && y.nff % 32 == 0;
    }
    for (int done = 0; done < n;) {
        int rows = n - done < m->max_rows ? n - done : m->max_rows;
        if (wide_ok && n - done >= LG_WIDE_ROWS && kv->wide_rows >= LG_WIDE_ROWS) rows = LG_WIDE_ROWS;     // matrix-core blocks while the prompt lasts,
        else if (wide_ok && n - done >= LG_WIDE_MID && kv->wide_rows >= LG_WIDE_MID) rows = LG_WIDE_MID;
        else if (wide_ok && n - done >= LG_WIDE && kv->wide_rows >= LG_WIDE) rows = LG_WIDE;        // a single row tile, then verify-width blocks for the tail
        int rc = check_block(m, kv, toks + done, rows, rows, pos0 + done, true);
        if (rc) return rc;
        if ((rc = load_block(m, toks + done, rows, pos0 + done))) return rc;
        if ((rc = launch_step(m, kv, rows, false))) return rc;
        HIP_TRY(hipStreamSynchronize(m->stream));       // the pinned staging is reused by the next block
        done += rows;
    }
    return 0;
}

extern "C" int lg_hip_tail_stamps(lg_hip_model *m, int which, unsigned long long *dst, int cap) {
    if (!m || !dst || !m->tstamps || which < 0 || which > 1) return fail(-1, "tail_stamps: the model has no one-XCD tail");
    if (cap < LG_XTAIL_UNITS * 8) return fail(-2, "tail_stamps: room for %d values needed", LG_XTAIL_UNITS * 8);
    HIP_TRY(hipSetDevice(m->device));
    HIP_TRY(hipStreamSynchronize(m->stream));
    HIP_TRY(hipMemcpy(dst, m->tstamps + (size_t)which * LG_XTAIL_UNITS * 8, (size_t)LG_XTAIL_UNITS * 8 * 8, hipMemcpyDeviceToHost));
    return LG_XTAIL_UNITS;
}

extern "C" int lg_hip_get_hidden(lg_hip_model *m, float *dst) {
    if (!m || !dst) return fail(-1, "get_hidden: null argument");
    HIP_TRY(hipSetDevice(m->device));
    HIP_TRY(hipStreamSynchronize(m->stream));
    HIP_TRY(hipMemcpy(dst, m->g_hidden, (size_t)m->E * 4, hipMemcpyDeviceToHost));
    return 0;
}
extern "C" int lg_hip_set_hidden_row(lg_hip_model *m, int row) {
    if (!m) return fail(-1, "set_hidden_row: null model");
    if (row < 0 || row >= m->last_rows) return fail(-2, "set_hidden_row: row %d of a %d-row step", row, m->last_rows);
    HIP_TRY(hipSetDevice(m->device));
    HIP_TRY(hipMemcpyAsync(m->g_hidden, m->hidden_rows + (size_t)row * m->E, (size_t)m->E * 4, hipMemcpyDeviceToDevice, m->stream));
    return 0;
}
extern "C" int lg_hip_get_logits(lg_hip_model *m, int row, float *dst) {
    if (!m || !dst) return fail(-1, "get_logits: null argument");
    if (!m->store_logits) return fail(-4, "get_logits: the store_logits option is off");
    if (row < 0 || row >= m->last_rows) return fail(-2, "get_logits: row %d of a %d-row step", row, m->last_rows);
    HIP_TRY(hipSetDevice(m->device));
    HIP_TRY(hipStreamSynchronize(m->stream));
    HIP_TRY(hipMemcpy(dst, m->logits + (size_t)row * m->n_vocab, (size_t)m->n_vocab * 4, hipMemcpyDeviceToHost));
    return 0;
}

// ---- device-resident schedule -----------------------------------------------------------------
extern "C" int lg_hip_schedule_load(lg_hip_model *m, const int32_t *toks, int n_steps, int rows, int pos0) {
    if (!m || !toks || !m->committed) return fail(-1, "schedule_load: bad argument");
    if (rows < 1 || rows > m->max_rows || n_steps < 1 || n_steps > m->sched_cap) return fail(-2, "schedule_load: %d steps of %d rows (limits %d, %d)", n_steps, rows, m->sched_cap, m->max_rows);
    if (pos0 < 0) return fail(-2, "schedule_load: position %d", pos0);
    for (size_t i = 0; i < (size_t)n_steps * rows; ++i) if (toks[i] < 0 || toks[i] >= m->n_vocab) return fail(-2, "schedule_load: token id %d outside the vocabulary", toks[i]);
    HIP_TRY(hipSetDevice(m->device));
    HIP_TRY(hipStreamSynchronize(m->stream));
    HIP_TRY(hipMemcpy(m->sched, toks, (size_t)n_steps * rows * 4, hipMemcpyHostToDevice));
    StepCtl c{ pos0, 0, 0, 0 };
    HIP_TRY(hipMemcpy(m->ctl, &c, sizeof c, hipMemcpyHostToDevice));
    m->sched_steps = n_steps; m->sched_rows = rows; m->sched_pos0 = pos0; m->sched_loaded = n_steps;
    return 0;
}
extern "C" int lg_hip_schedule_run(lg_hip_model *m, lg_hip_kv *kv, int n_steps) {
    if (!m || !kv || kv->m != m) return fail(-1, "schedule_run: bad argument");
    if (n_steps < 1 || n_steps > m->sched_steps) return fail(-2, "schedule_run: %d steps requested, %d loaded", n_steps, m->sched_steps);
    // every step may accept its whole block: the last one of this call may start rows * (steps so far) positions on
    const long long last = (long long)m->sched_pos0 + (long long)m->sched_rows * (m->sched_loaded - m->sched_steps + n_steps);
    if (last > kv->max_seq) return fail(-2, "schedule_run: positions up to %lld do not fit a cache of %d", last - 1, kv->max_seq);
    HIP_TRY(hipSetDevice(m->device));
    for (int s = 0; s < n_steps; ++s) { int rc = launch_step(m, kv, m->sched_rows, true); if (rc) return rc; }
    m->sched_steps -= n_steps;       // steps left to run
    m->last_rows = m->sched_rows;
    return 0;
}
extern "C" int lg_hip_schedule_wait(lg_hip_model *m, int32_t *out, int32_t *adv, int32_t *final_pos) {
    if (!m) return fail(-1, "schedule_wait: null model");
    HIP_TRY(hipSetDevice(m->device));
    HIP_TRY(hipStreamSynchronize(m->stream));
    StepCtl c;
    HIP_TRY(hipMemcpy(&c, m->ctl, sizeof c, hipMemcpyDeviceToHost));
    { const int erc = step_err("schedule_wait", c.err); if (erc) return erc; }
    // the step counter is device state: never copy more than the schedule that was loaded holds
    if (c.step < 0 || c.step > m->sched_loaded)
        return fail(-6, "schedule_wait: the device reports %d steps done, %d were loaded", c.step, m->sched_loaded);
    if (out) HIP_TRY(hipMemcpy(out, m->out, (size_t)c.step * m->sched_rows * 4, hipMemcpyDeviceToHost));
    if (adv) HIP_TRY(hipMemcpy(adv, m->adv, (size_t)c.step * 4, hipMemcpyDeviceToHost));
    if (final_pos) *final_pos = c.pos;
    return c.step;
}
extern "C" int lg_hip_schedule_time(lg_hip_model *m, lg_hip_kv *kv, int n_steps, float *ms) {
    if (!m || !ms) return fail(-1, "schedule_time: null argument");
    HIP_TRY(hipSetDevice(m->device));
    hipEvent_t a, b;
    HIP_TRY(hipEventCreate(&a));
    HIP_TRY(hipEventCreate(&b));
    HIP_TRY(hipEventRecord(a, m->stream));
    int rc = lg_hip_schedule_run(m, kv, n_steps);
    if (!rc) {
        (void)hipEventRecord(b, m->stream);
        hipError_t e = hipEventSynchronize(b);
        if (e != hipSuccess) rc = fail(-100 - (int)e, "hipEventSynchronize: %s", hipGetErrorString(e));
        else (void)hipEventElapsedTime(ms, a, b);
    }
    (void)hipEventDestroy(a); (void)hipEventDestroy(b);
    return rc;
}

// ---- measurement ------------------------------------------------------------------------------
static void class_bytes(const lg_hip_model *m, const lg_hip_kv *kv, int pos, int rows, double *b) {
    const double q = 18.0 / 32.0;                         // bytes per q4_0 weight
    for (int i = 0; i < KC_COUNT; ++i) b[i] = 0;
    if (m->ple) b[KC_PMP] = (double)m->E * m->ple * m->n_layer * (m->pmp_f ? 4.0 : q);
    for (int L = 0; L < m->n_layer; ++L) {
        const Layer &y = m->L[L];
        b[KC_QKV] += (double)m->E * y.qkv_m * q;
        {
            const int w = (y.is_local && m->window > 0) ? m->window : 0, st = (w > 0 && pos - w + 1 > 0) ? pos - w + 1 : 0;
            const int tiles = ((pos + rows - 1) >> 5) - (st >> 5) + 1;
            b[use_attn_tail(m, y, rows, tiles) ? KC_ATAIL : use_merge_o(m, y, rows, tiles) ? KC_MERGE : KC_O] += (double)y.qd * m->E * q;
        }
        if (m->xffn_built && m->xcd_ffn && rows >= 4) b[KC_FFN] += 3.0 * m->E * y.nff * q;
        else { b[KC_GATEUP] += 2.0 * m->E * y.nff * q; b[KC_DOWN] += (double)y.nff * m->E * q; }
        if (m->ple && !y.winp_f && use_ple_tail(m, rows)) b[KC_TAIL] += 2.0 * m->E * m->ple * q;
        else if (m->ple) { const double pq = y.winp_f ? 4.0 : q; b[KC_PLEGATE] += (double)m->E * m->ple * pq; b[KC_PLEPROJ] += (double)m->ple * m->E * pq; }
        const int window = (y.is_local && m->window > 0) ? m->window : 0;
        const int last = pos + rows - 1, start = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
        b[KC_ATTN] += 2.0 * (last - start + 1) * y.kd * 2.0;          // K and V rows, f16
    }
    b[KC_HEAD] = (double)m->E * m->n_vocab * q;
    b[KC_ROWS] = 0;
    (void)kv;
}

extern "C" int lg_hip_profile_step(lg_hip_model *m, lg_hip_kv *kv, const int32_t *toks, int rows, int pos, int repeats,
                                   const char **names, float *ms, int32_t *launches, double *bytes, int cap) {
    int rc = check_block(m, kv, toks, rows, rows, pos);
    if (rc) return rc;
    if (cap < KC_COUNT || repeats < 1) return fail(-2, "profile_step: need room for %d classes", KC_COUNT);
    HIP_TRY(hipSetDevice(m->device));
    double acc[KC_COUNT] = { 0 };
    int cnt[KC_COUNT] = { 0 };
    for (int r = 0; r < repeats + 1; ++r) {              // first pass warms up and is dropped
        if ((rc = load_block(m, toks, rows, pos))) return rc;
        m->prof.on = true;
        rc = enqueue_step_rows(m, kv, rows, true);
        m->prof.on = false;
        hipError_t e = hipStreamSynchronize(m->stream);
        if (!rc && e != hipSuccess) rc = fail(-100 - (int)e, "profile_step: %s", hipGetErrorString(e));
        for (size_t i = 0; i < m->prof.cls.size(); ++i) {
            float t = 0;
            if (!rc && r > 0 && hipEventElapsedTime(&t, m->prof.ev[2 * i], m->prof.ev[2 * i + 1]) == hipSuccess) { acc[m->prof.cls[i]] += t; cnt[m->prof.cls[i]]++; }
        }
        for (hipEvent_t ev : m->prof.ev) (void)hipEventDestroy(ev);
        m->prof.ev.clear(); m->prof.cls.clear();
        if (rc) return rc;
    }
    double b[KC_COUNT];
    class_bytes(m, kv, pos, rows, b);
    for (int i = 0; i < KC_COUNT; ++i) {
        names[i] = k_class_names[i]; ms[i] = (float)(acc[i] / repeats); launches[i] = cnt[i] / repeats; bytes[i] = b[i];
    }
    m->last_rows = rows;
    return KC_COUNT;
}

// ---- isolated kernels -------------------------------------------------------------------------
struct Scratch {            // device buffers freed on scope exit
    std::vector<void *> p;
    ~Scratch() { for (void *q : p) (void)hipFree(q); }
    template <typename T> int get(T **out, size_t n) {
        HIP_TRY(hipMalloc((void **)out, n * sizeof(T) ? n * sizeof(T) : 16));
        p.push_back(*out);
        return 0;
    }
};

template <int M>
static int matmul_rows(hipStream_t st, const uint8_t *dw, int k, int mrows, const float *dx, float *dout, int32_t *ddots,
                       int8_t *dq, int repeats, float *kernel_ms) {
    const int n32 = M * (k / 32);
    hipLaunchKernelGGL(lg_k_quant_flat, dim3((n32 * 8 + LG_WG - 1) / LG_WG), dim3(LG_WG), 0, st, dx, M, k, dq);
    MmArgs a{ dw, k, mrows, dout, dq, ddots };
    lg_hip_model shim;                       // the launcher only needs a stream and the profiling switch
    shim.stream = st;
    Launcher lx{ &shim, false };
    if (ddots) launch_mm<M, true>(lx, 0, a);
    hipEvent_t e0 = nullptr, e1 = nullptr;
    auto body = [&]() -> int {
        HIP_TRY(hipEventCreate(&e0)); HIP_TRY(hipEventCreate(&e1));
        a.dots = nullptr;
        launch_mm<M, false>(lx, 0, a);           // warm-up, also the result
        HIP_TRY(hipEventRecord(e0, st));
        for (int r = 0; r < repeats; ++r) launch_mm<M, false>(lx, 0, a);
        if (lx.rc) return lx.rc;
        HIP_TRY(hipEventRecord(e1, st));
        HIP_TRY(hipStreamSynchronize(st));
        HIP_TRY(hipGetLastError());
        float t = 0;
        if (repeats > 0) HIP_TRY(hipEventElapsedTime(&t, e0, e1));
        if (kernel_ms) *kernel_ms = repeats > 0 ? t / repeats : 0.0f;
        return 0;
    };
    const int rc = body();
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    return rc;
}

extern "C" int lg_hip_matmul_f32w(const float *w, int k, int mrows, const float *x, int rows, float *out) {
    if (!w || !x || !out) return fail(-1, "matmul_f32w: null argument");
    if (k < 256 || k % 256 || mrows < 1 || rows < 1) return fail(-2, "matmul_f32w: k %d (a multiple of 256), m %d, rows %d", k, mrows, rows);
    if (lg_hip_device_count() < 1) return fail(-3, "matmul_f32w: no HIP device");
    Scratch sc;
    float *dw, *dx, *dout;
    if (sc.get(&dw, (size_t)mrows * k) || sc.get(&dx, (size_t)rows * k) || sc.get(&dout, (size_t)rows * mrows)) return -7;
    HIP_TRY(hipMemcpy(dw, w, (size_t)mrows * k * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(dx, x, (size_t)rows * k * 4, hipMemcpyHostToDevice));
    MmfArgs a{ dw, k, mrows, dx, k, rows, dout, mrows, nullptr, 0 };
    hipLaunchKernelGGL((lg_k_mmf<8>), dim3((mrows + LG_WG / 64 - 1) / (LG_WG / 64), (rows + 7) / 8), dim3(LG_WG), 0, nullptr, a);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipDeviceSynchronize());
    HIP_TRY(hipMemcpy(out, dout, (size_t)rows * mrows * 4, hipMemcpyDeviceToHost));
    return 0;
}

extern "C" int lg_hip_matmul_q4q8(const void *w, int k, int mrows, const float *x, int rows, float *out, int32_t *dots,
                                  int8_t *xq, float *xd, int32_t *xsum, int repeats, float *kernel_ms) {
    if (!w || !x) return fail(-1, "matmul: null input");
    const bool wide = rows == LG_WIDE;                   // one full row tile through the matrix-core kernel
    if (rows < 1 || (rows > LG_HIP_MAX_ROWS && !wide) || !lg_hip_repacked_bytes(k, mrows) || (!wide && lds_mm(rows, k) > 160 * 1024) || (wide && mrows % 32))
        return fail(-2, "matmul: rows %d (1..%d, or %d with m %% 32 == 0), k %d (multiple of 256, rows*k*1.25 <= 160 KiB), m %d (multiple of 8)", rows, LG_HIP_MAX_ROWS, LG_WIDE, k, mrows);
    if (lg_hip_device_count() < 1) return fail(-3, "matmul: no HIP device");
    const int nb = k / 32;
    std::vector<uint8_t> tiled(lg_hip_repacked_bytes(k, mrows));
    int rc = lg_hip_repack_q4_0(w, k, mrows, tiled.data());
    if (rc) return rc;
    Scratch sc;
    uint8_t *dw; float *dx, *dout; int32_t *ddots = nullptr; int8_t *dq;
    if (sc.get(&dw, tiled.size()) || sc.get(&dx, (size_t)rows * k) || sc.get(&dout, (size_t)rows * mrows * 4) ||
        sc.get(&dq, (size_t)rows * k * 5 / 4)) return -7;
    if (dots && sc.get(&ddots, (size_t)rows * mrows * nb)) return -7;
    HIP_TRY(hipMemcpy(dw, tiled.data(), tiled.size(), hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(dx, x, (size_t)rows * k * 4, hipMemcpyHostToDevice));
    hipStream_t st;
    HIP_TRY(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
    switch (rows) {
#define CASE(M) case M: rc = matmul_rows<M>(st, dw, k, mrows, dx, dout, ddots, dq, repeats, kernel_ms); break;
        CASE(1) CASE(2) CASE(3) CASE(4) CASE(5) CASE(6) CASE(7) CASE(8) CASE(LG_WIDE)
#undef CASE
    }
    (void)hipStreamDestroy(st);
    if (rc) return rc;
    if (out && wide && lg_segments(k) == 32) {             // four slabs of partial sums: the top of the segment tree is added here
        std::vector<float> parts((size_t)4 * rows * mrows);
        HIP_TRY(hipMemcpy(parts.data(), dout, parts.size() * 4, hipMemcpyDeviceToHost));
        const size_t n = (size_t)rows * mrows;
        for (size_t i = 0; i < n; ++i) out[i] = (parts[i] + parts[n + i]) + (parts[2 * n + i] + parts[3 * n + i]);
    } else if (out) HIP_TRY(hipMemcpy(out, dout, (size_t)rows * mrows * 4, hipMemcpyDeviceToHost));
    if (dots) HIP_TRY(hipMemcpy(dots, ddots, (size_t)rows * mrows * nb * 4, hipMemcpyDeviceToHost));
    // the device keeps activation rows in the matmul's own order (lg_act_layout); hand them back in natural order
    const ActLayout lay = lg_act_layout(k);
    if (xq) {
        std::vector<int8_t> dev((size_t)rows * k);
        HIP_TRY(hipMemcpy(dev.data(), dq, dev.size(), hipMemcpyDeviceToHost));
        for (int j = 0; j < rows; ++j)
            for (int w = 0; w < k / 16; ++w) {
                const int u = lg_act_unit(lay, w);
                if (!wide) { memcpy(xq + (size_t)j * k + (size_t)w * 16, dev.data() + (size_t)j * k + (size_t)u * 16, 16); continue; }
                for (int hh = 0; hh < 2; ++hh)           // wide layout: halves of a unit of all 32 rows side by side
                    memcpy(xq + (size_t)j * k + (size_t)w * 16 + hh * 8, dev.data() + ((size_t)(u * 2 + hh) * 32 + j) * 8, 8);
            }
    }
    if (xd || xsum) {
        std::vector<float2> ds((size_t)rows * nb);
        HIP_TRY(hipMemcpy(ds.data(), dq + (size_t)rows * k, ds.size() * 8, hipMemcpyDeviceToHost));
        for (int j = 0; j < rows; ++j)
            for (int b = 0; b < nb; ++b) {
                const float2 v = wide ? ds[(size_t)lg_act_block(lay, b) * 32 + j] : ds[(size_t)j * nb + lg_act_block(lay, b)];
                if (xd) xd[(size_t)j * nb + b] = v.x;
                if (xsum) memcpy(&xsum[(size_t)j * nb + b], &v.y, 4);
            }
    }
    return 0;
}

// q8 rows of a verify-width block from the device's activation order back to natural order
static int read_back_q8(const int8_t *dq, int rows, int k, int8_t *xq, float *xd, int32_t *xsum) {
    const ActLayout lay = lg_act_layout(k);
    const int nb = k / 32;
    if (xq) {
        std::vector<int8_t> dev((size_t)rows * k);
        HIP_TRY(hipMemcpy(dev.data(), dq, dev.size(), hipMemcpyDeviceToHost));
        for (int j = 0; j < rows; ++j)
            for (int w = 0; w < k / 16; ++w)
                memcpy(xq + (size_t)j * k + (size_t)w * 16, dev.data() + (size_t)j * k + (size_t)lg_act_unit(lay, w) * 16, 16);
    }
    if (xd || xsum) {
        std::vector<float2> ds((size_t)rows * nb);
        HIP_TRY(hipMemcpy(ds.data(), dq + (size_t)rows * k, ds.size() * 8, hipMemcpyDeviceToHost));
        for (int j = 0; j < rows; ++j)
            for (int b = 0; b < nb; ++b) {
                const float2 v = ds[(size_t)j * nb + lg_act_block(lay, b)];
                if (xd) xd[(size_t)j * nb + b] = v.x;
                if (xsum) memcpy(&xsum[(size_t)j * nb + b], &v.y, 4);
            }
    }
    return 0;
}

template <int M>
static void rows_isolated(hipStream_t st, const RowArgs &s_in, StepCtl *ctl) {
    RowArgs s = s_in;
    const int slices = (s.E + 1023) / 1024;                   // as a verify step launches it: the tail sliced over workgroups
    s.slices = slices;
    hipLaunchKernelGGL((lg_k_rows<M>), dim3(M, slices), dim3(LG_WG), 0, st, ctl, LG_ROW_FIELDS(LG_XA, s) 0);
}
extern "C" int lg_hip_rows_norm_q8(const float *x, const float *dout, const float *w_post, const float *out_scale,
                                   const float *w_pre, int rows, int E, float eps, float *x_out, float *h_out,
                                   int8_t *xq, float *xd, int32_t *xsum) {
    if (!x) return fail(-1, "rows_norm_q8: null input");
    if (rows < 1 || rows > LG_HIP_MAX_ROWS || E < 256 || E % 256 || E > 4096) return fail(-2, "rows_norm_q8: rows %d (1..%d), E %d (a multiple of 256 up to 4096)", rows, LG_HIP_MAX_ROWS, E);
    if (dout && !w_post) return fail(-1, "rows_norm_q8: a sub-layer output needs its norm weight");
    if (lg_hip_device_count() < 1) return fail(-3, "rows_norm_q8: no HIP device");
    Scratch sc;
    float *dx, *dd = nullptr, *dwp = nullptr, *dos = nullptr, *dwr = nullptr, *dxo, *dho; int8_t *dq; StepCtl *ctl;
    const size_t n = (size_t)rows * E;
    if (sc.get(&dx, n) || sc.get(&dxo, n) || sc.get(&dho, n) || sc.get(&dq, n * 5 / 4) || sc.get(&ctl, 1)) return -7;
    HIP_TRY(hipMemcpy(dx, x, n * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemset(ctl, 0, sizeof(StepCtl)));
    if (dout) { if (sc.get(&dd, n) || sc.get(&dwp, (size_t)E)) return -7; HIP_TRY(hipMemcpy(dd, dout, n * 4, hipMemcpyHostToDevice)); HIP_TRY(hipMemcpy(dwp, w_post, (size_t)E * 4, hipMemcpyHostToDevice)); }
    if (out_scale) { if (sc.get(&dos, 1)) return -7; HIP_TRY(hipMemcpy(dos, out_scale, 4, hipMemcpyHostToDevice)); }
    if (w_pre) { if (sc.get(&dwr, (size_t)E)) return -7; HIP_TRY(hipMemcpy(dwr, w_pre, (size_t)E * 4, hipMemcpyHostToDevice)); }
    RowArgs s{};
    s.x = dx; s.dout = dd; s.dparts = 1; s.w_post = dwp; s.os = dos; s.x_out = dxo; s.w_pre = dwr; s.h_out = dho;
    s.q = dq; s.E = E; s.eps = eps;
    switch (rows) {
#define CASE(M) case M: rows_isolated<M>(nullptr, s, ctl); break;
        CASE(1) CASE(2) CASE(3) CASE(4) CASE(5) CASE(6) CASE(7) CASE(8)
#undef CASE
    }
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipDeviceSynchronize());
    if (x_out) HIP_TRY(hipMemcpy(x_out, dxo, n * 4, hipMemcpyDeviceToHost));
    if (h_out) HIP_TRY(hipMemcpy(h_out, dho, n * 4, hipMemcpyDeviceToHost));
    return read_back_q8(dq, rows, E, xq, xd, xsum);
}

// ---- isolated per-layer-embedding kernels (tests) ----------------------------------------------------
// lg_k_rows_plegate on its own: the residual update x + rmsnorm(dout) * w_post of `rows` rows, then the inp_gate
// matmul (w_gate: ple plain q4_0 rows of E) on the q8 of the new rows, gelu(.) * ipl and the q8 of that.
extern "C" int lg_hip_rows_ple_gate(const float *x, const float *dout, const float *w_post, const void *w_gate, const float *ipl,
                                    int rows, int E, int ple, float eps, float *x_out, int8_t *pq, float *pd, int32_t *psum) {
    if (!x || !dout || !w_post || !w_gate || !ipl) return fail(-1, "rows_ple_gate: null input");
    if (rows < 1 || rows > LG_HIP_MAX_ROWS || E < 256 || E % 256 || E > 4096 || ple != 256)
        return fail(-2, "rows_ple_gate: rows %d (1..%d), E %d (a multiple of 256 up to 4096), ple %d (256 is built)", rows, LG_HIP_MAX_ROWS, E, ple);
    if (lg_hip_device_count() < 1) return fail(-3, "rows_ple_gate: no HIP device");
    std::vector<uint8_t> tiled(lg_hip_repacked_bytes(E, ple));
    int rc = lg_hip_repack_q4_0(w_gate, E, ple, tiled.data());
    if (rc) return rc;
    Scratch sc;
    float *dx, *dd, *dw, *di, *dxo; uint8_t *dg; int8_t *dq;
    const size_t n = (size_t)rows * E;
    if (sc.get(&dx, n) || sc.get(&dd, n) || sc.get(&dw, (size_t)E) || sc.get(&di, (size_t)rows * ple) || sc.get(&dxo, n) ||
        sc.get(&dg, tiled.size()) || sc.get(&dq, (size_t)rows * ple * 5 / 4)) return -7;
    HIP_TRY(hipMemcpy(dx, x, n * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(dd, dout, n * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(dw, w_post, (size_t)E * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(di, ipl, (size_t)rows * ple * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(dg, tiled.data(), tiled.size(), hipMemcpyHostToDevice));
    PleGateArgs a{ dg, E, ple, nullptr, di, 0, 1, dq };
    RowsPleGateArgs r{ a, dx, dd, dw, dxo, eps, 1 };
    switch (rows) {
#define CASE(M) case M: rc = set_lds(lg_k_rows_plegate<M>, lds_mm(1, E)); \
        if (!rc) hipLaunchKernelGGL((lg_k_rows_plegate<M>), dim3(ple / 32, M), dim3(LG_WG), lds_mm(1, E), nullptr, LG_RPG_FIELDS(LG_XA, r) 0); break;
        CASE(1) CASE(2) CASE(3) CASE(4) CASE(5) CASE(6) CASE(7) CASE(8)
#undef CASE
    }
    if (rc) return rc;
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipDeviceSynchronize());
    if (x_out) HIP_TRY(hipMemcpy(x_out, dxo, n * 4, hipMemcpyDeviceToHost));
    return read_back_q8(dq, rows, ple, pq, pd, psum);
}

// lg_k_ipl on its own: the per-layer inputs of `rows` tokens from the raw per_layer_model_proj output
// (pmp [rows][n_layer*ple]) and the tokens' rows of per_layer_token_embd (pte: n_tok plain q4_0 rows of n_layer*ple).
extern "C" int lg_hip_ple_inputs(const float *pmp, const float *proj_norm, const void *pte, int n_tok, const int32_t *toks,
                                 int rows, int n_layer, int ple, int E, float eps, float *out) {
    if (!pmp || !proj_norm || !pte || !toks || !out) return fail(-1, "ple_inputs: null argument");
    if (rows < 1 || rows > LG_HIP_MAX_ROWS || n_layer < 1 || ple < 32 || ple % 32 || ple > 256 || n_tok < 1 || E < 1)
        return fail(-2, "ple_inputs: rows %d (1..%d), n_layer %d, ple %d (a multiple of 32 up to 256), %d token rows", rows, LG_HIP_MAX_ROWS, n_layer, ple, n_tok);
    for (int j = 0; j < rows; ++j) if (toks[j] < 0 || toks[j] >= n_tok) return fail(-2, "ple_inputs: token %d of row %d (table of %d rows)", toks[j], j, n_tok);
    if (lg_hip_device_count() < 1) return fail(-3, "ple_inputs: no HIP device");
    Scratch sc;
    const size_t w = (size_t)n_layer * ple, tb = (size_t)n_tok * (w / 32 * 18);
    float *dp, *dn; uint8_t *dt; int32_t *dk; StepCtl *ctl;
    if (sc.get(&dp, rows * w) || sc.get(&dn, (size_t)ple) || sc.get(&dt, tb) || sc.get(&dk, (size_t)rows) || sc.get(&ctl, 1)) return -7;
    HIP_TRY(hipMemcpy(dp, pmp, rows * w * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(dn, proj_norm, (size_t)ple * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(dt, pte, tb, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(dk, toks, (size_t)rows * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemset(ctl, 0, sizeof(StepCtl)));
    IplArgs i{ dp, ple, n_layer, rows, dn, dt, dk, 1.0f / sqrtf((float)E), sqrtf((float)ple), 1.0f / sqrtf(2.0f), eps };
    hipLaunchKernelGGL(lg_k_ipl, dim3(n_layer, rows), dim3(64), 0, nullptr, i, ctl);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipDeviceSynchronize());
    HIP_TRY(hipMemcpy(out, dp, rows * w * 4, hipMemcpyDeviceToHost));
    return 0;
}

// the two launches of an isolated attention: tile partials, then the ordered merge
// (the same choice of kernels as a verify step makes: many (tile, kv head) pairs -> one workgroup per pair serves all
// rows; many tiles per row -> the merge is cut by dims)
template <int M>
static int enqueue_attention(hipStream_t st, const AttnArgs &a_in, const MergeArgs &g, StepCtl *ctl, int tiles, size_t lds) {
    AttnArgs a = a_in;
    a.gx = tiles; a.gz = M;                               // the grid of lg_k_attn, which reads it from its arguments
    if (attention_rows_shared(M, tiles, a.nkv, a.hd, a.seq)) {
        if constexpr (M > 1 && M <= LG_HIP_MAX_ROWS) {
            const int units = M * (a.H / a.nkv);
            const size_t l2 = a.hd == 256 ? AttnRowsGeo<256>::bytes(units) : a.hd == 128 ? AttnRowsGeo<128>::bytes(units) : AttnRowsGeo<64>::bytes(units);
            int rc = a.hd == 256 ? set_lds(lg_k_attn_rows<M, 256>, l2) : a.hd == 128 ? set_lds(lg_k_attn_rows<M, 128>, l2) : set_lds(lg_k_attn_rows<M, 64>, l2);
            if (rc) return rc;
            const int tp = attention_rows_tp(tiles, a.nkv);
            const dim3 grid((tiles + tp - 1) / tp, a.nkv);
            if (a.hd == 256)      hipLaunchKernelGGL((lg_k_attn_rows<M, 256>), grid, dim3(LG_WG), l2, st, ctl, tp, LG_ATTN_FIELDS(LG_XA, a) 0);
            else if (a.hd == 128) hipLaunchKernelGGL((lg_k_attn_rows<M, 128>), grid, dim3(LG_WG), l2, st, ctl, tp, LG_ATTN_FIELDS(LG_XA, a) 0);
            else                  hipLaunchKernelGGL((lg_k_attn_rows<M, 64>), grid, dim3(LG_WG), l2, st, ctl, tp, LG_ATTN_FIELDS(LG_XA, a) 0);
        }
    } else hipLaunchKernelGGL((lg_k_attn<false, 1>), dim3(tiles, a.nkv, M), dim3(LG_WG), lds, st, ctl, LG_ATTN_FIELDS(LG_XA, a) 0);
    if (M <= LG_HIP_MAX_ROWS && tiles >= 128 && a.hd % 64 == 0) hipLaunchKernelGGL((lg_k_attn_merge_split<M>), dim3(a.H, M, a.hd / 64), dim3(LG_WG), 0, st, ctl, LG_MERGE_FIELDS(LG_XA, g) 0);
    else hipLaunchKernelGGL((lg_k_attn_merge<M>), dim3(a.H, M), dim3(LG_WG), 0, st, ctl, LG_MERGE_FIELDS(LG_XA, g) 0);
    return 0;
}

template <int M>
static int attention_rows(hipStream_t st, AttnArgs a, MergeArgs g, StepCtl *ctl, int tiles, int repeats, float *kernel_ms) {
    const size_t lds = attn_lds(a.H / a.nkv, a.hd, false);
    int rc = set_lds(lg_k_attn<false, 1>, lds);
    if (rc) return rc;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    auto body = [&]() -> int {
        HIP_TRY(hipEventCreate(&e0)); HIP_TRY(hipEventCreate(&e1));
        for (int r = 0; r < repeats + 1; ++r) {
            if (r == 1) HIP_TRY(hipEventRecord(e0, st));
            const int erc = enqueue_attention<M>(st, a, g, ctl, tiles, lds);
            if (erc) return erc;
        }
        HIP_TRY(hipEventRecord(e1, st));
        HIP_TRY(hipStreamSynchronize(st));
        HIP_TRY(hipGetLastError());
        float t = 0;
        if (repeats > 0) HIP_TRY(hipEventElapsedTime(&t, e0, e1));
        if (kernel_ms) *kernel_ms = repeats > 0 ? t / repeats : 0.0f;
        return 0;
    };
    rc = body();
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    return rc;
}

extern "C" int lg_hip_attention(const float *q, const uint16_t *kc, const uint16_t *vc, int rows, int n_head, int n_head_kv,
                                int hd, int seq, int window, int pos, float *out, int repeats, float *kernel_ms) {
    if (!q || !kc || !vc || !out) return fail(-1, "attention: null argument");
    if (rows < 1 || rows > LG_HIP_MAX_ROWS || n_head_kv < 1 || n_head % n_head_kv || n_head / n_head_kv > 8 ||
        (hd != 64 && hd != 128 && hd != 256 && hd != 512) || pos < 0 || seq < 1)
        return fail(-2, "attention: unsupported shape");
    if (window > 0 ? seq < window + rows - 1 && seq < pos + rows : seq < pos + rows)
        return fail(-2, "attention: a cache of %d rows cannot hold the keys of positions up to %d", seq, pos + rows - 1);
    if (lg_hip_device_count() < 1) return fail(-3, "attention: no HIP device");
    const int kd = n_head_kv * hd, qd = n_head * hd;
    const int start0 = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    const int tiles = ((pos + rows - 1) >> 5) - (start0 >> 5) + 1;
    Scratch sc;
    float *dq, *dpm, *dpl, *dpacc, *dxf; uint16_t *dk, *dv; int8_t *dxq; StepCtl *ctl;
    const size_t slots = (size_t)rows * n_head * tiles;
    if (sc.get(&dq, (size_t)rows * qd) || sc.get(&dk, (size_t)seq * kd) || sc.get(&dv, (size_t)seq * kd) ||
        sc.get(&dpm, slots) || sc.get(&dpl, slots) || sc.get(&dpacc, slots * hd) || sc.get(&dxf, (size_t)rows * qd) ||
        sc.get(&dxq, (size_t)rows * qd * 5 / 4) || sc.get(&ctl, (size_t)1)) return -7;
    HIP_TRY(hipMemcpy(dq, q, (size_t)rows * qd * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(dk, kc, (size_t)seq * kd * 2, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(dv, vc, (size_t)seq * kd * 2, hipMemcpyHostToDevice));
    StepCtl c{ pos, 0, 0, 0 };
    HIP_TRY(hipMemcpy(ctl, &c, sizeof c, hipMemcpyHostToDevice));
    AttnArgs a{};
    a.q = dq; a.H = n_head; a.nkv = n_head_kv; a.hd = hd;
    a.kc = dk; a.vc = dv; a.seq = seq; a.kv_dim = kd; a.window = window;
    a.pm = dpm; a.pl = dpl; a.pacc = dpacc; a.tiles_max = tiles;
    MergeArgs g{ dpm, dpl, dpacc, tiles, n_head, hd, window, 0, dxq, dxf };
    hipStream_t st;
    HIP_TRY(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
    int rc = 0;
    switch (rows) {
#define CASE(M) case M: rc = attention_rows<M>(st, a, g, ctl, tiles, repeats, kernel_ms); break;
        CASE(1) CASE(2) CASE(3) CASE(4) CASE(5) CASE(6) CASE(7) CASE(8) CASE(LG_WIDE)
#undef CASE
    }
    (void)hipStreamDestroy(st);
    if (rc) return rc;
    HIP_TRY(hipMemcpy(out, dxf, (size_t)rows * qd * 4, hipMemcpyDeviceToHost));
    return 0;
}

// ---- attention for callers that cannot allocate ---------------------------------------------------
// lg_hip_attention with every buffer given by the caller as DEVICE memory, and the kernels' own working
// memory (step state, tile partials, the q8 copy of the result that the merge kernel also writes) in a
// static device array instead of hipMalloc'ed scratch: nothing is allocated or freed, the launches are
// left on the caller's stream and the call returns without waiting.
#define LG_NOALLOC_BYTES (8u << 20)
#define LG_NOALLOC_DEVICES 16
static __device__ __align__(256) unsigned char lg_noalloc_scratch[LG_NOALLOC_BYTES];
// the array's device address, asked once per device (each device holds its own copy at its own address)
static unsigned char *g_noalloc_ptr[LG_NOALLOC_DEVICES];

__global__ void lg_k_set_ctl(StepCtl *ctl, int pos) { ctl->pos = pos; ctl->step = 0; ctl->err = 0; ctl->pad = 0; }

static size_t up256(size_t n) { return (n + 255) & ~(size_t)255; }

extern "C" size_t lg_hip_attention_noalloc_limit(void) { return LG_NOALLOC_BYTES; }

// Everything the entry point needs from the runtime besides launches, for the current device: the array's address
// and, for every kernel it may launch with more than the default dynamic LDS, the limit raised to the most any
// accepted shape asks for.  Neither call is legal while a stream is being captured, so a capturing caller calls
// this first; the entry point calls it by itself on its first use on a device.
template <int M>
static int noalloc_raise_rows() {
    int rc = set_lds(lg_k_attn_rows<M, 256>, AttnRowsGeo<256>::bytes(M * 8));
    if (!rc) rc = set_lds(lg_k_attn_rows<M, 128>, AttnRowsGeo<128>::bytes(M * 8));
    if (!rc) rc = set_lds(lg_k_attn_rows<M, 64>, AttnRowsGeo<64>::bytes(M * 8));
    return rc;
}
extern "C" int lg_hip_attention_noalloc_init(void) {
    int dev = -1;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= LG_NOALLOC_DEVICES) return fail(-3, "attention_noalloc: device %d (0..%d are served)", dev, LG_NOALLOC_DEVICES - 1);
    if (g_noalloc_ptr[dev]) return 0;
    int rc = set_lds(lg_k_attn<false, 1>, attn_lds(8, 512, false));
    if (!rc) rc = noalloc_raise_rows<2>();
    if (!rc) rc = noalloc_raise_rows<3>();
    if (!rc) rc = noalloc_raise_rows<4>();
    if (!rc) rc = noalloc_raise_rows<5>();
    if (!rc) rc = noalloc_raise_rows<6>();
    if (!rc) rc = noalloc_raise_rows<7>();
    if (!rc) rc = noalloc_raise_rows<8>();
    if (rc) return rc;
    void *p = nullptr;
    HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(lg_noalloc_scratch)));
    if (!p) return fail(-3, "attention_noalloc: the working array has no address on device %d", dev);
    g_noalloc_ptr[dev] = (unsigned char *)p;
    return 0;
}

extern "C" int lg_hip_attention_noalloc(const float *d_q, const uint16_t *d_kc, const uint16_t *d_vc, int rows, int n_head,
                                        int n_head_kv, int hd, int seq, int window, int pos, float *d_out, void *stream) {
    if (!d_q || !d_kc || !d_vc || !d_out) return fail(-1, "attention_noalloc: null argument");
    if (rows < 1 || rows > LG_HIP_MAX_ROWS || n_head_kv < 1 || n_head % n_head_kv || n_head / n_head_kv > 8 ||
        (hd != 64 && hd != 128 && hd != 256 && hd != 512) || pos < 0 || seq < 1)
        return fail(-2, "attention_noalloc: unsupported shape");
    if (window > 0 ? seq < window + rows - 1 && seq < pos + rows : seq < pos + rows)
        return fail(-2, "attention_noalloc: a cache of %d rows cannot hold the keys of positions up to %d", seq, pos + rows - 1);
    const int qd = n_head * hd;
    const int start0 = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    const int tiles = ((pos + rows - 1) >> 5) - (start0 >> 5) + 1;
    const size_t slots = (size_t)rows * n_head * tiles;
    const size_t o_pm = 256, o_pl = o_pm + up256(slots * 4), o_pacc = o_pl + up256(slots * 4),
                 o_xq = o_pacc + up256(slots * hd * 4), need = o_xq + up256((size_t)rows * qd * 5 / 4);
    if (need > LG_NOALLOC_BYTES)
        return fail(-2, "attention_noalloc: %d rows x %d heads x %d key tiles of %d need %zu bytes of working memory; the built-in array holds %u",
                    rows, n_head, tiles, hd, need, LG_NOALLOC_BYTES);
    int dev = -1;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= LG_NOALLOC_DEVICES) return fail(-3, "attention_noalloc: device %d (0..%d are served)", dev, LG_NOALLOC_DEVICES - 1);
    if (!g_noalloc_ptr[dev]) {
        const int irc = lg_hip_attention_noalloc_init();
        if (irc) return irc;
    }
    unsigned char *base = g_noalloc_ptr[dev];
    StepCtl *ctl = (StepCtl *)base;
    float *dpm = (float *)(base + o_pm), *dpl = (float *)(base + o_pl), *dpacc = (float *)(base + o_pacc);
    int8_t *dxq = (int8_t *)(base + o_xq);
    AttnArgs a{};
    a.q = d_q; a.H = n_head; a.nkv = n_head_kv; a.hd = hd;
    a.kc = d_kc; a.vc = d_vc; a.seq = seq; a.kv_dim = n_head_kv * hd; a.window = window;
    a.pm = dpm; a.pl = dpl; a.pacc = dpacc; a.tiles_max = tiles;
    MergeArgs g{ dpm, dpl, dpacc, tiles, n_head, hd, window, 0, dxq, d_out };
    const size_t lds = attn_lds(n_head / n_head_kv, hd, false);
    int rc = set_lds(lg_k_attn<false, 1>, lds);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    // every tile slot that the merge reads is written by the tile kernel of the same call, so nothing has to be
    // cleared; only the step state is set, by a kernel (a caller may be capturing this stream)
    hipLaunchKernelGGL(lg_k_set_ctl, dim3(1), dim3(1), 0, st, ctl, pos);
    switch (rows) {
#define CASE(M) case M: rc = enqueue_attention<M>(st, a, g, ctl, tiles, lds); break;
        CASE(1) CASE(2) CASE(3) CASE(4) CASE(5) CASE(6) CASE(7) CASE(8)
#undef CASE
    }
    if (rc) return rc;
    HIP_TRY(hipGetLastError());
    return 0;
}

// ---- launch floor -----------------------------------------------------------------------------------
// What a chain of dependent kernels costs before it does any work: a captured graph of n kernels in a row, each
// empty (mode 0) or reading the 64 bytes its predecessor wrote and writing 64 for its successor (mode 1).
__global__ void lg_k_floor_empty() {}
__global__ void lg_k_floor_chain(const int *src, int *dst) {
    if (blockIdx.x == 0 && threadIdx.x < 16) dst[threadIdx.x] = src[threadIdx.x] + 1;
}
extern "C" int lg_hip_launch_floor(int n_kernels, int mode, int grid, int block, int replays, float *us_per_kernel) {
    if (n_kernels < 1 || n_kernels > 4096 || mode < 0 || mode > 1 || grid < 1 || grid > 65536 || block < 1 || block > 1024 ||
        replays < 1 || !us_per_kernel) return fail(-2, "launch_floor: bad argument");
    if (lg_hip_device_count() < 1) return fail(-3, "launch_floor: no HIP device");
    hipStream_t st = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int *a = nullptr, *b = nullptr;
    auto body = [&]() -> int {
        HIP_TRY(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
        HIP_TRY(hipMalloc((void **)&a, 256)); HIP_TRY(hipMalloc((void **)&b, 256));
        HIP_TRY(hipMemset(a, 0, 256)); HIP_TRY(hipMemset(b, 0, 256));
        HIP_TRY(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
        for (int i = 0; i < n_kernels; ++i) {
            if (mode == 0) hipLaunchKernelGGL(lg_k_floor_empty, dim3(grid), dim3(block), 0, st);
            else hipLaunchKernelGGL(lg_k_floor_chain, dim3(grid), dim3(block), 0, st, (i & 1) ? b : a, (i & 1) ? a : b);
        }
        HIP_TRY(hipStreamEndCapture(st, &graph));
        HIP_TRY(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
        HIP_TRY(hipEventCreate(&e0)); HIP_TRY(hipEventCreate(&e1));
        HIP_TRY(hipGraphLaunch(exec, st));                   // warm-up
        HIP_TRY(hipStreamSynchronize(st));
        HIP_TRY(hipEventRecord(e0, st));
        for (int r = 0; r < replays; ++r) HIP_TRY(hipGraphLaunch(exec, st));
        HIP_TRY(hipEventRecord(e1, st));
        HIP_TRY(hipStreamSynchronize(st));
        float ms = 0;
        HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
        *us_per_kernel = ms * 1e3f / ((float)replays * (float)n_kernels);
        return 0;
    };
    const int rc = body();
    if (exec) (void)hipGraphExecDestroy(exec);
    if (graph) (void)hipGraphDestroy(graph);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (a) (void)hipFree(a);
    if (b) (void)hipFree(b);
    if (st) (void)hipStreamDestroy(st);
    return rc;
}

// ---- XCD placement and hand-over probes ------------------------------------------------------------
// Which XCD every workgroup of a grid x block launch (with lds_bytes of dynamic LDS) ran on, `launches` times in a
// row on one stream: xcc / hwid receive [launches][grid] values (XCC_ID and HW_ID registers).
__global__ void lg_k_xcd_map_lds(int32_t *xcc, int32_t *hwid) {
    extern __shared__ unsigned char smem[];
    if (threadIdx.x == 0) { smem[0] = 1; xcc[blockIdx.x] = lg_xcc_id(); hwid[blockIdx.x] = (int32_t)lg_hw_id(); }
}
extern "C" int lg_hip_xcd_map(int grid, int block, int lds_bytes, int launches, int32_t *xcc, int32_t *hwid) {
    if (grid < 1 || grid > 65536 || block < 1 || block > 1024 || lds_bytes < 0 || lds_bytes > 160 * 1024 || launches < 1 || !xcc || !hwid)
        return fail(-2, "xcd_map: bad argument");
    if (lg_hip_device_count() < 1) return fail(-3, "xcd_map: no HIP device");
    Scratch sc;
    int32_t *dx, *dh;
    const size_t n = (size_t)grid * launches;
    if (sc.get(&dx, n) || sc.get(&dh, n)) return -7;
    if (lds_bytes > 48 * 1024) HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(lg_k_xcd_map_lds), hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes));
    for (int l = 0; l < launches; ++l)
        hipLaunchKernelGGL(lg_k_xcd_map_lds, dim3(grid), dim3(block), (size_t)lds_bytes, nullptr, dx + (size_t)l * grid, dh + (size_t)l * grid);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipDeviceSynchronize());
    HIP_TRY(hipMemcpy(xcc, dx, n * 4, hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(hwid, dh, n * 4, hipMemcpyDeviceToHost));
    return 0;
}

// One hand-over experiment (lg_k_xcd_handover): n workgroups of a 256-workgroup launch, chosen by set_mode / sel,
// exchange `bytes` each per round through flags; store_scope / load_scope 0..3 = plain, sc0, sc1, sc0 sc1.
// res receives [n][4] = { ticks, mismatching words, polls given up, XCD id }; *tick_ns the length of a tick.
extern "C" int lg_hip_xcd_handover(int set_mode, int sel, int n, int store_scope, int load_scope, int bytes, int rounds,
                                   int32_t *res, float *tick_ns) {
    if (set_mode < 0 || set_mode > 1 || n < 2 || n > 32 || sel < 0 || (set_mode == 0 ? sel >= LG_XCDS : (sel + 1) * n > 256) ||
        store_scope < 0 || store_scope > 3 || load_scope < 0 || load_scope > 3 || bytes < 0 || bytes % 4 || bytes > (1 << 20) ||
        rounds < 1 || rounds > 100000 || !res || !tick_ns)
        return fail(-2, "xcd_handover: bad argument");
    if (lg_hip_device_count() < 1) return fail(-3, "xcd_handover: no HIP device");
    int dev = 0, khz = 0;
    HIP_TRY(hipGetDevice(&dev));
    HIP_TRY(hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev));
    *tick_ns = khz > 0 ? 1e6f / (float)khz : 10.0f;
    Scratch sc;
    XcdProbeArgs a{};
    a.n = n; a.words = bytes / 4; a.rounds = rounds; a.set_mode = set_mode; a.sel = sel; a.spin_limit = 4000;
    if (sc.get(&a.flags, (size_t)64) || sc.get(&a.data, (size_t)2 * n * (a.words ? a.words : 1)) || sc.get(&a.res, (size_t)n * 4)) return -7;
    HIP_TRY(hipMemset(a.flags, 0, 256));
    HIP_TRY(hipMemset(a.res, 0xFF, (size_t)n * 16));
    HIP_TRY(hipDeviceSynchronize());
    const int combo = store_scope * 4 + load_scope;
    switch (combo) {
#define CASE(S, L) case S * 4 + L: hipLaunchKernelGGL((lg_k_xcd_handover<S, L>), dim3(256), dim3(256), 0, nullptr, a); break;
        CASE(0, 0) CASE(0, 1) CASE(0, 2) CASE(0, 3) CASE(1, 0) CASE(1, 1) CASE(1, 2) CASE(1, 3)
        CASE(2, 0) CASE(2, 1) CASE(2, 2) CASE(2, 3) CASE(3, 0) CASE(3, 1) CASE(3, 2) CASE(3, 3)
#undef CASE
    }
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipDeviceSynchronize());
    HIP_TRY(hipMemcpy(res, a.res, (size_t)n * 16, hipMemcpyDeviceToHost));
    return 0;
}

// ---- the XCD-partitioned feed-forward half on its own (tests, timing) ------------------------------
// x_out = x + rmsnorm(dout) * w_post; h = rmsnorm(x_out) * w_pre; act = gelu(gate . q8(h)) * (up . q8(h));
// out = down . q8(act): lg_k_ffn_xcd on host data, the 8 slabs added here in tree order.
extern "C" int lg_hip_down_m(const float *act, const void *down, int rows, int E, int FF, int join, float *out, int repeats, float *kernel_ms) {
    if (!act || !down || !out) return fail(-1, "down_m: null argument");
    const DownMGeo g = lg_down_m_geo(E, FF);
    if (rows < 4 || rows > LG_HIP_MAX_ROWS || !down_m_shape(g)) return fail(-2, "down_m: rows %d (4..%d), E %d, FF %d: no instantiation for this shape", rows, LG_HIP_MAX_ROWS, E, FF);
    if (lg_hip_device_count() < 1) return fail(-3, "down_m: no HIP device");
    Scratch sc;
    std::vector<uint8_t> stage(256 * g.wg_bytes);
    uint8_t *dw; float *dx, *dslabs; uint32_t *dq; DownMSync *dsync; StepCtl *ctl;
    const size_t n = (size_t)rows * E;
    if (sc.get(&dw, 256 * g.wg_bytes) || sc.get(&dx, (size_t)rows * FF) || sc.get(&dslabs, 4 * n) || sc.get(&dq, (size_t)(FF / 32) * LG_MU_DWORDS) ||
        sc.get(&dsync, (size_t)1) || sc.get(&ctl, (size_t)1)) return -7;
    HIP_TRY(hipMemset(dsync, 0, sizeof(DownMSync)));
    HIP_TRY(hipMemset(ctl, 0, sizeof(StepCtl)));
    pack_down_m((const uint8_t *)down, g, stage.data());
    HIP_TRY(hipMemcpy(dw, stage.data(), 256 * g.wg_bytes, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(dx, act, (size_t)rows * FF * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemset(dq, 0, (size_t)(FF / 32) * LG_MU_DWORDS * 4));
    hipStream_t st;
    HIP_TRY(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
    lg_hip_model shim;
    shim.stream = st;
    Launcher lx{ &shim, false };
    DownMArgs a{ dw, dq, dslabs, E, FF, join ? dsync : nullptr, ctl, 1 << 16 };
    hipEvent_t e0 = nullptr, e1 = nullptr;
    auto body = [&]() -> int {
        HIP_TRY(hipEventCreate(&e0)); HIP_TRY(hipEventCreate(&e1));
        hipLaunchKernelGGL(lg_k_quant_mu, dim3((rows * (FF / 32) * 8 + LG_WG - 1) / LG_WG), dim3(LG_WG), 0, st, dx, rows, FF, dq);
        for (int r = 0; r < repeats + 1 && !lx.rc; ++r) {
            if (r == 1) HIP_TRY(hipEventRecord(e0, st));
            switch (rows) {
#define CASE(M) case M: launch_down_m<M>(lx, a); break;
                CASE(4) CASE(5) CASE(6) CASE(7) CASE(8)
#undef CASE
            }
        }
        if (lx.rc) return lx.rc;
        HIP_TRY(hipEventRecord(e1, st));
        HIP_TRY(hipStreamSynchronize(st));
        HIP_TRY(hipGetLastError());
        float t = 0;
        if (repeats > 0) HIP_TRY(hipEventElapsedTime(&t, e0, e1));
        if (kernel_ms) *kernel_ms = repeats > 0 ? t / repeats : 0.0f;
        return 0;
    };
    int rc = body();
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipStreamDestroy(st);
    if (rc) return rc;
    std::vector<float> slabs(4 * n);
    HIP_TRY(hipMemcpy(slabs.data(), dslabs, 4 * n * 4, hipMemcpyDeviceToHost));
    StepCtl c;
    HIP_TRY(hipMemcpy(&c, ctl, sizeof c, hipMemcpyDeviceToHost));
    { const int erc = step_err("down_m", c.err); if (erc) return erc; }
    for (size_t i = 0; i < n; ++i) out[i] = join ? slabs[i] : (slabs[i] + slabs[n + i]) + (slabs[2 * n + i] + slabs[3 * n + i]);    // (what the consumer kernel does)
    return 0;
}

// Gate/up + GeGLU of a verify block in isolation (tests): `rows` float rows of E are quantized as the step's row
// kernel does it (the q8 order of the kernel that follows: lg_k_geglu_t for 1..3 rows, lg_k_geglu_m for 4..8), then
// the kernel runs on gate / up (FF plain q4_0 rows of E each) and the q8 of gelu(gate) * up comes back in natural order.
extern "C" int lg_hip_gate_up_geglu(const float *x, const void *gate, const void *up, int rows, int E, int FF,
                                    int8_t *aq, float *ad, int32_t *asum, int repeats, float *kernel_ms) {
    if (!x || !gate || !up) return fail(-1, "gate_up_geglu: null argument");
    if (rows < 1 || rows > LG_HIP_MAX_ROWS || E < 256 || E % 256 || E > 4096 || FF < 32 || FF % 32 || lg_segments(E) != 8)
        return fail(-2, "gate_up_geglu: rows %d (1..%d), E %d (a multiple of 256 up to 4096), FF %d (a multiple of 32)", rows, LG_HIP_MAX_ROWS, E, FF);
    if (lg_hip_device_count() < 1) return fail(-3, "gate_up_geglu: no HIP device");
    const size_t rb = (size_t)(E / 32) * 18;
    std::vector<const uint8_t *> wrows;
    for (int t = 0; t < FF / 32; ++t) {
        for (int r = 0; r < 32; ++r) wrows.push_back((const uint8_t *)gate + ((size_t)t * 32 + r) * rb);
        for (int r = 0; r < 32; ++r) wrows.push_back((const uint8_t *)up + ((size_t)t * 32 + r) * rb);
    }
    std::vector<uint8_t> stage(lg_hip_repacked_bytes(E, 2 * FF));
    if (stage.empty()) return fail(-2, "gate_up_geglu: cannot tile a %d x %d matrix", 2 * FF, E);
    repack_rowblocks(wrows.data(), E, 2 * FF, stage.data());
    Scratch sc;
    uint8_t *dw; float *dx; int8_t *dq, *dgq; StepCtl *ctl;
    const size_t qbytes = (size_t)(E / 32) * LG_MU_DWORDS * 4 + (size_t)rows * E * 2;     // (room for either block order)
    if (sc.get(&dw, stage.size()) || sc.get(&dx, (size_t)rows * E) || sc.get(&dq, qbytes) || sc.get(&dgq, (size_t)rows * FF * 5 / 4) || sc.get(&ctl, (size_t)1)) return -7;
    HIP_TRY(hipMemcpy(dw, stage.data(), stage.size(), hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(dx, x, (size_t)rows * E * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemset(dq, 0, qbytes));                        // (row slots past the block are read as operand rows of the matrix cores)
    HIP_TRY(hipMemset(ctl, 0, sizeof(StepCtl)));
    hipStream_t st;
    HIP_TRY(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
    RowArgs s{};
    s.x = dx; s.dparts = 1; s.q = dq; s.E = E; s.eps = 1e-6f; s.q_units = rows >= 4 ? 2 : 1;
    GegluArgs a{ dw, E, FF, dq, dgq, 0 };
    hipEvent_t e0 = nullptr, e1 = nullptr;
    auto body = [&]() -> int {
        HIP_TRY(hipEventCreate(&e0)); HIP_TRY(hipEventCreate(&e1));
        int rc = 0;
        auto run = [&](auto tag) {
            constexpr int M = decltype(tag)::value;
            rows_isolated<M>(st, s, ctl);
            for (int r = 0; r < repeats + 1; ++r) {
                if (r == 1) (void)hipEventRecord(e0, st);
                if constexpr (M >= 4) {
                    const size_t lds = (size_t)(E / 32) * LG_MU_DWORDS * 4;
                    rc = set_lds(lg_k_geglu_m<M>, lds);
                    if (rc) return;
                    hipLaunchKernelGGL((lg_k_geglu_m<M>), dim3(FF / 32), dim3(512), lds, st, LG_GEGLU_FIELDS(LG_XA, a) 0);
                } else hipLaunchKernelGGL((lg_k_geglu_t<M>), dim3(FF / 32), dim3(512), 0, st, LG_GEGLU_FIELDS(LG_XA, a) 0);
            }
        };
        switch (rows) {
#define CASE(M) case M: run(std::integral_constant<int, M>{}); break;
            CASE(1) CASE(2) CASE(3) CASE(4) CASE(5) CASE(6) CASE(7) CASE(8)
#undef CASE
        }
        if (rc) return rc;
        HIP_TRY(hipEventRecord(e1, st));
        HIP_TRY(hipStreamSynchronize(st));
        HIP_TRY(hipGetLastError());
        float t = 0;
        if (repeats > 0) HIP_TRY(hipEventElapsedTime(&t, e0, e1));
        if (kernel_ms) *kernel_ms = repeats > 0 ? t / repeats : 0.0f;
        return 0;
    };
    int rc = body();
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipStreamDestroy(st);
    if (rc) return rc;
    return read_back_q8(dgq, rows, FF, aq, ad, asum);
}

extern "C" int lg_hip_ffn_xcd(const float *x, const float *dout, const float *w_post, const float *w_pre,
                              const void *gate, const void *up, const void *down, int rows, int E, int FF, float eps,
                              float *x_out, float *act, float *out, int repeats, float *kernel_ms, int flush_mb, int delay_w, int64_t *stamps) {
    if (!x || !dout || !w_post || !w_pre || !gate || !up || !down) return fail(-1, "ffn_xcd: null input");
    const XffnGeo g = lg_xffn_geo(E, FF);
    const int cls = xffn_class_of(g);
    if (rows < 4 || rows > LG_HIP_MAX_ROWS || cls < 0) return fail(-2, "ffn_xcd: rows %d (4..%d), E %d, FF %d: no instantiation for this shape", rows, LG_HIP_MAX_ROWS, E, FF);
    if (lg_hip_device_count() < 1) return fail(-3, "ffn_xcd: no HIP device");
    if (cu_count() != LG_XCDS * LG_XCD_WGS) return fail(-3, "ffn_xcd: the kernel needs %d compute units in %d XCDs, this device has %d", LG_XCDS * LG_XCD_WGS, LG_XCDS, cu_count());
    Scratch sc;
    std::vector<uint8_t> stage(256 * (g.gu_bytes > g.dn_bytes ? g.gu_bytes : g.dn_bytes));
    uint8_t *dgu, *ddn; float *dx, *dd, *dwp, *dwr, *dxo, *dslabs, *dact; uint32_t *dxq; XcdSync *dsync; StepCtl *ctl;
    const size_t n = (size_t)rows * E;
    if (sc.get(&dgu, 256 * g.gu_bytes) || sc.get(&ddn, 256 * g.dn_bytes) || sc.get(&dx, n) || sc.get(&dd, n) || sc.get(&dwp, (size_t)E) ||
        sc.get(&dwr, (size_t)E) || sc.get(&dxo, n) || sc.get(&dslabs, LG_XCDS * n) || sc.get(&dact, (size_t)LG_XCDS * rows * g.C) ||
        sc.get(&dxq, (size_t)LG_XCDS * g.nb * LG_MU_DWORDS) || sc.get(&dsync, (size_t)1) || sc.get(&ctl, (size_t)1)) return -7;
    xffn_pack_gu((const uint8_t *)gate, (const uint8_t *)up, g, stage.data());
    HIP_TRY(hipMemcpy(dgu, stage.data(), 256 * g.gu_bytes, hipMemcpyHostToDevice));
    xffn_pack_dn((const uint8_t *)down, g, stage.data());
    HIP_TRY(hipMemcpy(ddn, stage.data(), 256 * g.dn_bytes, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(dx, x, n * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(dd, dout, n * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(dwp, w_post, (size_t)E * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(dwr, w_pre, (size_t)E * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemset(dsync, 0, sizeof(XcdSync)));
    HIP_TRY(hipMemset(dxq, 0, (size_t)LG_XCDS * g.nb * LG_MU_DWORDS * 4));
    HIP_TRY(hipMemset(ctl, 0, sizeof(StepCtl)));
    hipStream_t st;
    HIP_TRY(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
    lg_hip_model shim;
    shim.stream = st;
    Launcher lx{ &shim, false };
    // measurement runs: something else streams through the caches between two launches (the step's weights never
    // come from a cache), and every workgroup records the device clock at its phase boundaries
    unsigned char *dflush = nullptr;
    unsigned long long *dstamps = nullptr;
    if (flush_mb > 0 && sc.get(&dflush, (size_t)flush_mb << 20)) return -7;
    if (stamps && sc.get(&dstamps, (size_t)512 * LG_XFFN_STAMPS)) return -7;
    if (dstamps) HIP_TRY(hipMemset(dstamps, 0, (size_t)512 * LG_XFFN_STAMPS * 8));
    XffnArgs f{ dgu, ddn, dx, dd, dwp, dwr, dxo, dslabs, dxq, dact, dsync, ctl, E, FF, eps, 1 << 16, delay_w, dstamps };
    hipEvent_t e0 = nullptr, e1 = nullptr;
    auto body = [&]() -> int {
        HIP_TRY(hipEventCreate(&e0)); HIP_TRY(hipEventCreate(&e1));
        for (int r = 0; r < repeats + 1 && !lx.rc; ++r) {
            if (r == 1) HIP_TRY(hipEventRecord(e0, st));
            if (dflush) HIP_TRY(hipMemsetAsync(dflush, r, (size_t)flush_mb << 20, st));
            switch (rows) {
#define CASE(M) case M: launch_xffn<M>(lx, f, cls); break;
                CASE(4) CASE(5) CASE(6) CASE(7) CASE(8)
#undef CASE
            }
        }
        if (lx.rc) return lx.rc;
        HIP_TRY(hipEventRecord(e1, st));
        HIP_TRY(hipStreamSynchronize(st));
        HIP_TRY(hipGetLastError());
        float t = 0;
        if (repeats > 0) HIP_TRY(hipEventElapsedTime(&t, e0, e1));
        if (kernel_ms) *kernel_ms = repeats > 0 ? t / repeats : 0.0f;
        return 0;
    };
    int rc = body();
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipStreamDestroy(st);
    if (rc) return rc;
    StepCtl c;
    HIP_TRY(hipMemcpy(&c, ctl, sizeof c, hipMemcpyDeviceToHost));
    if (c.err) return fail(-9, "ffn_xcd: the kernel reported %s%s (err 0x%x)", (c.err & LG_XFFN_ERR_PLACE) ? "a workgroup on an unexpected XCD " : "",
                           (c.err & LG_XFFN_ERR_WAIT) ? "a hand-over that was given up" : "", c.err);
    if (stamps) HIP_TRY(hipMemcpy(stamps, dstamps, (size_t)512 * LG_XFFN_STAMPS * 8, hipMemcpyDeviceToHost));
    if (x_out) HIP_TRY(hipMemcpy(x_out, dxo, n * 4, hipMemcpyDeviceToHost));
    if (act) {                                            // [rows][FF] from the 8 per-XCD pieces [rows][FF/8]
        std::vector<float> pieces((size_t)LG_XCDS * rows * g.C);
        HIP_TRY(hipMemcpy(pieces.data(), dact, pieces.size() * 4, hipMemcpyDeviceToHost));
        for (int xc = 0; xc < LG_XCDS; ++xc)
            for (int j = 0; j < rows; ++j)
                memcpy(act + (size_t)j * FF + (size_t)xc * g.C, pieces.data() + ((size_t)xc * rows + j) * g.C, (size_t)g.C * 4);
    }
    if (out) {
        std::vector<float> p(LG_XCDS * n);
        HIP_TRY(hipMemcpy(p.data(), dslabs, p.size() * 4, hipMemcpyDeviceToHost));
        for (size_t i = 0; i < n; ++i)
            out[i] = ((p[i] + p[n + i]) + (p[2 * n + i] + p[3 * n + i])) + ((p[4 * n + i] + p[5 * n + i]) + (p[6 * n + i] + p[7 * n + i]));
    }
    return 0;
}
