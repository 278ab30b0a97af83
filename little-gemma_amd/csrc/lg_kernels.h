// lg_kernels.h — the kernels of one verify step (rows = M draft-block rows, M <= 8).
//
// Per layer the step is a chain of matmul phases over pre-tiled q4_0 weights; everything
// between two matmuls (RMSNorm, residual add, output scale, GeGLU, PLE mixing, q8 activation
// quantization) is fused into the prologue or epilogue of the matmul kernels, so the
// reference's ~25 launches per layer (src/cuda/prefill-kernel.cuh:381-541) become 8:
//   qkv -> attention tiles -> attention merge -> o -> gate/up+GeGLU -> down -> ple gate -> ple proj
// Every kernel reads the block position from device memory (StepCtl), so launch parameters never
// change between steps and the whole step is captured once into a graph.
#pragma once
#include "lg_device.h"

struct StepCtl {            // device-resident step state
    int pos;                // position of row 0 of the current block
    int step;               // index of the current block in the token schedule
    int err;                // set by kernels on impossible arguments
    int pad;
};

// Where a matmul phase gets its M activation rows from.  The prologue turns this into q8 rows
// (int8 values + per-32 {scale, sum}) in LDS; workgroup 0 also writes the updated residual.
struct ActSrc {
    const float   *x;        // [M][E] residual stream; nullptr when the rows are embeddings
    const float   *dout;     // [M][E] previous sub-layer output to be rmsnormed and added, or nullptr
    const float   *w_post;   // [E] norm weight for dout
    const float   *os;       // scalar layer_output_scale applied after the add, or nullptr
    float         *x_out;    // [M][E] updated residual (written by workgroup 0), or nullptr
    const float   *w_pre;    // [E] norm weight applied before quantization, or nullptr (quantize x itself)
    float         *h_out;    // [M][E] normed rows before quantization (written by workgroup 0), or nullptr
    const uint8_t *emb;      // tiled token_embd: rows are token lookups scaled by emb_scale
    const int32_t *toks;     // token schedule base ([n_steps][M])
    int            emb_nit;
    float          emb_scale;
    int            E;
    float          eps;
};

// ---------------------------------------------------------------------------------------------
// Prologue: M rows -> q8.  One wavefront per row (rows round-robin over the 4 wavefronts), the
// row lives in registers as float4 per lane, lane l holds elements 256*v + 4*l .. +3.
// qdst/dsdst may point to LDS or global memory.
template <int M>
__device__ __forceinline__ void lg_act_prologue(const ActSrc &s, const StepCtl *ctl, int8_t *qdst,
                                                float2 *dsdst, bool writer) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int E = s.E, nv = E >> 8;
    for (int j = wave; j < M; j += LG_WG / 64) {
        float4 xv[LG_MAXV];
        if (s.emb) {
            const int tok = s.toks[ctl->step * M + j];
            #pragma unroll
            for (int v = 0; v < LG_MAXV; ++v) if (v < nv) {
                float4 t = lg_tiled_deq4(s.emb, s.emb_nit, tok, 256 * v + 4 * lane);
                xv[v] = make_float4(t.x * s.emb_scale, t.y * s.emb_scale, t.z * s.emb_scale, t.w * s.emb_scale);
            }
        } else {
            const float4 *xr = (const float4 *)(s.x + (size_t)j * E);
            #pragma unroll
            for (int v = 0; v < LG_MAXV; ++v) if (v < nv) xv[v] = xr[64 * v + lane];
        }
        if (s.dout) {
            float4 dv[LG_MAXV];
            const float4 *dr = (const float4 *)(s.dout + (size_t)j * E);
            float ss = 0.0f;
            #pragma unroll
            for (int v = 0; v < LG_MAXV; ++v) if (v < nv) { dv[v] = dr[64 * v + lane]; ss = lg_sumsq4(dv[v], ss); }
            ss = lg_wave_sum64(ss);
            const float sc = 1.0f / sqrtf(ss / (float)E + s.eps);
            const float4 *wr = (const float4 *)s.w_post;
            const bool has_os = s.os != nullptr;
            const float osv = has_os ? s.os[0] : 1.0f;
            #pragma unroll
            for (int v = 0; v < LG_MAXV; ++v) if (v < nv) {
                const float4 w = wr[64 * v + lane];
                float4 r;
                r.x = xv[v].x + dv[v].x * sc * w.x;  r.y = xv[v].y + dv[v].y * sc * w.y;
                r.z = xv[v].z + dv[v].z * sc * w.z;  r.w = xv[v].w + dv[v].w * sc * w.w;
                if (has_os) { r.x = r.x * osv; r.y = r.y * osv; r.z = r.z * osv; r.w = r.w * osv; }
                xv[v] = r;
            }
        }
        if (writer && s.x_out) {
            float4 *xo = (float4 *)(s.x_out + (size_t)j * E);
            #pragma unroll
            for (int v = 0; v < LG_MAXV; ++v) if (v < nv) xo[64 * v + lane] = xv[v];
        }
        if (s.w_pre) {
            float ss = 0.0f;
            #pragma unroll
            for (int v = 0; v < LG_MAXV; ++v) if (v < nv) ss = lg_sumsq4(xv[v], ss);
            ss = lg_wave_sum64(ss);
            const float sc = 1.0f / sqrtf(ss / (float)E + s.eps);
            const float4 *wr = (const float4 *)s.w_pre;
            #pragma unroll
            for (int v = 0; v < LG_MAXV; ++v) if (v < nv) {
                const float4 w = wr[64 * v + lane];
                xv[v] = make_float4(xv[v].x * sc * w.x, xv[v].y * sc * w.y, xv[v].z * sc * w.z, xv[v].w * sc * w.w);
            }
        }
        if (writer && s.h_out) {
            float4 *ho = (float4 *)(s.h_out + (size_t)j * E);
            #pragma unroll
            for (int v = 0; v < LG_MAXV; ++v) if (v < nv) ho[64 * v + lane] = xv[v];
        }
        uint32_t *qrow = (uint32_t *)(qdst + (size_t)j * E);
        float2 *drow = dsdst + (size_t)j * (E >> 5);
        #pragma unroll
        for (int v = 0; v < LG_MAXV; ++v) if (v < nv) {
            float d; int sum;
            const uint32_t packed = lg_quant4_8lanes(xv[v], &d, &sum);
            qrow[64 * v + lane] = packed;
            if ((lane & 7) == 0) drow[(64 * v + lane) >> 3] = make_float2(d, __int_as_float(sum));
        }
    }
}

// Copy M already-quantized rows (int8 + {scale,sum}) from global memory into LDS.
template <int M>
__device__ __forceinline__ void lg_load_q8(const int8_t *q, const float2 *ds, int k, int8_t *lq, float2 *lds_ds) {
    const int n16 = M * k / 16;
    const uint4 *src = (const uint4 *)q;
    uint4 *dst = (uint4 *)lq;
    for (int i = threadIdx.x; i < n16; i += LG_WG) dst[i] = src[i];
    const int nd = M * (k >> 5);
    for (int i = threadIdx.x; i < nd; i += LG_WG) lds_ds[i] = ds[i];
}

// ---------------------------------------------------------------------------------------------
// One group of 8 weight rows against M q8 activation rows held in LDS.  Lane = r*8 + c owns row
// r, K segment c.  On return every lane of a row holds that row's M results (segment tree done).
template <int M, bool DUMP>
__device__ __forceinline__ void lg_mm_group(const uint8_t *__restrict__ wgroup, int nit, const int8_t *act,
                                            const float2 *actds, int k, float (&acc)[M], int lane,
                                            int32_t *dots, int m, int row) {
    const int c = lane & 7, nb = k >> 5;
    const uint8_t *pq = wgroup + lane * 16;
    const uint8_t *ps = wgroup + 1024 + lane * 2;
    #pragma unroll
    for (int j = 0; j < M; ++j) acc[j] = 0.0f;
    #pragma unroll 4
    for (int it = 0; it < nit; ++it) {
        const uint4 wq = *(const uint4 *)(pq + (size_t)it * LG_TILE);
        const float dw = lg_h2f(*(const uint16_t *)(ps + (size_t)it * LG_TILE));
        const int b = c * nit + it;
        #pragma unroll
        for (int j = 0; j < M; ++j) {
            const float2 ds = actds[j * nb + b];
            const int dot = lg_block_dot(wq, act + (size_t)j * k + b * 32, __float_as_int(ds.y));
            if (DUMP) dots[((size_t)j * m + row) * nb + b] = dot;
            acc[j] = lg_fmaf(ds.x * dw, (float)dot, acc[j]);
        }
    }
    #pragma unroll
    for (int j = 0; j < M; ++j) acc[j] = lg_sum8(acc[j]);
}

template <int M>
__device__ __forceinline__ float lg_pick(const float (&acc)[M], int j) {
    float v = acc[0];
    #pragma unroll
    for (int t = 1; t < M; ++t) if (j == t) v = acc[t];
    return v;
}

struct MmArgs {
    const uint8_t *w;        // tiled weights
    int            k, m;     // row length, rows
    float         *out;      // [M][m]
    const int8_t  *q_in;     // pre-quantized input rows (SRC_Q8), [M][k]
    const float2  *ds_in;    //   their {scale,sum}, [M][k/32]
    int32_t       *dots;     // DUMP only: [M][m][k/32]
};

enum { SRC_ACT = 0, SRC_Q8 = 1 };

// Plain matmul: out[j][i] f32.  Workgroup = 4 wavefronts = 4 row groups = 32 output rows.
template <int M, int SRC, bool DUMP>
__global__ __launch_bounds__(LG_WG) void lg_k_mm(MmArgs a, ActSrc s, const StepCtl *ctl) {
    extern __shared__ __align__(16) unsigned char smem[];
    int8_t *lq = (int8_t *)smem;
    float2 *lds = (float2 *)(smem + (size_t)M * a.k);
    if (SRC == SRC_ACT) lg_act_prologue<M>(s, ctl, lq, lds, blockIdx.x == 0);
    else lg_load_q8<M>(a.q_in, a.ds_in, a.k, lq, lds);
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = blockIdx.x * 4 + wave, nit = a.k >> 8;
    if (g * 8 >= a.m) return;
    float acc[M];
    const int row = g * 8 + (lane >> 3);
    lg_mm_group<M, DUMP>(a.w + (size_t)g * nit * LG_TILE, nit, lq, lds, a.k, acc, lane, a.dots, a.m, row);
    const int c = lane & 7;
    if (c < M) a.out[(size_t)c * a.m + row] = lg_pick<M>(acc, c);
}

// Gate/up matmul with the GeGLU and the q8 quantization of its result as epilogue.  The tiled
// matrix interleaves 32 gate rows with the 32 up rows of the same indices, so a workgroup owns
// one 32-wide quantization group: wavefront w computes gate and up rows 8w..8w+7 of it.
struct GegluArgs {
    const uint8_t *w;        // tiled [2*n_ff][k], virtual row order: 32 gate, 32 up, 32 gate, ...
    int            k, n_ff;
    int8_t        *gq;       // [M][n_ff]
    float2        *gds;      // [M][n_ff/32]
};
template <int M>
__global__ __launch_bounds__(LG_WG) void lg_k_mm_geglu(GegluArgs a, ActSrc s, const StepCtl *ctl) {
    extern __shared__ __align__(16) unsigned char smem[];
    int8_t *lq = (int8_t *)smem;
    float2 *lds = (float2 *)(smem + (size_t)M * a.k);
    __shared__ float gbuf[LG_HIP_MAX_ROWS_DEV][32];
    lg_act_prologue<M>(s, ctl, lq, lds, blockIdx.x == 0);
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nit = a.k >> 8;
    const int t = blockIdx.x;                               // 32-wide slice of n_ff
    float gate[M], up[M];
    const size_t gstride = (size_t)nit * LG_TILE;
    lg_mm_group<M, false>(a.w + ((size_t)t * 8 + wave) * gstride, nit, lq, lds, a.k, gate, lane, nullptr, 0, 0);
    lg_mm_group<M, false>(a.w + ((size_t)t * 8 + 4 + wave) * gstride, nit, lq, lds, a.k, up, lane, nullptr, 0, 0);
    const int c = lane & 7, r = lane >> 3;
    if (c < M) gbuf[c][wave * 8 + r] = lg_gelu(lg_pick<M>(gate, c)) * lg_pick<M>(up, c);
    __syncthreads();
    // quantize: half-wavefront per row j, one value per lane
    for (int j = threadIdx.x >> 5; j < M; j += LG_WG / 32) {
        const int i = threadIdx.x & 31;
        float d; int sum;
        const int q = lg_quant1_32lanes(gbuf[j][i], &d, &sum);
        a.gq[(size_t)j * a.n_ff + t * 32 + i] = (int8_t)q;
        if (i == 0) a.gds[(size_t)j * (a.n_ff >> 5) + t] = make_float2(d, __int_as_float(sum));
    }
}

// PLE gate: inp_gate matmul on the q8 of the updated residual, then gelu(.) * ipl and q8.
// ipl for this layer is finished here from the raw per_layer_model_proj output and the token's
// per-layer embedding row (the reference builds it once per step in build_per_layer_n,
// src/cuda/model-cuda.cuh:1121-1147): ipl = (rmsnorm(proj/sqrt(E)) * w + tok*sqrt(ple)) / sqrt(2).
struct PleGateArgs {
    const uint8_t *w;        // tiled inp_gate [ple][E]
    int            k, ple;
    const float   *pmp_raw;  // [M][n_layer*ple] raw projection
    int            layer, n_layer;
    const float   *proj_norm;     // [ple]
    const uint8_t *pte;      // per_layer_token_embd, plain q4_0 rows of n_layer*ple
    const int32_t *toks;
    float          pscale, tscale, rsqrt2, eps;
    int8_t        *pq;       // [M][ple]
    float2        *pds;      // [M][ple/32]
};
template <int M>
__global__ __launch_bounds__(LG_WG) void lg_k_mm_plegate(PleGateArgs a, ActSrc s, const StepCtl *ctl) {
    extern __shared__ __align__(16) unsigned char smem[];
    int8_t *lq = (int8_t *)smem;
    float2 *lds = (float2 *)(smem + (size_t)M * a.k);
    float *ipl = (float *)(lds + (size_t)M * (a.k >> 5));        // [M][ple]
    __shared__ float gbuf[LG_HIP_MAX_ROWS_DEV][32];
    lg_act_prologue<M>(s, ctl, lq, lds, blockIdx.x == 0);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nit = a.k >> 8;
    const int ple = a.ple;
    for (int j = wave; j < M; j += LG_WG / 64) {              // one wavefront per row: slice norm
        const float *pr = a.pmp_raw + (size_t)j * a.n_layer * ple + (size_t)a.layer * ple;
        float ss = 0.0f;
        for (int v = 0; 256 * v < ple; ++v) {
            const int e0 = 256 * v + 4 * lane;
            if (e0 < ple) {
                float4 p = *(const float4 *)(pr + e0);
                p = make_float4(p.x * a.pscale, p.y * a.pscale, p.z * a.pscale, p.w * a.pscale);
                ss = lg_sumsq4(p, ss);
            }
        }
        ss = lg_wave_sum64(ss);
        const float sc = 1.0f / sqrtf(ss / (float)ple + a.eps);
        const int tok = a.toks[ctl->step * M + j];
        const uint8_t *trow = a.pte + (size_t)tok * ((size_t)a.n_layer * ple / 32 * 18);
        for (int e = lane; e < ple; e += 64) {
            const float p = pr[e] * a.pscale * sc * a.proj_norm[e];
            const float tk = lg_q4_0_elem(trow, a.layer * ple + e) * a.tscale;
            ipl[j * ple + e] = (p + tk) * a.rsqrt2;
        }
    }
    __syncthreads();
    const int g = blockIdx.x * 4 + wave;                    // ple/8 groups, 4 per workgroup
    float acc[M];
    lg_mm_group<M, false>(a.w + (size_t)g * nit * LG_TILE, nit, lq, lds, a.k, acc, lane, nullptr, 0, 0);
    const int c = lane & 7, r = lane >> 3;
    if (c < M) gbuf[c][wave * 8 + r] = lg_gelu(lg_pick<M>(acc, c)) * ipl[c * ple + g * 8 + r];
    __syncthreads();
    for (int j = threadIdx.x >> 5; j < M; j += LG_WG / 32) {
        const int i = threadIdx.x & 31;
        float d; int sum;
        const int q = lg_quant1_32lanes(gbuf[j][i], &d, &sum);
        a.pq[(size_t)j * ple + blockIdx.x * 32 + i] = (int8_t)q;
        if (i == 0) a.pds[(size_t)j * (ple >> 5) + blockIdx.x] = make_float2(d, __int_as_float(sum));
    }
}

// Rows -> q8 in global memory (final norm before lm_head; also the stand-alone quantizer).
struct QuantArgs { int8_t *q; float2 *ds; };
template <int M>
__global__ __launch_bounds__(LG_WG) void lg_k_act_quant(QuantArgs a, ActSrc s, const StepCtl *ctl) {
    lg_act_prologue<M>(s, ctl, a.q, a.ds, true);
}

// Plain q8 quantization of n32 groups of 32 floats (no norm): 8 lanes per group.
__global__ __launch_bounds__(LG_WG) void lg_k_quant_flat(const float *x, int n32, int8_t *q, float2 *ds) {
    const int g = (blockIdx.x * LG_WG + threadIdx.x) >> 3, l = threadIdx.x & 7;
    const bool live = g < n32;
    const float4 h = live ? ((const float4 *)x)[(size_t)g * 8 + l] : make_float4(0, 0, 0, 0);
    float d; int sum;
    const uint32_t packed = lg_quant4_8lanes(h, &d, &sum);
    if (!live) return;
    ((uint32_t *)q)[(size_t)g * 8 + l] = packed;
    if (l == 0) ds[g] = make_float2(d, __int_as_float(sum));
}

// lm_head: logits of 32 vocabulary rows per workgroup, soft cap, per-workgroup argmax partial
// (first maximum: lower index wins ties, src/cuda/model-cuda.cuh:703-720).
struct HeadArgs {
    const uint8_t *w; int k, n_vocab;
    const int8_t *q_in; const float2 *ds_in;
    float softcap;
    float *logits;          // [M][n_vocab] or nullptr
    float *pval; int *pidx; // [n_vocab/32][M]
};
template <int M>
__global__ __launch_bounds__(LG_WG) void lg_k_mm_head(HeadArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    int8_t *lq = (int8_t *)smem;
    float2 *lds = (float2 *)(smem + (size_t)M * a.k);
    __shared__ float vbuf[LG_HIP_MAX_ROWS_DEV][32];
    lg_load_q8<M>(a.q_in, a.ds_in, a.k, lq, lds);
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nit = a.k >> 8;
    const int g = blockIdx.x * 4 + wave;
    float acc[M];
    lg_mm_group<M, false>(a.w + (size_t)g * nit * LG_TILE, nit, lq, lds, a.k, acc, lane, nullptr, 0, 0);
    const int c = lane & 7, r = lane >> 3;
    if (c < M) {
        float v = lg_pick<M>(acc, c);
        if (a.softcap > 0.0f) v = a.softcap * lg_tanhf(v / a.softcap);
        vbuf[c][wave * 8 + r] = v;
        if (a.logits) a.logits[(size_t)c * a.n_vocab + g * 8 + r] = v;
    }
    __syncthreads();
    for (int j = threadIdx.x >> 5; j < M; j += LG_WG / 32) {
        const int i = threadIdx.x & 31;
        float v = vbuf[j][i];
        int idx = blockIdx.x * 32 + i;
        for (int o = 1; o < 32; o <<= 1) {
            const float ov = __shfl_xor(v, o);
            const int oi = __shfl_xor(idx, o);
            if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
        }
        if (i == 0) { a.pval[(size_t)blockIdx.x * M + j] = v; a.pidx[(size_t)blockIdx.x * M + j] = idx; }
    }
}

// Final argmax over the per-workgroup partials, accept rule, state advance
// (src/cuda/mtp-kernel.cuh:112-118 done on the device).
struct AcceptArgs {
    const float *pval; const int *pidx; int n_part;
    const int32_t *toks;     // schedule base
    int32_t *out;            // [n_steps][M]
    int32_t *adv;            // [n_steps]
    const float *hidden_rows; float *g_hidden; int E;
};
template <int M>
__global__ __launch_bounds__(LG_WG) void lg_k_accept(AcceptArgs a, StepCtl *ctl) {
    __shared__ float sv[LG_WG];
    __shared__ int si[LG_WG];
    __shared__ int best[LG_HIP_MAX_ROWS_DEV];
    __shared__ int s_adv;
    const int step = ctl->step;
    for (int j = 0; j < M; ++j) {
        float v = -INFINITY; int idx = 0x7fffffff;
        for (int p = threadIdx.x; p < a.n_part; p += LG_WG) {
            const float pv = a.pval[(size_t)p * M + j]; const int pi = a.pidx[(size_t)p * M + j];
            if (pv > v || (pv == v && pi < idx)) { v = pv; idx = pi; }
        }
        sv[threadIdx.x] = v; si[threadIdx.x] = idx;
        __syncthreads();
        for (int s = LG_WG / 2; s > 0; s >>= 1) {
            if ((int)threadIdx.x < s) {
                const float ov = sv[threadIdx.x + s]; const int oi = si[threadIdx.x + s];
                if (ov > sv[threadIdx.x] || (ov == sv[threadIdx.x] && oi < si[threadIdx.x])) { sv[threadIdx.x] = ov; si[threadIdx.x] = oi; }
            }
            __syncthreads();
        }
        if (threadIdx.x == 0) best[j] = si[0];
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        const int32_t *tk = a.toks + (size_t)step * M;
        int adv = 1;
        while (adv < M && best[adv - 1] == tk[adv]) adv++;
        for (int j = 0; j < M; ++j) a.out[(size_t)step * M + j] = best[j];
        a.adv[step] = adv;
        s_adv = adv;
    }
    __syncthreads();
    const int adv = s_adv;
    for (int i = threadIdx.x; i < a.E; i += LG_WG) a.g_hidden[i] = a.hidden_rows[(size_t)(adv - 1) * a.E + i];
    __syncthreads();
    if (threadIdx.x == 0) { ctl->pos += adv; ctl->step = step + 1; }
}

// Prefill blocks skip the head: only the position advances.
__global__ void lg_k_advance(StepCtl *ctl, int rows) { ctl->pos += rows; ctl->step += 1; }

// ---------------------------------------------------------------------------------------------
// Attention.  Keys are processed in tiles of 32 aligned to absolute positions (tile n covers
// positions 32n..32n+31; ring length is a multiple of 32, so a tile never wraps).  One workgroup
// per (kv head, tile): it norms+rotates the queries of the gqa*M (head,row) pairs that share the
// kv head, stages the tile's K and V in LDS once, and writes for each pair the tile's partial
// softmax (max, sum, V-accumulator).  The workgroup whose tile contains new positions also
// produces their K/V rows (k-norm, rotary, v-norm, f16 round) and stores them in the cache.
// Defined order: score = (a0+a1)+(a2+a3), a_c = fma chain over dims i%4==c; m = max over valid
// keys; e = exp(s-m); l = adjacent tree over the 32 key slots; acc[d] = fma chain over valid
// slots ascending.
struct AttnArgs {
    const float *qkv;        // [M][ld] raw projections: q at 0, k at k_off, v at v_off
    int ld, k_off, v_off;
    int H, nkv, hd;
    const float *q_norm, *k_norm;       // [hd]
    const float *rope_tab, *rope_ff;    // [hd/2]; ff may be nullptr
    uint16_t *kc, *vc;       // cache of the layer this one reads
    int seq, kv_dim, window; // ring rows, row width, 0 = global
    int owns;                // 1: this layer's K/V rows are produced and stored here
    int prerotated;          // 1: q already normed+rotated (isolated attention entry point)
    float eps;
    float *pm, *pl, *pacc;   // partials: [M*H][tiles_max], [M*H][tiles_max][hd]
    int tiles_max;
};

__device__ __forceinline__ int lg_win_start(int pos, int window) {
    return (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
}

template <int M>
__global__ __launch_bounds__(LG_WG) void lg_k_attn(AttnArgs a, const StepCtl *ctl) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int hd = a.hd, half = hd >> 1, G = a.H / a.nkv, nq = G * M;
    const int kst = hd + 8;                                   // padded K/V tile row (halves)
    float *qs = (float *)smem;                                // [nq + M][hd]: queries, then new K rows
    uint16_t *kt = (uint16_t *)(qs + (size_t)(nq + M) * hd);  // [32][kst]
    uint16_t *vt = kt + 32 * kst;                             // [32][kst]
    float *es = (float *)(vt + 32 * kst);                     // [nq][32]
    uint32_t *vmask = (uint32_t *)(es + nq * 32);             // [nq]
    const int pos = ctl->pos, kvh = blockIdx.y;
    const int start0 = lg_win_start(pos, a.window);
    const int n = (start0 >> 5) + blockIdx.x, n_last = (pos + M - 1) >> 5;
    if (n > n_last) return;
    const int t0 = n << 5;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

    // A: rmsnorm of queries and of the new K / V rows that fall in this tile
    for (int job = wave; job < nq + 2 * M; job += LG_WG / 64) {
        const bool isq = job < nq;
        const int j = isq ? job / G : (job - nq) % M;
        const bool isv = !isq && job >= nq + M;
        if (!isq) { const int t = pos + j; if (!a.owns || t < t0 || t >= t0 + 32) continue; }
        else if (a.prerotated) {
            const float *src = a.qkv + (size_t)j * a.ld + (size_t)(kvh * G + job % G) * hd;
            for (int e = lane; e < hd; e += 64) qs[(size_t)job * hd + e] = src[e];
            continue;
        }
        const float *src = a.qkv + (size_t)j * a.ld +
            (isq ? (size_t)(kvh * G + job % G) * hd : (size_t)(isv ? a.v_off : a.k_off) + (size_t)kvh * hd);
        const float *w = isq ? a.q_norm : (isv ? nullptr : a.k_norm);
        float4 xv[2];
        float ss = 0.0f;
        #pragma unroll
        for (int v = 0; v < 2; ++v) {
            const int e0 = 256 * v + 4 * lane;
            if (e0 < hd) { xv[v] = *(const float4 *)(src + e0); ss = lg_sumsq4(xv[v], ss); }
        }
        ss = lg_wave_sum64(ss);
        const float sc = 1.0f / sqrtf(ss / (float)hd + a.eps);
        #pragma unroll
        for (int v = 0; v < 2; ++v) {
            const int e0 = 256 * v + 4 * lane;
            if (e0 >= hd) continue;
            float4 r;
            if (w) { const float4 ww = *(const float4 *)(w + e0);
                     r = make_float4(xv[v].x * sc * ww.x, xv[v].y * sc * ww.y, xv[v].z * sc * ww.z, xv[v].w * sc * ww.w); }
            else r = make_float4(xv[v].x * sc, xv[v].y * sc, xv[v].z * sc, xv[v].w * sc);
            if (isv) {
                const int t = pos + j;
                uint16_t h4[4] = { lg_f2h(r.x), lg_f2h(r.y), lg_f2h(r.z), lg_f2h(r.w) };
                uint16_t *lv = vt + (t - t0) * kst + e0;
                uint16_t *gv = a.vc + (size_t)(t % a.seq) * a.kv_dim + (size_t)kvh * hd + e0;
                #pragma unroll
                for (int u = 0; u < 4; ++u) { lv[u] = h4[u]; gv[u] = h4[u]; }
            } else {
                float *dst = qs + (size_t)(isq ? job : nq + j) * hd + e0;
                dst[0] = r.x; dst[1] = r.y; dst[2] = r.z; dst[3] = r.w;
            }
        }
    }
    __syncthreads();
    // B: rotary on queries and new K rows (pairs i, i + hd/2), in LDS
    for (int idx = threadIdx.x; idx < (nq + M) * half; idx += LG_WG) {
        const int vec = idx / half, p = idx - vec * half;
        const int j = vec < nq ? vec / G : vec - nq;
        if (vec >= nq) { const int t = pos + j; if (!a.owns || t < t0 || t >= t0 + 32) continue; }
        else if (a.prerotated) continue;
        const float ang = (float)(pos + j) * a.rope_tab[p] / (a.rope_ff ? a.rope_ff[p] : 1.0f);
        float sn, cs;
        lg_sincosf(ang, &sn, &cs);
        float *vp = qs + (size_t)vec * hd;
        const float x0 = vp[p], x1 = vp[p + half];
        vp[p] = x0 * cs - x1 * sn;
        vp[p + half] = x0 * sn + x1 * cs;
    }
    __syncthreads();
    // C: K/V tile into LDS: new K rows from qs (f16 round + cache store), older rows from the cache
    const int last_needed = pos + M - 1;
    for (int idx = threadIdx.x; idx < 32 * (hd >> 2); idx += LG_WG) {
        const int sl = idx / (hd >> 2), e0 = (idx - sl * (hd >> 2)) << 2;
        const int t = t0 + sl;
        uint16_t *lk = kt + sl * kst + e0, *lv = vt + sl * kst + e0;
        const bool fresh = a.owns && t >= pos && t <= last_needed;
        if (fresh) {
            const float *kn = qs + (size_t)(nq + t - pos) * hd + e0;
            uint16_t *gk = a.kc + (size_t)(t % a.seq) * a.kv_dim + (size_t)kvh * hd + e0;
            #pragma unroll
            for (int u = 0; u < 4; ++u) { const uint16_t h = lg_f2h(kn[u]); lk[u] = h; gk[u] = h; }
        } else if (t >= start0 && t <= last_needed) {
            const size_t off = (size_t)(t % a.seq) * a.kv_dim + (size_t)kvh * hd + e0;
            *(uint2 *)lk = *(const uint2 *)(a.kc + off);
            *(uint2 *)lv = *(const uint2 *)(a.vc + off);
        } else {
            *(uint2 *)lk = make_uint2(0, 0);
            *(uint2 *)lv = make_uint2(0, 0);
        }
    }
    __syncthreads();
    // D: scores, tile max, exp, tile sum.  Thread = (key slot, query group of 8).
    {
        const int sl = threadIdx.x & 31, qg = threadIdx.x >> 5, t = t0 + sl;
        for (int qi = qg; qi < nq; qi += LG_WG / 32) {
            const int j = qi / G, pj = pos + j;
            const bool valid = t >= lg_win_start(pj, a.window) && t <= pj;
            float s = -INFINITY;
            if (valid) {
                const float *qv = qs + (size_t)qi * hd;
                const uint16_t *kr = kt + sl * kst;
                float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
                for (int i = 0; i < hd; i += 4) {
                    const float4 q4 = *(const float4 *)(qv + i);
                    const uint2 k2 = *(const uint2 *)(kr + i);
                    a0 = lg_fmaf(q4.x, lg_h2f((uint16_t)(k2.x & 0xFFFF)), a0);
                    a1 = lg_fmaf(q4.y, lg_h2f((uint16_t)(k2.x >> 16)), a1);
                    a2 = lg_fmaf(q4.z, lg_h2f((uint16_t)(k2.y & 0xFFFF)), a2);
                    a3 = lg_fmaf(q4.w, lg_h2f((uint16_t)(k2.y >> 16)), a3);
                }
                s = (a0 + a1) + (a2 + a3);
            }
            const float mx = lg_max_n(s, 32);
            const float e = valid ? lg_expf(s - mx) : 0.0f;
            const float l = lg_sum32(e);
            const unsigned long long bal = __ballot(valid);
            const uint32_t mask = (uint32_t)(threadIdx.x & 32 ? bal >> 32 : bal);
            es[qi * 32 + sl] = e;
            if (sl == 0) {
                vmask[qi] = mask;
                if (mask) {
                    const int head = kvh * G + qi % G;
                    const size_t pi = ((size_t)j * a.H + head) * a.tiles_max + blockIdx.x;
                    a.pm[pi] = mx; a.pl[pi] = l;
                }
            }
        }
    }
    __syncthreads();
    // E: acc[d] = sum over valid slots of e * V[slot][d]
    {
        const int parts = hd >= LG_WG ? 1 : LG_WG / hd;       // thread groups splitting the queries
        const int qpart = hd >= LG_WG ? 0 : threadIdx.x / hd;
        for (int d = hd >= LG_WG ? threadIdx.x : threadIdx.x % hd; d < hd; d += LG_WG) {
            for (int qi = qpart; qi < nq; qi += parts) {
                const uint32_t mask = vmask[qi];
                if (!mask) continue;
                float acc = 0.0f;
                for (int sl = 0; sl < 32; ++sl)
                    if (mask >> sl & 1) acc = lg_fmaf(es[qi * 32 + sl], lg_h2f(vt[sl * kst + d]), acc);
                const int j = qi / G, head = kvh * G + qi % G;
                const size_t pi = ((size_t)j * a.H + head) * a.tiles_max + blockIdx.x;
                a.pacc[pi * hd + d] = acc;
            }
        }
    }
}

// Merge the tile partials of one (row, head) in ascending tile order, divide, quantize to q8.
struct MergeArgs {
    const float *pm, *pl, *pacc; int tiles_max;
    int H, hd, window;
    int8_t *xq; float2 *xds;   // [M][H*hd] q8 of the attention output (input of attn_output)
    float *xf;                 // optional f32 copy [M][H*hd]
};
template <int M>
__global__ __launch_bounds__(LG_WG) void lg_k_attn_merge(MergeArgs a, const StepCtl *ctl) {
    const int head = blockIdx.x, j = blockIdx.y, hd = a.hd, qd = a.H * hd;
    const int pos = ctl->pos, pj = pos + j;
    const int first = lg_win_start(pos, a.window) >> 5;
    const int lo = (lg_win_start(pj, a.window) >> 5) - first, hi = (pj >> 5) - first;
    const size_t base = ((size_t)j * a.H + head) * a.tiles_max;
    float mx = -INFINITY;
    for (int n = lo; n <= hi; ++n) mx = fmaxf(mx, a.pm[base + n]);
    for (int d0 = 0; d0 < hd; d0 += LG_WG) {
        const int d = d0 + threadIdx.x;
        float L = 0.0f, o = 0.0f;
        for (int n = lo; n <= hi; ++n) {
            const float wn = lg_expf(a.pm[base + n] - mx);
            L = lg_fmaf(a.pl[base + n], wn, L);
            if (d < hd) o = lg_fmaf(a.pacc[(base + n) * hd + d], wn, o);
        }
        const float r = d < hd ? o / L : 0.0f;
        float dq; int sum;
        const int q = lg_quant1_32lanes(r, &dq, &sum);
        if (d < hd) {
            const size_t e = (size_t)j * qd + (size_t)head * hd + d;
            a.xq[e] = (int8_t)q;
            if ((d & 31) == 0) a.xds[e >> 5] = make_float2(dq, __int_as_float(sum));
            if (a.xf) a.xf[e] = r;
        }
    }
}
