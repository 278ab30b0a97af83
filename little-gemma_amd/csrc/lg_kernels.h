// lg_kernels.h — the kernels of one verify step (rows = M draft-block rows, M <= 8).
//
// One step is a graph of small kernels; a dependent kernel boundary costs ~1.5 us on MI355X, an
// all-CU software barrier ten times that, so the step is NOT a persistent megakernel.  Per layer:
//   rows(norm+q8) -> qkv -> qkv_post(norm,rope,KV write) -> attn tiles -> attn merge(+q8) -> o
//   -> rows -> gate/up+GeGLU(+q8) -> down -> rows -> ple gate(+q8) -> ple proj
// Every matmul reads its M activation rows already quantized (int8 + per-32 {scale,sum}) and
// stages them in LDS once per workgroup; weights stream from HBM exactly once per step in
// pre-tiled order (one 16-byte + one 2-byte load per lane per tile).  All kernels read the block
// position from device memory (StepCtl), so launch parameters never change between steps and the
// whole step is captured once into a graph.
#pragma once
#include "lg_device.h"

struct StepCtl {            // device-resident step state
    int pos;                // position of row 0 of the current block
    int step;               // index of the current block in the token schedule
    int err;
    int pad;
};

// ---------------------------------------------------------------------------------------------
// Row kernel: everything that happens to the M residual rows between two matmuls, one wavefront
// per row:  x (+= rmsnorm(dout) * w_post) (* os)  ->  x_out ;  h = rmsnorm(x) * w_pre (or x)
//           ->  q8(h) in global memory (+ optional f32 copy h_out).
// The row lives in registers as float4 per lane; lane l holds elements 256*v + 4*l .. +3, which
// is also the lane assignment of the defined sum-of-squares order.
struct RowArgs {
    const float   *x;        // [M][E] residual stream; nullptr when the rows are embeddings
    const float   *dout;     // [M][E] previous sub-layer output to be rmsnormed and added, or nullptr
    const float   *w_post;   // [E] norm weight for dout
    const float   *os;       // scalar layer_output_scale applied after the add, or nullptr
    float         *x_out;    // [M][E] updated residual, or nullptr
    const float   *w_pre;    // [E] norm weight applied before quantization, or nullptr (quantize x itself)
    float         *h_out;    // [M][E] normed rows before quantization, or nullptr
    const uint8_t *emb;      // tiled token_embd: rows are token lookups scaled by emb_scale
    const int32_t *toks;     // token schedule base ([n_steps][M])
    int8_t        *q;        // [M][E] q8 values
    float2        *ds;       // [M][E/32] {scale, sum}
    int            emb_nit, emb_seg;
    float          emb_scale;
    int            E;
    float          eps;
};

template <int M>
__global__ __launch_bounds__(64) void lg_k_rows(RowArgs s, const StepCtl *ctl) {
    const int lane = threadIdx.x, j = blockIdx.x;
    const int E = s.E, nv = E >> 8;
    float4 xv[LG_MAXV], dv[LG_MAXV], wpost[LG_MAXV], wpre[LG_MAXV];
    // issue every load up front: one memory round trip for the whole row
    if (s.emb) {
        const int tok = s.toks[ctl->step * M + j];
        #pragma unroll
        for (int v = 0; v < LG_MAXV; ++v) if (v < nv) {
            const float4 t = lg_tiled_deq4(s.emb, s.emb_nit, s.emb_seg, tok, 256 * v + 4 * lane);
            xv[v] = make_float4(t.x * s.emb_scale, t.y * s.emb_scale, t.z * s.emb_scale, t.w * s.emb_scale);
        }
    } else {
        const float4 *xr = (const float4 *)(s.x + (size_t)j * E);
        #pragma unroll
        for (int v = 0; v < LG_MAXV; ++v) if (v < nv) xv[v] = xr[64 * v + lane];
    }
    if (s.dout) {
        const float4 *dr = (const float4 *)(s.dout + (size_t)j * E), *wr = (const float4 *)s.w_post;
        #pragma unroll
        for (int v = 0; v < LG_MAXV; ++v) if (v < nv) { dv[v] = dr[64 * v + lane]; wpost[v] = wr[64 * v + lane]; }
    }
    if (s.w_pre) {
        const float4 *wr = (const float4 *)s.w_pre;
        #pragma unroll
        for (int v = 0; v < LG_MAXV; ++v) if (v < nv) wpre[v] = wr[64 * v + lane];
    }
    if (s.dout) {
        float ss = 0.0f;
        #pragma unroll
        for (int v = 0; v < LG_MAXV; ++v) if (v < nv) ss = lg_sumsq4(dv[v], ss);
        ss = lg_wave_sum64(ss);
        const float sc = 1.0f / sqrtf(ss / (float)E + s.eps);
        const bool has_os = s.os != nullptr;
        const float osv = has_os ? s.os[0] : 1.0f;
        #pragma unroll
        for (int v = 0; v < LG_MAXV; ++v) if (v < nv) {
            const float4 w = wpost[v];
            float4 r;
            r.x = xv[v].x + dv[v].x * sc * w.x;  r.y = xv[v].y + dv[v].y * sc * w.y;
            r.z = xv[v].z + dv[v].z * sc * w.z;  r.w = xv[v].w + dv[v].w * sc * w.w;
            if (has_os) { r.x = r.x * osv; r.y = r.y * osv; r.z = r.z * osv; r.w = r.w * osv; }
            xv[v] = r;
        }
    }
    if (s.x_out) {
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
        #pragma unroll
        for (int v = 0; v < LG_MAXV; ++v) if (v < nv) {
            const float4 w = wpre[v];
            xv[v] = make_float4(xv[v].x * sc * w.x, xv[v].y * sc * w.y, xv[v].z * sc * w.z, xv[v].w * sc * w.w);
        }
    }
    if (s.h_out) {
        float4 *ho = (float4 *)(s.h_out + (size_t)j * E);
        #pragma unroll
        for (int v = 0; v < LG_MAXV; ++v) if (v < nv) ho[64 * v + lane] = xv[v];
    }
    uint32_t *qrow = (uint32_t *)(s.q + (size_t)j * E);
    float2 *drow = s.ds + (size_t)j * (E >> 5);
    #pragma unroll
    for (int v = 0; v < LG_MAXV; ++v) if (v < nv) {
        float d; int sum;
        const uint32_t packed = lg_quant4_8lanes(xv[v], &d, &sum);
        qrow[64 * v + lane] = packed;
        if ((lane & 7) == 0) drow[(64 * v + lane) >> 3] = make_float2(d, __int_as_float(sum));
    }
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

// Copy M already-quantized rows (int8 + {scale,sum}) from global memory into LDS.
template <int M>
__device__ __forceinline__ void lg_load_q8(const int8_t *q, const float2 *ds, int k, int8_t *lq, float2 *lds_ds) {
    const int n16 = M * k / 16, nt = blockDim.x;
    const uint4 *src = (const uint4 *)q;
    uint4 *dst = (uint4 *)lq;
    for (int i = threadIdx.x; i < n16; i += nt) dst[i] = src[i];
    const int nd = M * (k >> 5);
    for (int i = threadIdx.x; i < nd; i += nt) lds_ds[i] = ds[i];
}

// ---------------------------------------------------------------------------------------------
// G row groups against M q8 activation rows held in LDS.  A row is cut into S contiguous K
// segments (S = 8, or 32 for rows longer than 128 blocks); lane = r*S + c owns row r of the group
// (64/S rows per group) and segment c, and walks the segment's nit blocks with a serial fma chain.
// The G groups share every activation load (gate with up, or two neighbouring groups).  On return
// every lane of a row holds that row's M results (adjacent-pair tree over the S lanes done).
template <int M, int S, int G, bool DUMP>
__device__ __forceinline__ void lg_mm_groups(const uint8_t *const (&wg)[G], int nit, const int8_t *act,
                                             const float2 *actds, int k, float (&acc)[G][M], int lane,
                                             int32_t *dots, int m, const int (&row)[G]) {
    constexpr int U = 5;                                   // tiles in flight per group
    const int c = lane & (S - 1), nb = k >> 5;
    #pragma unroll
    for (int g = 0; g < G; ++g)
        #pragma unroll
        for (int j = 0; j < M; ++j) acc[g][j] = 0.0f;
    for (int it0 = 0; it0 < nit; it0 += U) {
        uint4 wq[G][U];
        uint16_t ws[G][U];
        #pragma unroll
        for (int u = 0; u < U; ++u)
            #pragma unroll
            for (int g = 0; g < G; ++g) {
                const int it = it0 + u < nit ? it0 + u : nit - 1;             // clamp: no out-of-range load
                wq[g][u] = *(const uint4 *)(wg[g] + (size_t)it * LG_TILE + lane * 16);
                ws[g][u] = *(const uint16_t *)(wg[g] + (size_t)it * LG_TILE + 1024 + lane * 2);
            }
        #pragma unroll
        for (int u = 0; u < U; ++u) {
            if (it0 + u >= nit) break;
            const int b = c * nit + it0 + u;
            #pragma unroll
            for (int j = 0; j < M; ++j) {
                const float2 ds = actds[j * nb + b];
                const int4 a0 = *(const int4 *)(act + (size_t)j * k + b * 32), a1 = *(const int4 *)(act + (size_t)j * k + b * 32 + 16);
                #pragma unroll
                for (int g = 0; g < G; ++g) {
                    const int dot = lg_block_dot(wq[g][u], a0, a1, __float_as_int(ds.y));
                    if (DUMP) dots[((size_t)j * m + row[g]) * nb + b] = dot;
                    acc[g][j] = lg_fmaf(ds.x * lg_h2f(ws[g][u]), (float)dot, acc[g][j]);
                }
            }
        }
    }
    #pragma unroll
    for (int g = 0; g < G; ++g)
        #pragma unroll
        for (int j = 0; j < M; ++j) {
            float v = acc[g][j];
            #pragma unroll
            for (int o = 1; o < S; o <<= 1) v = v + __shfl_xor(v, o);
            acc[g][j] = v;
        }
}

template <int M>
__device__ __forceinline__ float lg_pick(const float (&acc)[M], int j) {
    float v = acc[0];
    #pragma unroll
    for (int t = 1; t < M; ++t) v = j == t ? acc[t] : v;
    return v;
}

struct MmArgs {
    const uint8_t *w;        // tiled weights
    int            k, m;     // row length, rows
    float         *out;      // [M][m]
    const int8_t  *q_in;     // [M][k] q8 input rows
    const float2  *ds_in;    // [M][k/32]
    int32_t       *dots;     // DUMP only: [M][m][k/32]
};

// Plain matmul: out[j][i] f32.  blockDim = 64*W wavefronts, each wavefront takes G neighbouring
// row groups (G*64/S rows) per pass; grid covers ceil(m / (W*G*64/S)) passes.
template <int M, int S, int G, bool DUMP>
__global__ __launch_bounds__(LG_WG) void lg_k_mm(MmArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    int8_t *lq = (int8_t *)smem;
    float2 *lds = (float2 *)(smem + (size_t)M * a.k);
    lg_load_q8<M>(a.q_in, a.ds_in, a.k, lq, lds);
    __syncthreads();
    constexpr int RW = 64 / S;                                // rows per group
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const int nit = (a.k >> 5) / S, ngroups = a.m / RW;
    const int g0 = (blockIdx.x * nw + wave) * G;
    if (g0 >= ngroups) return;
    const uint8_t *wg[G];
    int row[G];
    #pragma unroll
    for (int g = 0; g < G; ++g) {
        const int gi = g0 + g < ngroups ? g0 + g : ngroups - 1;   // ragged tail: recompute the last group
        wg[g] = a.w + (size_t)gi * nit * LG_TILE;
        row[g] = gi * RW + lane / S;
    }
    float acc[G][M];
    lg_mm_groups<M, S, G, DUMP>(wg, nit, lq, lds, a.k, acc, lane, a.dots, a.m, row);
    const int c = lane & (S - 1);
    if (c < M) {
        #pragma unroll
        for (int g = 0; g < G; ++g) a.out[(size_t)c * a.m + row[g]] = lg_pick<M>(acc[g], c);
    }
}

// Gate/up matmul with the GeGLU and the q8 quantization of its result as epilogue.  The tiled
// matrix interleaves 32 gate rows with the 32 up rows of the same indices, so a workgroup of 4
// wavefronts owns one 32-wide quantization group: wavefront w computes gate and up rows 8w..8w+7
// of it, sharing each activation load between the two.
struct GegluArgs {
    const uint8_t *w;        // tiled [2*n_ff][k], virtual row order: 32 gate, 32 up, 32 gate, ...
    int            k, n_ff;
    const int8_t  *q_in; const float2 *ds_in;
    int8_t        *gq;       // [M][n_ff]
    float2        *gds;      // [M][n_ff/32]
};
template <int M>
__global__ __launch_bounds__(LG_WG) void lg_k_mm_geglu(GegluArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    int8_t *lq = (int8_t *)smem;
    float2 *lds = (float2 *)(smem + (size_t)M * a.k);
    __shared__ float gbuf[LG_HIP_MAX_ROWS_DEV][32];
    lg_load_q8<M>(a.q_in, a.ds_in, a.k, lq, lds);
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nit = a.k >> 8;
    const int t = blockIdx.x;                               // 32-wide slice of n_ff
    const size_t gstride = (size_t)nit * LG_TILE;
    const uint8_t *wg[2] = { a.w + ((size_t)t * 8 + wave) * gstride, a.w + ((size_t)t * 8 + 4 + wave) * gstride };
    const int row[2] = { 0, 0 };
    float acc[2][M];
    lg_mm_groups<M, 8, 2, false>(wg, nit, lq, lds, a.k, acc, lane, nullptr, 0, row);
    const int c = lane & 7, r = lane >> 3;
    if (c < M) gbuf[c][wave * 8 + r] = lg_gelu(lg_pick<M>(acc[0], c)) * lg_pick<M>(acc[1], c);
    __syncthreads();
    for (int j = threadIdx.x >> 5; j < M; j += LG_WG / 32) {       // half-wavefront per row, one value per lane
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
    const int8_t  *q_in; const float2 *ds_in;
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
__global__ __launch_bounds__(LG_WG) void lg_k_mm_plegate(PleGateArgs a, const StepCtl *ctl) {
    extern __shared__ __align__(16) unsigned char smem[];
    int8_t *lq = (int8_t *)smem;
    float2 *lds = (float2 *)(smem + (size_t)M * a.k);
    float *ipl = (float *)(lds + (size_t)M * (a.k >> 5));        // [M][32]: this workgroup's slice
    __shared__ float gbuf[LG_HIP_MAX_ROWS_DEV][32];
    lg_load_q8<M>(a.q_in, a.ds_in, a.k, lq, lds);
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
        if (lane < 32) {
            const int e = blockIdx.x * 32 + lane;
            const int tok = a.toks[ctl->step * M + j];
            const uint8_t *trow = a.pte + (size_t)tok * ((size_t)a.n_layer * ple / 32 * 18);
            const float p = pr[e] * a.pscale * sc * a.proj_norm[e];
            const float tk = lg_q4_0_elem(trow, a.layer * ple + e) * a.tscale;
            ipl[j * 32 + lane] = (p + tk) * a.rsqrt2;
        }
    }
    __syncthreads();
    const uint8_t *wg[1] = { a.w + (size_t)(blockIdx.x * 4 + wave) * nit * LG_TILE };
    const int row[1] = { 0 };
    float acc[1][M];
    lg_mm_groups<M, 8, 1, false>(wg, nit, lq, lds, a.k, acc, lane, nullptr, 0, row);
    const int c = lane & 7, r = lane >> 3;
    if (c < M) gbuf[c][wave * 8 + r] = lg_gelu(lg_pick<M>(acc[0], c)) * ipl[c * 32 + wave * 8 + r];
    __syncthreads();
    for (int j = threadIdx.x >> 5; j < M; j += LG_WG / 32) {
        const int i = threadIdx.x & 31;
        float d; int sum;
        const int q = lg_quant1_32lanes(gbuf[j][i], &d, &sum);
        a.pq[(size_t)j * ple + blockIdx.x * 32 + i] = (int8_t)q;
        if (i == 0) a.pds[(size_t)j * (ple >> 5) + blockIdx.x] = make_float2(d, __int_as_float(sum));
    }
}

// lm_head: each workgroup walks `passes` blocks of 64 vocabulary rows (4 wavefronts x 2 groups
// sharing activation loads), applies the soft cap and keeps a running argmax per draft row
// (first maximum: lower index wins ties, src/cuda/model-cuda.cuh:703-720); one partial per
// workgroup and row goes to global memory.
struct HeadArgs {
    const uint8_t *w; int k, n_vocab, passes;
    const int8_t *q_in; const float2 *ds_in;
    float softcap;
    float *logits;          // [M][n_vocab] or nullptr
    float *pval; int *pidx; // [gridDim.x][M]
};
template <int M>
__global__ __launch_bounds__(LG_WG) void lg_k_mm_head(HeadArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    int8_t *lq = (int8_t *)smem;
    float2 *lds = (float2 *)(smem + (size_t)M * a.k);
    __shared__ float sv[4][LG_HIP_MAX_ROWS_DEV];
    __shared__ int si[4][LG_HIP_MAX_ROWS_DEV];
    lg_load_q8<M>(a.q_in, a.ds_in, a.k, lq, lds);
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nit = a.k >> 8;
    const int c = lane & 7, r = lane >> 3, ngroups = a.n_vocab >> 3;
    float best = -INFINITY;                                  // lane c < M tracks draft row c
    int besti = 0x7fffffff;
    for (int p = 0; p < a.passes; ++p) {
        const int g0 = ((blockIdx.x * a.passes + p) * 4 + wave) * 2;
        if (g0 >= ngroups) break;
        const uint8_t *wg[2] = { a.w + (size_t)g0 * nit * LG_TILE, a.w + (size_t)(g0 + 1) * nit * LG_TILE };
        const int row[2] = { g0 * 8 + r, g0 * 8 + 8 + r };
        float acc[2][M];
        lg_mm_groups<M, 8, 2, false>(wg, nit, lq, lds, a.k, acc, lane, nullptr, 0, row);
        if (c < M) {
            #pragma unroll
            for (int g = 0; g < 2; ++g) {
                float v = lg_pick<M>(acc[g], c);
                if (a.softcap > 0.0f) v = a.softcap * lg_tanhf(v / a.softcap);
                if (a.logits) a.logits[(size_t)c * a.n_vocab + row[g]] = v;
                if (v > best || (v == best && row[g] < besti)) { best = v; besti = row[g]; }
            }
        }
    }
    // lanes with the same c (one per row r of the group) hold candidates for draft row c
    #pragma unroll
    for (int o = 8; o < 64; o <<= 1) {
        const float ov = __shfl_xor(best, o);
        const int oi = __shfl_xor(besti, o);
        if (ov > best || (ov == best && oi < besti)) { best = ov; besti = oi; }
    }
    if (lane < M) { sv[wave][lane] = best; si[wave][lane] = besti; }
    __syncthreads();
    if (threadIdx.x < M) {
        float v = sv[0][threadIdx.x]; int idx = si[0][threadIdx.x];
        for (int w = 1; w < 4; ++w) {
            const float ov = sv[w][threadIdx.x]; const int oi = si[w][threadIdx.x];
            if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
        }
        a.pval[(size_t)blockIdx.x * M + threadIdx.x] = v;
        a.pidx[(size_t)blockIdx.x * M + threadIdx.x] = idx;
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
    __shared__ float sv[LG_HIP_MAX_ROWS_DEV][LG_WG / 64];
    __shared__ int si[LG_HIP_MAX_ROWS_DEV][LG_WG / 64];
    __shared__ int s_adv;
    const int step = ctl->step, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float v[M]; int idx[M];
    #pragma unroll
    for (int j = 0; j < M; ++j) { v[j] = -INFINITY; idx[j] = 0x7fffffff; }
    for (int p = threadIdx.x; p < a.n_part; p += LG_WG) {
        #pragma unroll
        for (int j = 0; j < M; ++j) {
            const float pv = a.pval[(size_t)p * M + j]; const int pi = a.pidx[(size_t)p * M + j];
            if (pv > v[j] || (pv == v[j] && pi < idx[j])) { v[j] = pv; idx[j] = pi; }
        }
    }
    #pragma unroll
    for (int j = 0; j < M; ++j) {
        for (int o = 1; o < 64; o <<= 1) {
            const float ov = __shfl_xor(v[j], o); const int oi = __shfl_xor(idx[j], o);
            if (ov > v[j] || (ov == v[j] && oi < idx[j])) { v[j] = ov; idx[j] = oi; }
        }
        if (lane == 0) { sv[j][wave] = v[j]; si[j][wave] = idx[j]; }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int best[M];
        for (int j = 0; j < M; ++j) {
            float bv = sv[j][0]; int bi = si[j][0];
            for (int w = 1; w < LG_WG / 64; ++w)
                if (sv[j][w] > bv || (sv[j][w] == bv && si[j][w] < bi)) { bv = sv[j][w]; bi = si[j][w]; }
            best[j] = bi;
        }
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
// After the q/k/v projection: per-head rmsnorm (q and k weighted, v plain), rotary on q and k,
// f16 round and store of the block's K/V rows into the ring (src/cuda/prefill-kernel.cuh:403-421).
// One wavefront per (head vector, draft row).
struct QkvPostArgs {
    const float *qkv;        // [M][ld] raw projections: q at 0, k at k_off, v at v_off
    int ld, k_off, v_off;
    int H, nkv, hd;
    const float *q_norm, *k_norm;       // [hd]
    const float *rope_tab, *rope_ff;    // [hd/2]; ff may be nullptr
    float *q_rot;            // [M][H*hd] normed + rotated queries
    uint16_t *kc, *vc;       // this layer's cache (nullptr when it shares another layer's)
    int seq, kv_dim;
    float eps;
};
__global__ __launch_bounds__(64) void lg_k_qkv_post(QkvPostArgs a, const StepCtl *ctl) {
    __shared__ float vec[512];
    const int lane = threadIdx.x, job = blockIdx.x, j = blockIdx.y, hd = a.hd, half = hd >> 1;
    const int pos = ctl->pos + j;
    const bool isq = job < a.H, isv = job >= a.H + a.nkv;
    const int head = isq ? job : (job - a.H) % a.nkv;
    const float *src = a.qkv + (size_t)j * a.ld + (isq ? (size_t)head * hd : (size_t)(isv ? a.v_off : a.k_off) + (size_t)head * hd);
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
        vec[e0] = r.x; vec[e0 + 1] = r.y; vec[e0 + 2] = r.z; vec[e0 + 3] = r.w;
    }
    __syncthreads();
    if (!isv) {
        for (int p = lane; p < half; p += 64) {
            const float ang = (float)pos * a.rope_tab[p] / (a.rope_ff ? a.rope_ff[p] : 1.0f);
            float sn, cs;
            lg_sincosf(ang, &sn, &cs);
            const float x0 = vec[p], x1 = vec[p + half];
            vec[p] = x0 * cs - x1 * sn;
            vec[p + half] = x0 * sn + x1 * cs;
        }
        __syncthreads();
    }
    if (isq) {
        float *dst = a.q_rot + (size_t)j * a.H * hd + (size_t)head * hd;
        for (int e = lane; e < hd; e += 64) dst[e] = vec[e];
    } else {
        uint16_t *dst = (isv ? a.vc : a.kc) + (size_t)(pos % a.seq) * a.kv_dim + (size_t)head * hd;
        for (int e = lane; e < hd; e += 64) dst[e] = lg_f2h(vec[e]);
    }
}

// ---------------------------------------------------------------------------------------------
// Attention.  Keys are processed in tiles of 32 aligned to absolute positions (tile n covers
// positions 32n..32n+31).  One workgroup per (kv head, tile): it stages the tile's K and V rows in
// LDS once for the gqa*M (head,row) queries that share the kv head, and writes for each query the
// tile's partial softmax (max, sum, V-accumulator).
// Defined order: score = (a0+a1)+(a2+a3), a_c = fma chain over dims i%4==c; m = max over valid
// keys; e = exp(s-m); l = adjacent tree over the 32 key slots; acc[d] = fma chain over valid
// slots ascending.
struct AttnArgs {
    const float *q;          // [M][H*hd] normed + rotated queries
    int H, nkv, hd;
    const uint16_t *kc, *vc; // cache of the layer this one reads
    int seq, kv_dim, window; // ring rows, row width, 0 = global
    float *pm, *pl, *pacc;   // partials: [M*H][tiles_max], [M*H][tiles_max][hd]
    int tiles_max;
};

__device__ __forceinline__ int lg_win_start(int pos, int window) {
    return (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
}

template <int M>
__global__ __launch_bounds__(LG_WG) void lg_k_attn(AttnArgs a, const StepCtl *ctl) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int hd = a.hd, G = a.H / a.nkv, nq = G * M;
    const int kst = hd + 8;                                   // padded K/V tile row (halves)
    float *qs = (float *)smem;                                // [nq][hd]
    uint16_t *kt = (uint16_t *)(qs + (size_t)nq * hd);        // [32][kst]
    uint16_t *vt = kt + 32 * kst;                             // [32][kst]
    float *es = (float *)(vt + 32 * kst);                     // [nq][32]
    uint32_t *vmask = (uint32_t *)(es + nq * 32);             // [nq]
    const int pos = ctl->pos, kvh = blockIdx.y;
    const int start0 = lg_win_start(pos, a.window), last_needed = pos + M - 1;
    const int n = (start0 >> 5) + blockIdx.x;
    if (n > (last_needed >> 5)) return;
    const int t0 = n << 5;
    // queries of this kv head's group, K/V tile rows
    for (int idx = threadIdx.x; idx < nq * (hd >> 2); idx += LG_WG) {
        const int qi = idx / (hd >> 2), e0 = (idx - qi * (hd >> 2)) << 2;
        const int j = qi / G, head = kvh * G + qi % G;
        *(float4 *)(qs + (size_t)qi * hd + e0) = *(const float4 *)(a.q + (size_t)j * a.H * hd + (size_t)head * hd + e0);
    }
    for (int idx = threadIdx.x; idx < 32 * (hd >> 3); idx += LG_WG) {
        const int sl = idx / (hd >> 3), e0 = (idx - sl * (hd >> 3)) << 3;
        const int t = t0 + sl;
        uint4 kk = make_uint4(0, 0, 0, 0), vv = make_uint4(0, 0, 0, 0);
        if (t >= start0 && t <= last_needed) {
            const size_t off = (size_t)(t % a.seq) * a.kv_dim + (size_t)kvh * hd + e0;
            kk = *(const uint4 *)(a.kc + off);
            vv = *(const uint4 *)(a.vc + off);
        }
        *(uint4 *)(kt + sl * kst + e0) = kk;
        *(uint4 *)(vt + sl * kst + e0) = vv;
    }
    __syncthreads();
    // scores, tile max, exp, tile sum.  Thread = (key slot, query group of 8).
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
                for (int i = 0; i < hd; i += 8) {
                    const float4 q4 = *(const float4 *)(qv + i), q5 = *(const float4 *)(qv + i + 4);
                    const uint4 k4 = *(const uint4 *)(kr + i);
                    a0 = lg_fmaf(q4.x, lg_h2f((uint16_t)(k4.x & 0xFFFF)), a0);
                    a1 = lg_fmaf(q4.y, lg_h2f((uint16_t)(k4.x >> 16)), a1);
                    a2 = lg_fmaf(q4.z, lg_h2f((uint16_t)(k4.y & 0xFFFF)), a2);
                    a3 = lg_fmaf(q4.w, lg_h2f((uint16_t)(k4.y >> 16)), a3);
                    a0 = lg_fmaf(q5.x, lg_h2f((uint16_t)(k4.z & 0xFFFF)), a0);
                    a1 = lg_fmaf(q5.y, lg_h2f((uint16_t)(k4.z >> 16)), a1);
                    a2 = lg_fmaf(q5.z, lg_h2f((uint16_t)(k4.w & 0xFFFF)), a2);
                    a3 = lg_fmaf(q5.w, lg_h2f((uint16_t)(k4.w >> 16)), a3);
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
    // acc[d] = sum over valid slots of e * V[slot][d]
    {
        const int parts = hd >= LG_WG ? 1 : LG_WG / hd;       // thread groups splitting the queries
        const int qpart = hd >= LG_WG ? 0 : threadIdx.x / hd;
        for (int d = hd >= LG_WG ? threadIdx.x : threadIdx.x % hd; d < hd; d += LG_WG) {
            for (int qi = qpart; qi < nq; qi += parts) {
                const uint32_t mask = vmask[qi];
                if (!mask) continue;
                float acc = 0.0f;
                #pragma unroll 8
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
    __shared__ float wts[512];                                // exp(m_tile - M) of up to 512 tiles at a time
    const int head = blockIdx.x, j = blockIdx.y, hd = a.hd, qd = a.H * hd;
    const int pos = ctl->pos, pj = pos + j;
    const int first = lg_win_start(pos, a.window) >> 5;
    const int lo = (lg_win_start(pj, a.window) >> 5) - first, hi = (pj >> 5) - first;
    const size_t base = ((size_t)j * a.H + head) * a.tiles_max;
    float mx = -INFINITY;
    for (int n = lo + (int)threadIdx.x; n <= hi; n += LG_WG) mx = fmaxf(mx, a.pm[base + n]);
    mx = lg_max_n(mx, 64);
    __shared__ float wmx[LG_WG / 64];
    if ((threadIdx.x & 63) == 0) wmx[threadIdx.x >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(wmx[0], wmx[1]), fmaxf(wmx[2], wmx[3]));
    float L = 0.0f, o[2] = { 0.0f, 0.0f };
    for (int c0 = lo; c0 <= hi; c0 += 512) {
        const int cn = hi - c0 + 1 < 512 ? hi - c0 + 1 : 512;
        __syncthreads();
        for (int n = threadIdx.x; n < cn; n += LG_WG) wts[n] = lg_expf(a.pm[base + c0 + n] - mx);
        __syncthreads();
        for (int n0 = 0; n0 < cn; n0 += 8) {                   // 8 independent loads in flight, fma in tile order
            float pl8[8], pa8[2][8];
            #pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int n = n0 + u < cn ? n0 + u : cn - 1;
                pl8[u] = a.pl[base + c0 + n];
                #pragma unroll
                for (int h2 = 0; h2 < 2; ++h2) {
                    const int d = h2 * LG_WG + threadIdx.x;
                    pa8[h2][u] = d < hd ? a.pacc[(base + c0 + n) * hd + d] : 0.0f;
                }
            }
            #pragma unroll
            for (int u = 0; u < 8; ++u) {
                if (n0 + u >= cn) break;
                const float wn = wts[n0 + u];
                L = lg_fmaf(pl8[u], wn, L);
                o[0] = lg_fmaf(pa8[0][u], wn, o[0]);
                o[1] = lg_fmaf(pa8[1][u], wn, o[1]);
            }
        }
    }
    #pragma unroll
    for (int h2 = 0; h2 < 2; ++h2) {
        const int d = h2 * LG_WG + threadIdx.x;
        if (h2 * LG_WG >= hd) break;
        const float r = d < hd ? o[h2] / L : 0.0f;
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
