// lg_fused.h — verify-step kernels that do the row work of a layer themselves.
//
// Between two matmuls of a layer the residual rows are updated, normed and quantized (lg_k_rows).  As a kernel
// of its own that is M workgroups on a 256-CU chip and a launch boundary either side.  Here every workgroup of
// the consuming matmul repeats the row work of all M rows (same lane assignment, same summation order: the
// results are the bits lg_k_rows produces) straight into its LDS operand buffer, and one workgroup also writes
// the new residual.  The repetition costs each workgroup one round trip for 2 x M rows plus the two norm
// weights, and M x E/4 quantizations of four values (about 50 instructions each): for one or two rows that is
// less than the launch it replaces (one-row decode: 2.8 us per layer saved), for four and more rows it is more
// (a 5-row block: +0.3 ms per step, also in the gate/up kernel), so wider blocks keep lg_k_rows.
#pragma once
#include "lg_kernels.h"

struct RowWork {
    const float *x;          // [M][E] residual
    const float *dout;       // [M][E] previous sub-layer output: x += rmsnorm(dout) * w_post; nullptr: x stays as it is
    const float *w_post;     // [E]
    const float *os;         // scalar applied after the add, or nullptr
    float       *x_out;      // [M][E] new residual (written by one workgroup)
    const float *w_pre;      // [E] norm weight applied before quantization
    int          E;
    float        eps;
};

// The rows of a block on NE engines of 256 lanes: engine e (threads 256e..256e+255) takes rows e, e+NE, ...
// NV = float4 per lane and row (ceil(E/1024)).  Rows are taken BJ per engine at a time; every load of such a
// batch goes out before its first use, so a batch costs one round trip (BJ bounds the registers: 2*BJ*NV float4).
// red: [2][LG_HIP_MAX_ROWS_DEV][4] floats of LDS.  sink(j, quad, packed, d, sum) receives the q8 of row j,
// four values at a time (quad = index of the float4 in the row), in all lanes of a group of 8.
// All threads of the workgroup must call it (two barriers per batch inside).
template <int M, int NV, int NE, int BJ, typename Sink>
__device__ __forceinline__ void lg_rows_fused(const RowWork &s, bool write_x, float *red, Sink sink) {
    constexpr int JB = (M + NE - 1) / NE;
    const int t = threadIdx.x & 255, e = NE > 1 ? (int)(threadIdx.x >> 8) : 0, wave = t >> 6;
    const int E = s.E, nq = E >> 2;
    const bool has_d = s.dout != nullptr;                     // false: the rows are only normed and quantized
    float4 wpost[NV], wpre[NV];
    const float4 *wr = (const float4 *)s.w_post, *wp = (const float4 *)s.w_pre;
    const bool has_os = has_d && s.os != nullptr;
    float *red0 = red, *red1 = red + LG_HIP_MAX_ROWS_DEV * 4;
    #pragma unroll
    for (int b0 = 0; b0 < JB; b0 += BJ) {
        float4 xv[BJ][NV], dv[BJ][NV];
        #pragma unroll
        for (int jb = 0; jb < BJ; ++jb) {
            const int j = e + (b0 + jb) * NE;
            if (b0 + jb >= JB || j >= M) continue;
            const float4 *xr = (const float4 *)(s.x + (size_t)j * E), *dr = (const float4 *)(s.dout + (size_t)j * E);
            #pragma unroll
            for (int v = 0; v < NV; ++v) if (t + 256 * v < nq) {
                xv[jb][v] = xr[t + 256 * v];
                dv[jb][v] = has_d ? dr[t + 256 * v] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            }
        }
        if (b0 == 0) {
            #pragma unroll
            for (int v = 0; v < NV; ++v) if (t + 256 * v < nq) {
                wpost[v] = has_d ? wr[t + 256 * v] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                wpre[v] = wp[t + 256 * v];
            }
        }
        const float osv = has_os ? s.os[0] : 1.0f;
        #pragma unroll
        for (int jb = 0; jb < BJ; ++jb) {
            const int j = e + (b0 + jb) * NE;
            if (b0 + jb >= JB || j >= M || !has_d) continue;
            float ss = 0.0f;
            #pragma unroll
            for (int v = 0; v < NV; ++v) if (t + 256 * v < nq) ss = lg_sumsq4(dv[jb][v], ss);
            ss = lg_wave_sum64(ss);
            if ((t & 63) == 0) red0[j * 4 + wave] = ss;
        }
        if (has_d) __syncthreads();
        #pragma unroll
        for (int jb = 0; jb < BJ; ++jb) {
            const int j = e + (b0 + jb) * NE;
            if (b0 + jb >= JB || j >= M) continue;
            float sc = 0.0f;
            if (has_d) {
                const float ssd = (red0[j * 4] + red0[j * 4 + 1]) + (red0[j * 4 + 2] + red0[j * 4 + 3]);
                sc = 1.0f / sqrtf(ssd / (float)E + s.eps);
            }
            float ss = 0.0f;
            #pragma unroll
            for (int v = 0; v < NV; ++v) if (t + 256 * v < nq) {
                float4 r = xv[jb][v];
                if (has_d) {
                    const float4 w = wpost[v], d = dv[jb][v];
                    r.x = r.x + d.x * sc * w.x;  r.y = r.y + d.y * sc * w.y;
                    r.z = r.z + d.z * sc * w.z;  r.w = r.w + d.w * sc * w.w;
                    if (has_os) { r.x = r.x * osv; r.y = r.y * osv; r.z = r.z * osv; r.w = r.w * osv; }
                    xv[jb][v] = r;
                    if (write_x) ((float4 *)(s.x_out + (size_t)j * E))[t + 256 * v] = r;
                }
                ss = lg_sumsq4(r, ss);
            }
            ss = lg_wave_sum64(ss);
            if ((t & 63) == 0) red1[j * 4 + wave] = ss;
        }
        __syncthreads();
        #pragma unroll
        for (int jb = 0; jb < BJ; ++jb) {
            const int j = e + (b0 + jb) * NE;
            if (b0 + jb >= JB || j >= M) continue;
            const float ssx = (red1[j * 4] + red1[j * 4 + 1]) + (red1[j * 4 + 2] + red1[j * 4 + 3]);
            const float sc = 1.0f / sqrtf(ssx / (float)E + s.eps);
            #pragma unroll
            for (int v = 0; v < NV; ++v) {
                if (t + 256 * v >= nq) break;                // nq is a multiple of 64: whole wavefronts
                const float4 w = wpre[v], x = xv[jb][v];
                const float4 h = make_float4(x.x * sc * w.x, x.y * sc * w.y, x.z * sc * w.z, x.w * sc * w.w);
                float d; int sum;
                const uint32_t packed = lg_quant4_8lanes(h, &d, &sum);
                sink(j, t + 256 * v, packed, d, sum);
            }
        }
    }
}
// rows per engine and batch that keep 2*BJ*NV float4 within `budget` float4 registers
__host__ __device__ constexpr int lg_rows_batch(int jb, int nv, int budget) {
    return (budget / (2 * nv) < 1) ? 1 : (budget / (2 * nv) < jb ? budget / (2 * nv) : jb);
}

// Row work + plain matmul (k = E, 8 K segments): the q/k/v projection after the attention norm.
// 256 threads: all four wavefronts do the row work, the first NW of them then take one row group each.
struct RowsMmArgs {
    MmArgs  mm;
    RowWork rows;
};
#define LG_ROWSMM_FIELDS(X, v) X(const float *, rx, rows.x, v) X(const float *, rdout, rows.dout, v) X(const float *, rw_post, rows.w_post, v) X(const float *, rw_pre, rows.w_pre, v) X(const uint8_t *, mw, mm.w, v) X(int, rE, rows.E, v) X(int, mk, mm.k, v) X(int, mm_, mm.m, v) X(const float *, ros, rows.os, v) X(float *, rx_out, rows.x_out, v) X(float, reps, rows.eps, v) X(float *, mout, mm.out, v) X(const int8_t *, mq_in, mm.q_in, v) X(int32_t *, mdots, mm.dots, v)
template <int M, int NV, int NW>
__global__ __launch_bounds__(LG_WG) void lg_k_rows_mm(LG_ROWSMM_FIELDS(LG_XP, _) int p_end_) {
    RowsMmArgs a; LG_ROWSMM_FIELDS(LG_XI, a)
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float red[2 * LG_HIP_MAX_ROWS_DEV * 4];
    const int k = a.mm.k;
    int8_t *lq = (int8_t *)smem;
    float2 *lds = (float2 *)(smem + (size_t)M * k);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nit = (k >> 5) / 8, ngroups = a.mm.m / 8, nb = k >> 5;
    const int g0 = blockIdx.x * NW + (wave < NW ? wave : 0);
    const int gi = g0 < ngroups ? g0 : ngroups - 1;
    const uint8_t *wg[1] = { a.mm.w + (size_t)gi * nit * LG_TILE };
    const int row[1] = { gi * 8 + lane / 8 };
    WChunk<1> first;
    if (wave < NW) lg_mm_fetch<1>(first, wg, 0, nit, lane);
    const ActLayout lay = lg_act_layout(k);
    lg_rows_fused<M, NV, 1, lg_rows_batch(M, NV, 40)>(a.rows, blockIdx.x == 0, red, [&](int j, int quad, uint32_t packed, float d, int sum) {
        *(uint32_t *)(lq + (size_t)j * k + (size_t)lg_act_unit(lay, quad >> 2) * 16 + (quad & 3) * 4) = packed;
        if ((threadIdx.x & 7) == 0) lds[j * nb + lg_act_block(lay, quad >> 3)] = make_float2(d, __int_as_float(sum));
    });
    __syncthreads();
    if (wave >= NW || g0 >= ngroups) return;
    float acc[1][M];
    lg_mm_groups<M, 8, 1, false>(wg, first, nit, lq, lds, k, acc, lane, nullptr, a.mm.m, row);
    const int c = lane & 7;
    if (c < M) a.mm.out[(size_t)c * a.mm.m + row[0]] = lg_pick<M>(acc[0], c);
}

// ---------------------------------------------------------------------------------------------
// Plain 8-segment matmul for blocks of several rows, the K range of every row group cut over KP wavefronts.
// With four or more rows the dot phase of lg_k_mm is bound by the instruction issue of its one wavefront per row
// group (about 125 instructions per tile at five rows, ten tiles at k = 2560) while half of the chip's SIMDs have
// nothing to do.  Here wavefront (group, part) takes the tiles [part*nit/KP, (part+1)*nit/KP) of its group: it
// requests all of them at once, forms the exact block dots and the scale products of its tiles, and the float
// chain p = fma(xd*dw, (float)dot, p) then runs through the parts in order (part p starts from the value part
// p-1 left in LDS), so every sum is formed in the order of lg_mm_groups and the result is the same bits.
template <int M, int KP>
__global__ __launch_bounds__(128 * KP) void lg_k_mm_ks(LG_MM_FIELDS(LG_XP, _) int p_end_) {
    MmArgs a; LG_MM_FIELDS(LG_XI, a)
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int TMAX = (16 + KP - 1) / KP;                  // k <= 4096: at most 16 tiles per group
    const int k = a.k, nb = k >> 5, nit = nb >> 3, ngroups = a.m >> 3;
    int8_t *lq = (int8_t *)smem;
    const float2 *lds = (const float2 *)(smem + (size_t)M * k);
    float *xch = (float *)(smem + (((size_t)M * k + (size_t)M * nb * 8 + 15) & ~(size_t)15));   // [2 groups][M][64 lanes]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, gsel = wave / KP, part = wave - gsel * KP;
    const int g0 = blockIdx.x * 2 + gsel, gi = g0 < ngroups ? g0 : ngroups - 1;
    const int it_lo = part * nit / KP, nt = (part + 1) * nit / KP - it_lo;
    const uint8_t *wg = a.w + (size_t)gi * nit * LG_TILE;
    const CopyBatch rows = lg_load_q8_issue<M>(a.q_in, k, 128 * KP);   // the rows first, then the tiles
    uint4 wq[TMAX]; uint32_t ws[TMAX];
    #pragma unroll
    for (int u = 0; u < TMAX; ++u) {
        const int it = it_lo + u < nit ? it_lo + u : nit - 1;
        wq[u] = lg_ldt16(wg, it, lane);
        ws[u] = lg_ldt2(wg, it, lane);
    }
    __builtin_amdgcn_sched_barrier(0);
    lg_load_q8_commit<M>(rows, a.q_in, k, lq, 128 * KP);
    __syncthreads();
    const int c = lane & 7;
    float sc[TMAX][M], fd[TMAX][M];
    #pragma unroll
    for (int u = 0; u < TMAX; ++u) {
        if (u >= nt) continue;                                // (a guard, not a break: the arrays stay in registers)
        const int it = it_lo + u;
        float2 ds[M]; int4 a0[M], a1[M];
        #pragma unroll
        for (int j = 0; j < M; ++j) {
            ds[j] = lds[j * nb + it * 8 + c];
            const int8_t *au = lq + (size_t)j * k + (size_t)(it * 16 + c) * 16;
            a0[j] = *(const int4 *)au; a1[j] = *(const int4 *)(au + 8 * 16);
        }
        __builtin_amdgcn_sched_barrier(0);
        const float dw = lg_h2f((uint16_t)ws[u]);
        #pragma unroll
        for (int j = 0; j < M; ++j) {
            fd[u][j] = (float)lg_block_dot(wq[u], a0[j], a1[j], __float_as_int(ds[j].y));
            sc[u][j] = ds[j].x * dw;
        }
    }
    float acc[M];
    #pragma unroll
    for (int j = 0; j < M; ++j) acc[j] = 0.0f;
    float *mine = xch + (size_t)gsel * M * 64 + lane;
    #pragma unroll
    for (int p = 0; p < KP; ++p) {
        if (part == p) {
            if (p > 0) {
                #pragma unroll
                for (int j = 0; j < M; ++j) acc[j] = mine[j * 64];
            }
            #pragma unroll
            for (int u = 0; u < TMAX; ++u) {
                if (u >= nt) continue;
                #pragma unroll
                for (int j = 0; j < M; ++j) acc[j] = lg_fmaf(sc[u][j], fd[u][j], acc[j]);
            }
            if (p < KP - 1) {
                #pragma unroll
                for (int j = 0; j < M; ++j) mine[j * 64] = acc[j];
            }
        }
        if (p < KP - 1) __syncthreads();
    }
    if (part != KP - 1 || g0 >= ngroups) return;
    #pragma unroll
    for (int j = 0; j < M; ++j) acc[j] = lg_sum_seg<8>(acc[j]);
    if (c < M) a.out[(size_t)c * a.m + gi * 8 + (lane >> 3)] = lg_pick<M>(acc, c);
}

// ---------------------------------------------------------------------------------------------
// Matmul against a weight matrix kept in f32 (the per-layer-embedding matrices of QAT conversions, which the
// reference's int8 backend also multiplies unquantized: src/cuda/model-cuda-i8.cu:645-653, :846-895; f16 and bf16
// files are widened to f32 at upload, which is exact).  Activations are the f32 rows themselves.  One wavefront per
// weight row and MC block rows (blockIdx.y: which MC rows of a wider block); order: lane (e/4)%64 takes element e,
// fma in ascending e, adjacent-pair tree over the 64 lanes.  Optional epilogue of the per-layer gate:
// out = gelu(sum) * ipl[row][i].
struct MmfArgs {
    const float *w; int k, m;                                 // [m][k], k a multiple of 256
    const float *x; int ldx, rows;                            // [rows][ldx]
    float *out; int ldo;                                      // [rows][ldo]
    const float *ipl; int ipl_ld;                             // nullptr, or [rows][ipl_ld] (already at the layer's slice)
};
template <int MC>
__global__ __launch_bounds__(LG_WG) void lg_k_mmf(MmfArgs a) {
    const int lane = threadIdx.x & 63, i = blockIdx.x * (LG_WG / 64) + (threadIdx.x >> 6), j0 = blockIdx.y * MC;
    if (i >= a.m) return;
    const float4 *wr = (const float4 *)(a.w + (size_t)i * a.k);
    float acc[MC];
    #pragma unroll
    for (int j = 0; j < MC; ++j) acc[j] = 0.0f;
    for (int q = lane; q < (a.k >> 2); q += 64) {             // (k/4 is a multiple of 64: whole wavefronts)
        const float4 w4 = wr[q];
        #pragma unroll
        for (int j = 0; j < MC; ++j) {
            const int jj = j0 + j < a.rows ? j0 + j : a.rows - 1;             // past the block: the last row again, never stored
            const float4 x4 = ((const float4 *)(a.x + (size_t)jj * a.ldx))[q];
            acc[j] = lg_fmaf(w4.x, x4.x, acc[j]); acc[j] = lg_fmaf(w4.y, x4.y, acc[j]);
            acc[j] = lg_fmaf(w4.z, x4.z, acc[j]); acc[j] = lg_fmaf(w4.w, x4.w, acc[j]);
        }
    }
    #pragma unroll
    for (int j = 0; j < MC; ++j) acc[j] = lg_wave_sum64(acc[j]);
    if (lane < MC && j0 + lane < a.rows) {
        float v = lg_pick<MC>(acc, lane);
        if (a.ipl) v = lg_gelu(v) * a.ipl[(size_t)(j0 + lane) * a.ipl_ld + i];
        a.out[(size_t)(j0 + lane) * a.ldo + i] = v;
    }
}

// ---------------------------------------------------------------------------------------------
// lm_head for verify blocks of 4..8 rows on the matrix cores: lg_k_geglu_m's tile loop (row-block tiles of the
// vocabulary matrix, a wavefront = 64 vocabulary rows x one of the 8 K segments, two v_mfma_i32_32x32x32_i8 per
// tile whatever M is, the activations in the same 80-dword block order) with lg_k_mm_head's epilogue: the 8
// segment sums of a logit meet in the adjacent-pair tree, soft cap, optional store, running argmax per draft row
// (first maximum: the lower index wins ties).  A workgroup walks `passes` consecutive blocks of 64 rows; the
// first tiles of the next block are requested while the last of this one are multiplied, and the segment sums
// go through one of two LDS buffers in turn, so a block costs one barrier.
template <int M>
__global__ __launch_bounds__(512, 2) void lg_k_head_m(LG_HEAD_FIELDS(LG_XP, _) int p_end_) {
    HeadArgs a; LG_HEAD_FIELDS(LG_XI, a)
    extern __shared__ __align__(16) unsigned char smem[];     // [8 segments][nit][80 dwords]
    __shared__ float red[2][8][LG_HIP_MAX_ROWS_DEV][64];
    constexpr int CH = 2;
    const int lane = threadIdx.x & 63, n = lane & 31, h = lane >> 5;
    const int s = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));      // K segment of this wavefront, and its draft row in the epilogue
    const int nb = a.k >> 5, nit = nb >> 3, nblk = a.n_vocab >> 6;
    const int t0 = blockIdx.x * a.passes, np = nblk - t0 < a.passes ? nblk - t0 : a.passes;
    uint4 wq[CH], nwq[CH]; uint32_t wd[CH], nwd[CH];
    auto fetch = [&](int p, int it0) {
        const uint8_t *wt = a.w + ((size_t)(t0 + p) * nb + (size_t)s * nit) * LG_TILE;
        #pragma unroll
        for (int u = 0; u < CH; ++u) {
            const int it = it0 + u < nit ? it0 + u : nit - 1;
            nwq[u] = lg_ldt16(wt, it, lane);
            nwd[u] = lg_ldt2(wt, it, lane);
        }
    };
    unsigned char *la = smem + (size_t)s * nit * (LG_MU_DWORDS * 4);
    {   // the wavefront's K segment of the activations, once (wave-private, no barrier); its first loads go out
        // ahead of the first weight tiles
        const uint4 *src = (const uint4 *)(a.q_in + (size_t)s * nit * (LG_MU_DWORDS * 4));
        const int nu = nit * (LG_MU_DWORDS / 4);
        {   // (every lane takes part, past the end with the last unit again: the tiles are requested in here)
            const int i0 = min(lane, nu - 1), i1 = min(lane + 64, nu - 1), i2 = min(lane + 128, nu - 1), i3 = min(lane + 192, nu - 1);
            const uint4 t0v = src[i0], t1 = src[i1], t2 = src[i2], t3 = src[i3];
            __builtin_amdgcn_sched_barrier(0);
            if (np > 0) fetch(0, 0);
            __builtin_amdgcn_sched_barrier(0);
            ((uint4 *)la)[i0] = t0v; ((uint4 *)la)[i1] = t1; ((uint4 *)la)[i2] = t2; ((uint4 *)la)[i3] = t3;
        }
        for (int i0 = lane + 256; i0 < nu; i0 += 256) {
            const int i1 = min(i0 + 64, nu - 1), i2 = min(i0 + 128, nu - 1), i3 = min(i0 + 192, nu - 1);
            const uint4 t0v = src[i0], t1 = src[i1], t2 = src[i2], t3 = src[i3];
            __builtin_amdgcn_sched_barrier(0);
            ((uint4 *)la)[i0] = t0v; ((uint4 *)la)[i1] = t1; ((uint4 *)la)[i2] = t2; ((uint4 *)la)[i3] = t3;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    lg_v16i magic;                                            // (float)(dot - 8*sum) in one subtraction: see lg_k_geglu_m
    #pragma unroll
    for (int i = 0; i < 16; ++i) magic[i] = 0x4B400000;
    const int arow = n < 8 ? n : 7;
    float best = -INFINITY;                                   // wavefront s < M tracks draft row s, one vocabulary row per lane and block
    int besti = 0x7fffffff;
    for (int p = 0; p < np; ++p) {
        float p0[4] = { 0.0f, 0.0f, 0.0f, 0.0f }, p1[4] = { 0.0f, 0.0f, 0.0f, 0.0f };
        for (int it0 = 0; it0 < nit; it0 += CH) {
            #pragma unroll
            for (int u = 0; u < CH; ++u) { wq[u] = nwq[u]; wd[u] = nwd[u]; }
            if (it0 + CH < nit) fetch(p, it0 + CH);
            else if (p + 1 < np) fetch(p + 1, 0);
            #pragma unroll
            for (int c = 0; c < CH; ++c) {
                if (it0 + c < nit) {
                    const unsigned char *lb = la + (size_t)(it0 + c) * (LG_MU_DWORDS * 4);
                    const lg_v4i av = *(const lg_v4i *)(lb + arow * 32 + h * 16);
                    const int4 sc0 = *(const int4 *)(lb + 256 + h * 32), sc1 = *(const int4 *)(lb + 256 + h * 32 + 16);
                    const uint4 q = wq[c];
                    const lg_v2u s0 = __builtin_amdgcn_permlane32_swap(q.x, q.z, false, false);
                    const lg_v2u s1 = __builtin_amdgcn_permlane32_swap(q.y, q.w, false, false);
                    const lg_v2u sd = __builtin_amdgcn_permlane32_swap(wd[c], wd[c], false, false);
                    lg_v4i b0, b1;
                    b0.x = s0.x & 0x0F0F0F0F; b0.y = s1.x & 0x0F0F0F0F; b0.z = (s0.x >> 4) & 0x0F0F0F0F; b0.w = (s1.x >> 4) & 0x0F0F0F0F;
                    b1.x = s0.y & 0x0F0F0F0F; b1.y = s1.y & 0x0F0F0F0F; b1.z = (s0.y >> 4) & 0x0F0F0F0F; b1.w = (s1.y >> 4) & 0x0F0F0F0F;
                    const float w0 = lg_h2f((uint16_t)sd.x), w1 = lg_h2f((uint16_t)sd.y);
                    const lg_v16i d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, b0, magic, 0, 0, 0);
                    const lg_v16i d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, b1, magic, 0, 0, 0);
                    const float xd[4] = { __int_as_float(sc0.x), __int_as_float(sc0.z), __int_as_float(sc1.x), __int_as_float(sc1.z) };
                    const float cf[4] = { __int_as_float(sc0.y), __int_as_float(sc0.w), __int_as_float(sc1.y), __int_as_float(sc1.w) };
                    #pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        p0[i] = lg_fmaf(xd[i] * w0, __int_as_float(d0[i]) - cf[i], p0[i]);
                        p1[i] = lg_fmaf(xd[i] * w1, __int_as_float(d1[i]) - cf[i], p1[i]);
                    }
                }
            }
        }
        float (*rb)[LG_HIP_MAX_ROWS_DEV][64] = red[p & 1];
        #pragma unroll
        for (int i = 0; i < 4; ++i) { rb[s][4 * h + i][n] = p0[i]; rb[s][4 * h + i][32 + n] = p1[i]; }
        __syncthreads();                                      // (the buffer written two blocks ago was read before the barrier of the last block)
        if (s < M) {
            float g[8];
            #pragma unroll
            for (int c = 0; c < 8; ++c) g[c] = rb[c][s][lane];
            float v = ((g[0] + g[1]) + (g[2] + g[3])) + ((g[4] + g[5]) + (g[6] + g[7]));
            if (a.softcap > 0.0f) v = a.softcap * lg_tanhf(v / a.softcap);
            const int row = (t0 + p) * 64 + lane;
            if (a.logits) a.logits[(size_t)s * a.n_vocab + row] = v;
            if (v > best) { best = v; besti = row; }          // (rows ascend with p: a later equal value never replaces)
        }
    }
    if (s < M) {
        #pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const float ov = __shfl_xor(best, o);
            const int oi = __shfl_xor(besti, o);
            if (ov > best || (ov == best && oi < besti)) { best = ov; besti = oi; }
        }
        if (lane == 0) { a.pval[(size_t)blockIdx.x * M + s] = best; a.pidx[(size_t)blockIdx.x * M + s] = besti; }
    }
}

// ---------------------------------------------------------------------------------------------
// Matmul of a verify block (4..8 rows) against a long-row matrix (S = 32 K segments per row, ffn_down), cut by K
// quarter: workgroup (x, q) takes 8 rows per wavefront and the segments 8q .. 8q+7 of them, so it stages a quarter
// of the activations (24 KB at 5 x 15360, where a workgroup that owns whole rows stages all 96 KB and a CU then
// holds a single workgroup of four wavefronts).  A lane is (row r8, segment sg) and walks the segment's tiles with
// the same serial fma chain as lg_k_mm; the 8 segment sums of a row meet in the same adjacent-pair tree (lg_sum8),
// which is the bottom of the 32-segment tree.  The quarter's partial sums go to slab q of `out` ([4][M][m]); the
// consumer adds the top of the tree, (p0+p1)+(p2+p3).
template <int M>
__global__ __launch_bounds__(320, 2) void lg_k_mm_kq(LG_MM_FIELDS(LG_XP, _) int p_end_) {
    MmArgs a; LG_MM_FIELDS(LG_XI, a)
    extern __shared__ __align__(16) unsigned char smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = a.nthreads >> 6;
    const int q = blockIdx.y, nb = a.k >> 5, nit = nb >> 5;
    uint4 *lq = (uint4 *)smem;                                // [M][nit][2 halves][8 segments] 16-byte units
    float2 *lds = (float2 *)(smem + (size_t)M * nit * 256);   // [M][nit][8 segments] {scale, sum}
    const int r8 = lane >> 3, sg = lane & 7, c = 8 * q + sg;
    const int row0 = (blockIdx.x * nw + wave) * 8;
    const int row = row0 + r8 < a.m ? row0 + r8 : a.m - 1;    // ragged tail: recompute the last row
    // tiles hold two rows x 32 segments: this lane's 16 nibble bytes sit at (row & 1) * 32 + c
    const uint8_t *wt = a.w + (size_t)(row >> 1) * nit * LG_TILE + ((row & 1) * 32 + c) * 16;
    const uint8_t *ws = a.w + (size_t)(row >> 1) * nit * LG_TILE + 1024 + ((row & 1) * 32 + c) * 2;
    constexpr int U = 4;
    struct Chunk { uint4 q[U]; uint32_t s[U]; } cur, nxt;
    auto fetch = [&](Chunk &w, int it0) {
        #pragma unroll
        for (int u = 0; u < U; ++u) {
            const int it = it0 + u < nit ? it0 + u : nit - 1;
            w.q[u] = lg_ldw16(wt + (size_t)it * LG_TILE);
            w.s[u] = lg_ldw2(ws + (size_t)it * LG_TILE);
        }
    };
    {   // the quarter of the activations: per (row, tile) two runs of 8 units and one run of 8 {scale, sum} = 20 x 16 bytes
        // (their first pass is requested ahead of the first weight tiles and stored after them: loads return in order)
        const int n = M * nit * 20, T = a.nthreads;
        const uint4 *gq = (const uint4 *)a.q_in, *gd = (const uint4 *)(a.q_in + (size_t)M * a.k);
        auto where = [&](int i, int &dst) -> const uint4 * {
            const int jt = i / 20, r = i - jt * 20, j = jt / nit, it = jt - j * nit;
            dst = r < 16 ? jt * 16 + r : M * nit * 16 + jt * 4 + (r - 16);
            return r < 16 ? gq + ((size_t)j * (a.k >> 4) + it * 64 + (r >> 3) * 32 + 8 * q + (r & 7))
                          : gd + ((((size_t)j * nb + it * 32 + 8 * q) >> 1) + (r - 16));
        };
        {   // four loads in flight per thread (past the end: the last unit again); every thread takes part in the first pass
            const int i0 = threadIdx.x;
            int d0, d1, d2, d3;
            const uint4 *s0 = where(min(i0, n - 1), d0), *s1 = where(min(i0 + T, n - 1), d1);
            const uint4 *s2 = where(min(i0 + 2 * T, n - 1), d2), *s3 = where(min(i0 + 3 * T, n - 1), d3);
            const uint4 v0 = *s0, v1 = *s1, v2 = *s2, v3 = *s3;
            __builtin_amdgcn_sched_barrier(0);
            fetch(nxt, 0);                                    // (weights depend on nothing)
            __builtin_amdgcn_sched_barrier(0);
            lq[d0] = v0; lq[d1] = v1; lq[d2] = v2; lq[d3] = v3;
        }
        for (int i0 = threadIdx.x + 4 * T; i0 < n; i0 += 4 * T) {
            int d0, d1, d2, d3;
            const uint4 *s0 = where(min(i0, n - 1), d0), *s1 = where(min(i0 + T, n - 1), d1);
            const uint4 *s2 = where(min(i0 + 2 * T, n - 1), d2), *s3 = where(min(i0 + 3 * T, n - 1), d3);
            const uint4 v0 = *s0, v1 = *s1, v2 = *s2, v3 = *s3;
            __builtin_amdgcn_sched_barrier(0);
            lq[d0] = v0; lq[d1] = v1; lq[d2] = v2; lq[d3] = v3;
        }
    }
    __syncthreads();
    if (row0 >= a.m) return;
    float acc[M];
    #pragma unroll
    for (int j = 0; j < M; ++j) acc[j] = 0.0f;
    for (int it0 = 0; it0 < nit; it0 += U) {
        cur = nxt;
        if (it0 + U < nit) fetch(nxt, it0 + U);
        #pragma unroll
        for (int u = 0; u < U; ++u) {
            if (it0 + u < nit) {
                const int it = it0 + u;
                float2 ds[M]; int4 a0[M], a1[M];
                #pragma unroll
                for (int j = 0; j < M; ++j) {
                    const int jt = j * nit + it;
                    ds[j] = lds[jt * 8 + sg];
                    a0[j] = *(const int4 *)(lq + jt * 16 + sg); a1[j] = *(const int4 *)(lq + jt * 16 + 8 + sg);
                }
                __builtin_amdgcn_sched_barrier(0);
                const float dw = lg_h2f((uint16_t)cur.s[u]);
                #pragma unroll
                for (int j = 0; j < M; ++j) {
                    const int dot = lg_block_dot(cur.q[u], a0[j], a1[j], __float_as_int(ds[j].y));
                    acc[j] = lg_fmaf(ds[j].x * dw, (float)dot, acc[j]);
                }
            }
        }
    }
    #pragma unroll
    for (int j = 0; j < M; ++j) acc[j] = lg_sum8(acc[j]);
    if (sg < M && row0 + r8 < a.m) a.out[((size_t)q * M + sg) * a.m + row] = lg_pick<M>(acc, sg);
}

// ---------------------------------------------------------------------------------------------
// Attention tiles of a verify block for layers with many tiles (long global contexts, wide sliding windows):
// one workgroup per (tile, kv head) serves ALL rows of the block against one staged K/V tile, where lg_k_attn
// runs a workgroup per row and stages every tile once per row.  FQ = false: the queries arrive normed and rotated
// (lg_k_qkv_post has run and has written the block's K/V rows to the cache).  FQ = true: the kernel does that work
// itself from the raw projections, one launch less per layer: every workgroup norms and rotates the M*G queries of
// its kv head (a wavefront per query, written in the staged order), and the one workgroup whose tile holds rows of
// the block builds those K/V rows straight into its LDS tile and stores them to the cache (K row r by wavefront
// r % 4, V row r by wavefront 3 - r % 4; the ring has spare rows, so no row another workgroup reads is overwritten).
// Same arithmetic and order as
// lg_k_attn: score = (a0+a1)+(a2+a3) over four fma chains, tile max / exp / 32-lane tree sum, value accumulation
// over the slots ascending; the partials go to the same slots and lg_k_attn_merge finishes them.
//
// A unit is one (row, query head) pair, M*G of them; a wavefront takes the units wave, wave + 4, ... three at a
// time, so that one LDS read of a K (V) row serves three units and 6 (12) independent fma chains are in flight.
// K is staged in reader order (the lane of key slot sl and chain pair hf finds its hd/4 dwords as consecutive
// 16-byte units); the queries are read 16 bytes at a time, the same address in all lanes of a half.  Every slot of
// a tile goes through the value chains: slots outside a row's keys have exponential zero and zeroed or finite
// values, and fma(0, v, acc) is acc for every acc that a chain started at +0 can hold.
//
// A workgroup takes `tp` consecutive tiles; the next tile's rows are requested into registers before the current
// tile is computed, so the memory latency of all tiles but the first is covered.

// fmaf(x, (float)h, acc) with h the low (high) f16 half of a packed pair: one instruction; the conversion is exact
// and the sum rounds once, as the two-instruction form does.  The compiler picks this instruction by itself when a
// converted value feeds one fma; written out here because each key/value element feeds one fma per unit.
__device__ __forceinline__ float lg_fma_hlo(float x, uint32_t hp, float acc) {
    asm("v_fma_mix_f32 %0, %1, %2, %0 op_sel_hi:[0,1,0]" : "+v"(acc) : "v"(x), "v"(hp));
    return acc;
}
__device__ __forceinline__ float lg_fma_hhi(float x, uint32_t hp, float acc) {
    asm("v_fma_mix_f32 %0, %1, %2, %0 op_sel:[0,1,0] op_sel_hi:[0,1,0]" : "+v"(acc) : "v"(x), "v"(hp));
    return acc;
}

template <int HD>
struct AttnRowsGeo {
    static constexpr int KSD = HD / 2 + 4;                    // dwords per staged K row (16-byte reads of 8 slots cover all banks)
    static constexpr int VST = HD + 8;                        // halves per staged V row
    static size_t bytes(int units, bool fq = false) {         // fq: a vector of staging per wavefront for the rotary
        return (size_t)units * HD * 4 + (size_t)32 * KSD * 4 + (size_t)32 * VST * 2 + (size_t)units * 32 * 4 + (fq ? (size_t)(LG_WG / 64) * HD * 4 : 0);
    }
};
template <int M, int HD, bool FQ = false>
__global__ __launch_bounds__(LG_WG) void lg_k_attn_rows(const StepCtl *ctl, int tp, LG_ATTN_FIELDS(LG_XP, _) int p_end_) {
    AttnArgs a; LG_ATTN_FIELDS(LG_XI, a)
    using Geo = AttnRowsGeo<HD>;
    extern __shared__ __align__(16) unsigned char smem[];
    const int G = a.H / a.nkv, units = M * G;
    float *qs = (float *)smem;                                // [unit][hf][HD/2]: element i at hf = (i%4)/2, 2*(i/4) + i%2
    uint32_t *kt = (uint32_t *)(qs + (size_t)units * HD);     // [32][KSD]: row sl = [hf][HD/4 dwords]
    uint16_t *vt = (uint16_t *)(kt + 32 * Geo::KSD);          // [32][VST]
    float *es = (float *)(vt + 32 * Geo::VST);                // [unit][32]
    float *hv = es + (size_t)units * 32;                      // FQ: [wavefront][HD] staging of the rotary
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int kvh = blockIdx.y;
    const int pos0 = ctl->pos + a.pos_off, plast = pos0 + M - 1;
    // FQ: positions tnew..plast are rows of the block itself (none when the layer reads another layer's cache)
    const int tnew = (FQ && a.kcw) ? ctl->pos : 0x7FFFFFFF;
    const int start0 = lg_win_start(pos0, a.window), first = start0 >> 5, last = plast >> 5;
    const int b0 = blockIdx.x * tp;                           // tiles first + b0 .. first + b0 + tp - 1
    if (first + b0 > last) return;                            // no row of the block has keys here
    constexpr int U4R = HD / 8;                               // 16-byte units per K/V row
    constexpr int KL = (32 * U4R + LG_WG - 1) / LG_WG;        // 16-byte units of K (and of V) per thread
    static_assert(32 * U4R % LG_WG == 0 || 32 * U4R < LG_WG, "tile staging assumes whole passes");
    uint4 kq[KL], vq[KL];
    auto fetch = [&](int bx) {
        const int r0 = ((first + bx) << 5) % a.seq;
        #pragma unroll
        for (int u = 0; u < KL; ++u) {
            const int idx = min((int)threadIdx.x + u * LG_WG, 32 * U4R - 1), row = idx / U4R, u4 = idx - row * U4R;
            int rr = r0 + row; if (rr >= a.seq) rr -= a.seq;
            const size_t go = (size_t)rr * a.kv_dim + (size_t)kvh * HD + u4 * 8;
            kq[u] = a.kc4s(go); vq[u] = a.vc4s(go);
        }
    };
    auto stash = [&](int bx) {
        // slots outside the keys of every row of the block are zeroed (their exponentials are zero, and zero times
        // a finite value leaves the sums as they are; stale bits that read as infinities would not)
        const int t0 = (first + bx) << 5, slo = start0 - t0, shi = plast - t0;
        #pragma unroll
        for (int u = 0; u < KL; ++u) {
            const int idx = (int)threadIdx.x + u * LG_WG, row = idx / U4R, u4 = idx - row * U4R;
            if (32 * U4R < LG_WG && idx >= 32 * U4R) continue;
            if (FQ && t0 + row >= tnew && row <= shi) continue;               // a row of the block: built below, not in the cache yet
            const uint32_t mk = (row >= slo && row <= shi) ? 0xFFFFFFFFu : 0u;
            uint32_t *d = kt + row * Geo::KSD + 2 * u4;
            *(uint2 *)d = make_uint2(kq[u].x & mk, kq[u].z & mk);             // chains 0,1 of two groups of four dims
            *(uint2 *)(d + HD / 4) = make_uint2(kq[u].y & mk, kq[u].w & mk);  // chains 2,3
            *(uint4 *)(vt + row * Geo::VST + u4 * 8) = make_uint4(vq[u].x & mk, vq[u].y & mk, vq[u].z & mk, vq[u].w & mk);
        }
    };
    constexpr int JOBS = 2 * ((M + 3) / 4);                   // FQ: K and V rows of the block one wavefront may have to build
    constexpr int QBATCH = 4;                                 // FQ: queries one wavefront prepares at a time
    HeadVec<1> hj[FQ ? JOBS : 1], hq[FQ ? QBATCH : 1], wk, wq;
    RopeVals<1> rv;
    if constexpr (FQ) {
        // What the preparation reads is requested ahead of the tile (loads return in order): the block's projections
        // come from the cache levels, the tile from memory, so the queries are prepared while the tile is on its way.
        // Raw rows of the block that fall into this workgroup's tiles are requested here too and used when their tile
        // is staged.
        const int tlo = (first + b0) << 5, thi = ((first + b0 + tp) << 5) - 1;
        rv = lg_rope_load<1>(a.rope_tab, a.rope_ff, HD);
        wq = lg_head_load<1>(a.q_norm, HD);
        #pragma unroll
        for (int b = 0; b < QBATCH; ++b) {                    // unit u = (row j, head g), by wavefront u % 4
            const int u = wave + b * (LG_WG / 64) < units ? wave + b * (LG_WG / 64) : min(wave, units - 1), j = u / G, g = u - j * G;
            hq[b] = lg_head_load<1>(a.qkv + (size_t)j * a.ld + (size_t)(kvh * G + g) * HD, HD);
        }
        const bool any = tnew <= plast && plast >= tlo && tnew <= thi;
        wk = lg_head_load<1>(any ? a.k_norm : a.q_norm, HD);  // (no K rows to build: k_norm may not exist)
        #pragma unroll
        for (int u = 0; u < JOBS; ++u) {                      // first half of the slots: K rows wave, wave+4; second half: V rows 3-wave, 7-wave
            const bool isv = u >= JOBS / 2;
            const int r = (isv ? 3 - wave : wave) + 4 * (u % (JOBS / 2)), t = tnew + r;
            if (any && r < M && t >= tlo && t <= thi) hj[u] = lg_head_load<1>(a.qkv + (size_t)r * a.ld + (isv ? a.v_off : a.k_off) + (size_t)kvh * HD, HD);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    fetch(b0);
    if constexpr (FQ) {
        __builtin_amdgcn_sched_barrier(0);
        // a batch in stages, so that the sums and the rotary of its queries overlap: norms of all, each into its own
        // slot of qs in natural order; all rotary pairs read back; then the slots rewritten in the staged order
        // (a unit past the last repeats the batch's first one, a slot of this wavefront, and stores nothing)
        auto unit_of = [&](int base, int b) { return base + b * (LG_WG / 64) < units ? base + b * (LG_WG / 64) : base; };
        for (int base = wave; base < units; base += QBATCH * (LG_WG / 64)) {
            if (base != wave) {
                #pragma unroll
                for (int b = 0; b < QBATCH; ++b) {
                    const int u = unit_of(base, b), j = u / G, g = u - j * G;
                    hq[b] = lg_head_load<1>(a.qkv + (size_t)j * a.ld + (size_t)(kvh * G + g) * HD, HD);
                }
            }
            HeadVec<1> nq[QBATCH];
            #pragma unroll
            for (int b = 0; b < QBATCH; ++b) nq[b] = lg_head_norm<1>(hq[b], wq, true, HD, a.eps);
            #pragma unroll
            for (int b = 0; b < QBATCH; ++b)
                if (4 * lane < HD) *(float4 *)(qs + (size_t)unit_of(base, b) * HD + 4 * lane) = nq[b].x[0];
            lg_wave_lds_sync();
            float lo[QBATCH][2], hi[QBATCH][2];
            #pragma unroll
            for (int b = 0; b < QBATCH; ++b) {
                const int u = unit_of(base, b), j = u / G;
                const float *vec = qs + (size_t)u * HD;
                #pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const int p = min(lane + 64 * i, HD / 2 - 1);
                    const float ang = (float)(ctl->pos + j) * rv.tab[i] / rv.ff[i];
                    float sn, cs;
                    lg_sincosf(ang, &sn, &cs);
                    const float x0 = vec[p], x1 = vec[p + HD / 2];
                    lo[b][i] = x0 * cs - x1 * sn; hi[b][i] = x0 * sn + x1 * cs;
                }
            }
            lg_wave_lds_sync();                               // (LDS serves a wavefront in order: every read above is ahead of the stores below)
            #pragma unroll
            for (int b = 0; b < QBATCH; ++b) {
                const int u = base + b * (LG_WG / 64);
                float *qd = qs + (size_t)unit_of(base, b) * HD;
                #pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const int p = lane + 64 * i, p1 = p + HD / 2;
                    if (u >= units || p >= HD / 2) continue;
                    // element i sits at hf = (i%4)/2, 2*(i/4) + i%2
                    qd[((p & 3) >> 1) * (HD / 2) + 2 * (p >> 2) + (p & 1)] = lo[b][i];
                    qd[((p1 & 3) >> 1) * (HD / 2) + 2 * (p1 >> 2) + (p1 & 1)] = hi[b][i];
                }
            }
            lg_wave_lds_sync();
        }
    } else {   // the queries, once per workgroup (their loads follow the first tile's before any store)
        constexpr int QB = 4;                                 // float4 of query per thread and pass
        const int nq4 = units * (HD / 4);
        for (int base = 0; base < nq4; base += QB * LG_WG) {
            float4 qreg[QB];
            #pragma unroll
            for (int i = 0; i < QB; ++i) {
                const int idx = min(base + (int)threadIdx.x + i * LG_WG, nq4 - 1);
                const int u = idx / (HD / 4), g4 = idx - u * (HD / 4), j = u / G, g = u - j * G;
                qreg[i] = *(const float4 *)(a.q + (size_t)j * a.H * HD + (size_t)(kvh * G + g) * HD + 4 * g4);
            }
            #pragma unroll
            for (int i = 0; i < QB; ++i) {
                const int idx = base + (int)threadIdx.x + i * LG_WG;
                if (idx < nq4) {
                    const int u = idx / (HD / 4), g4 = idx - u * (HD / 4);
                    float *qd = qs + (size_t)u * HD + 2 * g4;
                    *(float2 *)qd = make_float2(qreg[i].x, qreg[i].y);
                    *(float2 *)(qd + HD / 2) = make_float2(qreg[i].z, qreg[i].w);
                }
            }
        }
    }
    constexpr int NWV = LG_WG / 64, UB = 3;
    for (int i = 0; i < tp; ++i) {
        const int bx = b0 + i, n = first + bx, t0 = n << 5;
        if (n > last) break;
        if (i > 0) __syncthreads();                           // the previous tile has been read by every wavefront
        if constexpr (FQ) {                                   // rows of the block in this tile: built while the tile is on its way (stash leaves their slots alone)
            if (tnew <= plast && tnew <= t0 + 31 && plast >= t0) {            // this tile holds rows of the block
                float *vec = hv + (size_t)wave * HD;
                HeadVec<1> nr[JOBS];
                int slj[JOBS];
                #pragma unroll
                for (int u = 0; u < JOBS; ++u) {              // the norms of all of them first: their sums overlap
                    const bool isv = u >= JOBS / 2;
                    const int r = (isv ? 3 - wave : wave) + 4 * (u % (JOBS / 2)), sl = tnew + r - t0;
                    slj[u] = (r < M && sl >= 0 && sl <= 31) ? sl : -1;
                    if (slj[u] >= 0) nr[u] = lg_head_norm<1>(hj[u], wk, !isv, HD, a.eps);
                }
                #pragma unroll
                for (int u = 0; u < JOBS; ++u) {
                    const bool isv = u >= JOBS / 2;
                    const int sl = slj[u], t = t0 + sl;
                    if (sl < 0) continue;
                    const size_t coff = (size_t)(t % a.seq) * a.kv_dim + (size_t)kvh * HD;
                    if (isv) {                                // V: no rotary, straight from the registers
                        if (4 * lane < HD) {
                            const uint2 h4 = make_uint2((uint32_t)lg_f2h(nr[u].x[0].x) | ((uint32_t)lg_f2h(nr[u].x[0].y) << 16),
                                                        (uint32_t)lg_f2h(nr[u].x[0].z) | ((uint32_t)lg_f2h(nr[u].x[0].w) << 16));
                            *(uint2 *)(vt + sl * Geo::VST + 4 * lane) = h4;
                            *(uint2 *)(a.vcw + coff + 4 * lane) = h4;
                        }
                    } else {
                        uint16_t *row = (uint16_t *)(kt + sl * Geo::KSD), *crow = a.kcw + coff;
                        lg_head_rope<1>(nr[u], HD, t, rv, vec, [&](int p, float lo, float hi) {
                            const int p1 = p + HD / 2;        // dims 4g, 4g+1 in dword g of the first half, 4g+2, 4g+3 of the second
                            const uint16_t hl = lg_f2h(lo), hh = lg_f2h(hi);
                            row[2 * (((p & 3) >> 1) * (HD / 4) + (p >> 2)) + (p & 1)] = hl;
                            row[2 * (((p1 & 3) >> 1) * (HD / 4) + (p1 >> 2)) + (p1 & 1)] = hh;
                            crow[p] = hl; crow[p1] = hh;
                        });
                    }
                }
            }
        }
        stash(bx);
        __syncthreads();
        if (i + 1 < tp && n + 1 <= last) fetch(bx + 1);
        {   // scores
            const int sl = lane & 31, hf = lane >> 5, t = t0 + sl;
            const uint32_t *ks = kt + sl * Geo::KSD + hf * (HD / 4);
            for (int ub = wave; ub < units; ub += UB * NWV) {
                int un[UB];
                const float *qr[UB];
                float ax[UB], ay[UB];
                #pragma unroll
                for (int b = 0; b < UB; ++b) {                // (a missing unit repeats the first one and stores nothing)
                    un[b] = ub + b * NWV < units ? ub + b * NWV : ub;
                    qr[b] = qs + (size_t)un[b] * HD + hf * (HD / 2);
                    ax[b] = 0.0f; ay[b] = 0.0f;
                }
                #pragma unroll 2
                for (int u = 0; u < HD / 16; ++u) {
                    const uint4 k4 = *(const uint4 *)(ks + 4 * u);
                    #pragma unroll
                    for (int b = 0; b < UB; ++b) {
                        const float4 p0 = *(const float4 *)(qr[b] + 8 * u), p1 = *(const float4 *)(qr[b] + 8 * u + 4);
                        ax[b] = lg_fma_hlo(p0.x, k4.x, ax[b]); ay[b] = lg_fma_hhi(p0.y, k4.x, ay[b]);
                        ax[b] = lg_fma_hlo(p0.z, k4.y, ax[b]); ay[b] = lg_fma_hhi(p0.w, k4.y, ay[b]);
                        ax[b] = lg_fma_hlo(p1.x, k4.z, ax[b]); ay[b] = lg_fma_hhi(p1.y, k4.z, ay[b]);
                        ax[b] = lg_fma_hlo(p1.z, k4.w, ax[b]); ay[b] = lg_fma_hhi(p1.w, k4.w, ay[b]);
                    }
                }
                #pragma unroll
                for (int b = 0; b < UB; ++b) {
                    if (b > 0 && un[b] == ub) continue;
                    const int unit = un[b], j = unit / G, pj = pos0 + j, startj = lg_win_start(pj, a.window);
                    if (n < (startj >> 5) || n > (pj >> 5)) continue;         // tile outside this row's keys (wavefront-uniform)
                    const bool valid = t >= startj && t <= pj;
                    float s = lg_add_x32(ax[b] + ay[b]);      // (a0+a1) + (a2+a3): the two halves sit 32 lanes apart
                    if (!valid) s = -INFINITY;
                    const float mx = lg_max_n(s, 32);
                    const float e = valid ? lg_expf(s - mx) : 0.0f;
                    const float l = lg_sum32(e);
                    if (hf == 0) es[unit * 32 + sl] = e;
                    if (lane == 0) {
                        const size_t pi = ((size_t)j * a.H + kvh * G + (unit - j * G)) * a.tiles_max + bx;
                        a.pm[pi] = mx; a.pl[pi] = l;
                    }
                }
            }
        }
        __syncthreads();
        {   // values (lane = 4 dims)
            const uint16_t *vl = vt + (4 * lane < HD ? 4 * lane : 0);
            for (int ub = wave; ub < units; ub += UB * NWV) {
                int un[UB];
                bool on[UB];
                const float *er[UB];
                float4 acc[UB];
                #pragma unroll
                for (int b = 0; b < UB; ++b) {
                    un[b] = ub + b * NWV < units ? ub + b * NWV : ub;
                    const int j = un[b] / G, pj = pos0 + j, startj = lg_win_start(pj, a.window);
                    on[b] = !(n < (startj >> 5) || n > (pj >> 5)) && !(b > 0 && un[b] == ub);
                    er[b] = es + un[b] * 32;                  // (a unit that skipped the scores has stale rows here: never stored)
                    acc[b] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                }
                #pragma unroll 2
                for (int u4 = 0; u4 < 8; ++u4) {
                    float ev[UB][4];
                    #pragma unroll
                    for (int b = 0; b < UB; ++b) {
                        const float4 e4 = *(const float4 *)(er[b] + 4 * u4);
                        ev[b][0] = e4.x; ev[b][1] = e4.y; ev[b][2] = e4.z; ev[b][3] = e4.w;
                    }
                    #pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const uint2 v = *(const uint2 *)(vl + (4 * u4 + q) * Geo::VST);
                        #pragma unroll
                        for (int b = 0; b < UB; ++b) {
                            acc[b].x = lg_fma_hlo(ev[b][q], v.x, acc[b].x); acc[b].y = lg_fma_hhi(ev[b][q], v.x, acc[b].y);
                            acc[b].z = lg_fma_hlo(ev[b][q], v.y, acc[b].z); acc[b].w = lg_fma_hhi(ev[b][q], v.y, acc[b].w);
                        }
                    }
                }
                #pragma unroll
                for (int b = 0; b < UB; ++b) {
                    if (!on[b]) continue;
                    const int unit = un[b], j = unit / G;
                    const size_t pi = ((size_t)j * a.H + kvh * G + (unit - j * G)) * a.tiles_max + bx;
                    if (4 * lane < HD) *(float4 *)(a.pacc + pi * HD + 4 * lane) = acc[b];
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Attention tiles of prompt blocks with the queries in registers: a workgroup is 8 (row, head) units (two rows x four
// heads, four x two, ...), a wavefront IS a unit.
// In the score phase lane (k, c) = key k of 16, chain c of the 4, holds the unit's query elements of its chain
// (q[4g+c], g = 0..hd/4-1: hd/4 registers, loaded once per workgroup) and reads its key's elements of that chain from
// a K tile staged chain-major, 16 bytes = 8 steps of the chain at a time: no LDS traffic for the queries at all, where
// lg_k_attn and lg_k_attn_rows fetch a query element per fma from LDS and are bound by that.  The two 16-key
// halves of a tile run as two independent chains.  The chains of a key meet as (a0+a1)+(a2+a3) by two quad swaps;
// the tile sum of the exponentials is the same adjacent-pair tree as lg_sum32 (slot = 16 * half + k: lane bits 2..5
// are slot bits 0..3, the halves are bit 4).  In the value phase (lane = 4 dims) the weight of slot s is read out of
// the lane of its key into a scalar register.  Every slot goes through the value chains (masked slots weigh exactly
// zero and their rows are zeroed at staging).  A workgroup walks `tp` tiles, the next one's rows in flight while the
// current one is computed; the first four wavefronts stage.  Partials as lg_k_attn writes them.
__device__ __forceinline__ float lg_fma_hlo_s(float x, uint32_t hp, float acc) {
    asm("v_fma_mix_f32 %0, %1, %2, %0 op_sel_hi:[0,1,0]" : "+v"(acc) : "s"(x), "v"(hp));
    return acc;
}
__device__ __forceinline__ float lg_fma_hhi_s(float x, uint32_t hp, float acc) {
    asm("v_fma_mix_f32 %0, %1, %2, %0 op_sel:[0,1,0] op_sel_hi:[0,1,0]" : "+v"(acc) : "s"(x), "v"(hp));
    return acc;
}
template <int HD>
struct AttnUGeo {
    static constexpr int CS = HD / 2 + 16;                    // bytes per (key, chain) run of the K tile: hd/4 halves + pad
    static constexpr int KS = 4 * CS;                         // bytes per key (groups of 8 lanes = 2 keys x 4 chains cover all banks)
    static constexpr int VS = HD * 2 + 16;                    // bytes per V row
    static constexpr int QC = HD / 4 + 4;                     // floats per chain of a staged query
    static size_t bytes(int units) { return (size_t)units * 4 * QC * 4 + (size_t)32 * KS + (size_t)32 * VS; }
};
template <int HD>                                             // (up to 256-wide heads: 128 registers a lane, two workgroups per CU)
__global__ __launch_bounds__(512, HD > 256 ? 2 : 4) void lg_k_attn_u(AttnArgs a, const StepCtl *ctl, int rw, int tp) {
    using Geo = AttnUGeo<HD>;
    extern __shared__ __align__(16) unsigned char smem[];
    const int G = a.H / a.nkv, units = 8;                     // rw * G == 8, blockDim.x == 512
    float *qs = (float *)smem;                                // [unit][4 chains][QC]
    unsigned char *kt = smem + (size_t)units * 4 * Geo::QC * 4;               // [32 keys][4 chains][CS]
    unsigned char *vt = kt + 32 * Geo::KS;                    // [32][VS]
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    const int kvh = blockIdx.y, j0 = blockIdx.z * rw, posb = ctl->pos + a.pos_off;
    // tiles are numbered from the first tile of the whole block, as lg_k_attn_merge reads them
    const int first = lg_win_start(posb, a.window) >> 5;
    const int glo = lg_win_start(posb + j0, a.window), ghi = posb + j0 + rw - 1;         // keys any row of the group sees
    const int n0 = (glo >> 5) + blockIdx.x * tp;
    int n1 = n0 + tp - 1; if (n1 > (ghi >> 5)) n1 = ghi >> 5;
    if (n0 > n1) return;
    constexpr int U4R = HD / 8;                               // 16-byte units per row
    constexpr int STG = 32 * U4R >= 512 ? 512 : 256;          // staging threads
    constexpr int KL = 32 * U4R / STG;                        // units per staging thread and matrix
    static_assert(32 * U4R % STG == 0, "tile staging assumes whole passes");
    const bool stager = threadIdx.x < STG;
    uint4 kq[KL], vq[KL];
    auto fetch = [&](int n) {
        const int r0 = (n << 5) % a.seq;
        #pragma unroll
        for (int u = 0; u < KL; ++u) {
            const int idx = (int)threadIdx.x + u * STG, row = idx / U4R, u4 = idx - row * U4R;
            int rr = r0 + row; if (rr >= a.seq) rr -= a.seq;
            const size_t go = (size_t)rr * a.kv_dim + (size_t)kvh * HD + u4 * 8;
            kq[u] = a.kc4s(go); vq[u] = a.vc4s(go);
        }
    };
    auto stash = [&](int n) {
        const int t0 = n << 5;
        #pragma unroll
        for (int u = 0; u < KL; ++u) {
            const int idx = (int)threadIdx.x + u * STG, row = idx / U4R, u4 = idx - row * U4R;
            const uint32_t mk = (t0 + row >= glo && t0 + row <= ghi) ? 0xFFFFFFFFu : 0u;
            const uint4 k = make_uint4(kq[u].x & mk, kq[u].y & mk, kq[u].z & mk, kq[u].w & mk);
            unsigned char *d = kt + row * Geo::KS + u4 * 4;   // steps 2*u4, 2*u4+1 of every chain: elements c and 4+c of the 8
            *(uint32_t *)(d) = (k.x & 0xFFFFu) | (k.z << 16);
            *(uint32_t *)(d + Geo::CS) = (k.x >> 16) | (k.z & 0xFFFF0000u);
            *(uint32_t *)(d + 2 * Geo::CS) = (k.y & 0xFFFFu) | (k.w << 16);
            *(uint32_t *)(d + 3 * Geo::CS) = (k.y >> 16) | (k.w & 0xFFFF0000u);
            *(uint4 *)(vt + row * Geo::VS + u4 * 16) = make_uint4(vq[u].x & mk, vq[u].y & mk, vq[u].z & mk, vq[u].w & mk);
        }
    };
    if (stager) fetch(n0);
    // this wavefront's unit and its query, chain-major through its own LDS rows into registers
    const int j = j0 + wave / G, head = kvh * G + wave % G, pj = posb + j, startj = lg_win_start(pj, a.window);
    const int kk = lane >> 2, c = lane & 3;
    float qreg[HD / 4];
    {
        float *qw = qs + (size_t)wave * 4 * Geo::QC;
        const float4 *qrow = (const float4 *)(a.q + (size_t)j * a.H * HD + (size_t)head * HD);
        #pragma unroll
        for (int i = 0; i < (HD / 4 + 63) / 64; ++i) {
            const int g = lane + 64 * i;
            if (g < HD / 4) {
                const float4 f = qrow[g];
                qw[g] = f.x; qw[Geo::QC + g] = f.y; qw[2 * Geo::QC + g] = f.z; qw[3 * Geo::QC + g] = f.w;
            }
        }
        lg_wave_lds_sync();
        #pragma unroll
        for (int i = 0; i < HD / 16; ++i) {
            const float4 f = *(const float4 *)(qw + c * Geo::QC + 4 * i);
            qreg[4 * i] = f.x; qreg[4 * i + 1] = f.y; qreg[4 * i + 2] = f.z; qreg[4 * i + 3] = f.w;
        }
    }
    for (int n = n0; n <= n1; ++n) {
        if (n > n0) __syncthreads();                          // the previous tile has been read by every wavefront
        if (stager) stash(n);
        __syncthreads();
        if (stager && n < n1) fetch(n + 1);
        if (n < (startj >> 5) || n > (pj >> 5)) continue;     // tile outside this unit's keys (wavefront-uniform; barriers are above)
        const int t0 = n << 5, bx = n - first;
        float e0, e1;
        {   // scores of keys kk and 16 + kk, chain c
            const unsigned char *k0 = kt + kk * Geo::KS + c * Geo::CS, *k1 = k0 + 16 * Geo::KS;
            float a0 = 0.0f, a1 = 0.0f;
            #pragma unroll
            for (int i = 0; i < HD / 32; ++i) {
                const uint4 x = *(const uint4 *)(k0 + 16 * i), y = *(const uint4 *)(k1 + 16 * i);
                a0 = lg_fma_hlo(qreg[8 * i], x.x, a0);     a1 = lg_fma_hlo(qreg[8 * i], y.x, a1);
                a0 = lg_fma_hhi(qreg[8 * i + 1], x.x, a0); a1 = lg_fma_hhi(qreg[8 * i + 1], y.x, a1);
                a0 = lg_fma_hlo(qreg[8 * i + 2], x.y, a0); a1 = lg_fma_hlo(qreg[8 * i + 2], y.y, a1);
                a0 = lg_fma_hhi(qreg[8 * i + 3], x.y, a0); a1 = lg_fma_hhi(qreg[8 * i + 3], y.y, a1);
                a0 = lg_fma_hlo(qreg[8 * i + 4], x.z, a0); a1 = lg_fma_hlo(qreg[8 * i + 4], y.z, a1);
                a0 = lg_fma_hhi(qreg[8 * i + 5], x.z, a0); a1 = lg_fma_hhi(qreg[8 * i + 5], y.z, a1);
                a0 = lg_fma_hlo(qreg[8 * i + 6], x.w, a0); a1 = lg_fma_hlo(qreg[8 * i + 6], y.w, a1);
                a0 = lg_fma_hhi(qreg[8 * i + 7], x.w, a0); a1 = lg_fma_hhi(qreg[8 * i + 7], y.w, a1);
            }
            // (a0+a1)+(a2+a3) over the four chain lanes of a key
            a0 = a0 + lg_dpp_f<LG_DPP_SWAP1>(a0); a0 = a0 + lg_dpp_f<LG_DPP_SWAP2>(a0);
            a1 = a1 + lg_dpp_f<LG_DPP_SWAP1>(a1); a1 = a1 + lg_dpp_f<LG_DPP_SWAP2>(a1);
            const int ta = t0 + kk, tb = ta + 16;
            const bool va = ta >= startj && ta <= pj, vb = tb >= startj && tb <= pj;
            const float s0 = va ? a0 : -INFINITY, s1 = vb ? a1 : -INFINITY;
            const float mx = lg_max_n(fmaxf(s0, s1), 64);
            e0 = va ? lg_expf(s0 - mx) : 0.0f;
            e1 = vb ? lg_expf(s1 - mx) : 0.0f;
            // lg_sum32 over slot = 16 * half + kk: slot bits 0..3 are lane bits 2..5 (values repeat over the chain lanes,
            // so the mirrors that also flip lower lane bits pair the same values), bit 4 is the half
            float l0 = e0, l1 = e1;
            l0 = l0 + lg_dpp_f<LG_DPP_MIRROR8>(l0);  l1 = l1 + lg_dpp_f<LG_DPP_MIRROR8>(l1);
            l0 = l0 + lg_dpp_f<LG_DPP_MIRROR16>(l0); l1 = l1 + lg_dpp_f<LG_DPP_MIRROR16>(l1);
            l0 = lg_add_x16(l0); l1 = lg_add_x16(l1);
            l0 = lg_add_x32(l0); l1 = lg_add_x32(l1);
            if (lane == 0) {
                const size_t pi = ((size_t)j * a.H + head) * a.tiles_max + bx;
                a.pm[pi] = mx; a.pl[pi] = l0 + l1;
            }
        }
        // values: lane = 4 dims of each 256
        #pragma unroll
        for (int dh = 0; dh < HD; dh += 256) {
            const bool live = dh + 4 * lane < HD;
            const unsigned char *vl = vt + (live ? (dh + 4 * lane) * 2 : 0);
            float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            #pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int eb = __float_as_int(half ? e1 : e0);
                // eight slots' values requested together, then their 32 fma (lane numbers of the weights are constants:
                // left as a loop, every slot pays a scalar add, its wait states and an LDS round trip of its own)
                #pragma unroll
                for (int k0 = 0; k0 < 16; k0 += 8) {
                    uint2 v[8];
                    #pragma unroll
                    for (int k = 0; k < 8; ++k) v[k] = *(const uint2 *)(vl + (16 * half + k0 + k) * Geo::VS);
                    __builtin_amdgcn_sched_barrier(0);
                    #pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        const float es = __int_as_float(__builtin_amdgcn_readlane(eb, 4 * (k0 + k)));
                        acc.x = lg_fma_hlo_s(es, v[k].x, acc.x); acc.y = lg_fma_hhi_s(es, v[k].x, acc.y);
                        acc.z = lg_fma_hlo_s(es, v[k].y, acc.z); acc.w = lg_fma_hhi_s(es, v[k].y, acc.w);
                    }
                }
            }
            if (live) {
                const size_t pi = ((size_t)j * a.H + head) * a.tiles_max + bx;
                *(float4 *)(a.pacc + pi * HD + dh + 4 * lane) = acc;
            }
        }
    }
}

// lg_k_attn_merge for rows with very many tiles: one workgroup of four wavefronts per (head, row, 64 dims).  The
// merge is one fma chain over the tiles ascending, and walked by a single wavefront its time is the instruction issue
// of 2 loads + 2 fma per tile, tile after tile.  Here the tiles go in rounds of 256: wavefront w requests the 64
// partials of tiles 64w..64w+63 of the round at once (all four wavefronts' loads in flight together) while the
// workgroup computes the round's weights exp(m_t - M) into LDS; then the chain passes through the wavefronts in
// order, each running its 64 fma back to back from registers and handing (L, o) to the next through LDS.  Same
// order, same bits: weights exp(m_t - M), L and the output as fma chains over the tiles ascending, divide, q8.
template <int M>
__global__ __launch_bounds__(LG_WG) void lg_k_attn_merge_split(const StepCtl *ctl, LG_MERGE_FIELDS(LG_XP, _) int p_end_) {
    MergeArgs a; LG_MERGE_FIELDS(LG_XI, a)
    __shared__ float wts[256], pls[256], hand[2][64], wmx[4];
    const int head = blockIdx.x, j = blockIdx.y, hd = a.hd, qd = a.H * hd, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int d = blockIdx.z * 64 + lane;                     // hd is a multiple of 64
    const int pos = ctl->pos + a.pos_off, pj = pos + j;
    const int first = lg_win_start(pos, a.window) >> 5;
    const int lo = (lg_win_start(pj, a.window) >> 5) - first, hi = (pj >> 5) - first;
    const size_t base = ((size_t)j * a.H + head) * a.tiles_max + lo;
    const int nt = hi - lo + 1;
    constexpr int U = 64;
    float pa[U];
    // (buffer loads: the row's partials as the base in scalar registers, the lane's dim as the lane offset, the tile's
    // offset in a scalar register; a flat load each cost a dozen vector instructions of 64-bit address arithmetic)
    const __amdgpu_buffer_rsrc_t rp = lg_buffer_rsrc(a.pacc + base * hd);
    auto fetch = [&](int t0_) {                               // tiles t0 .. t0+63 of this row (past the end: the last one again)
        const int t0 = __builtin_amdgcn_readfirstlane(t0_);
        #pragma unroll
        for (int u = 0; u < U; ++u) {
            const int n = t0 + u < nt ? t0 + u : nt - 1;
            pa[u] = __int_as_float(__builtin_amdgcn_raw_buffer_load_b32(rp, d * 4, n * hd * 4, 0));
        }
    };
    fetch(wave * U);                                          // the partials do not depend on the weights
    float mx = -INFINITY;
    for (int n = threadIdx.x; n < nt; n += LG_WG) mx = fmaxf(mx, a.pm[base + n]);
    mx = lg_max_n(mx, 64);
    if (lane == 0) wmx[wave] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(wmx[0], wmx[1]), fmaxf(wmx[2], wmx[3]));
    float L = 0.0f, o = 0.0f;
    for (int r0 = 0; r0 < nt; r0 += 4 * U) {
        if (r0 > 0) fetch(r0 + wave * U);
        {   // the round's weights and sums (one tile per thread)
            const int n = r0 + (int)threadIdx.x;
            if (n < nt) { wts[threadIdx.x] = lg_expf(a.pm[base + n] - mx); pls[threadIdx.x] = a.pl[base + n]; }
        }
        __syncthreads();
        #pragma unroll
        for (int turn = 0; turn < 4; ++turn) {
            if (wave == turn && r0 + turn * U < nt) {
                if (r0 + turn > 0) { L = hand[0][lane]; o = hand[1][lane]; }
                #pragma unroll
                for (int u = 0; u < U; ++u) {
                    if (r0 + turn * U + u < nt) {             // (a guard, not a break: the partials stay in registers)
                        const float wn = wts[turn * U + u];
                        L = lg_fmaf(pls[turn * U + u], wn, L);
                        o = lg_fmaf(pa[u], wn, o);
                    }
                }
                hand[0][lane] = L; hand[1][lane] = o;
            }
            __syncthreads();
        }
    }
    if (wave != 0) return;
    L = hand[0][lane]; o = hand[1][lane];
    const float r = o / L;
    float dq; int sum;
    const int q = lg_quant1_32lanes(r, &dq, &sum);
    const int e = head * hd + d;
    a.xq[lg_q8_off<M>(qd, j, e >> 4, e & 15)] = (int8_t)q;
    if ((d & 31) == 0) lg_q8_ds<M>(a.xq, qd)[lg_q8_ds_idx<M>(qd, j, e >> 5)] = make_float2(dq, __int_as_float(sum));
    if (a.xf) a.xf[(size_t)j * qd + e] = r;
}

// ---------------------------------------------------------------------------------------------
// Attention merge + output projection in one launch, with no hand-over between workgroups.
// With 8 query heads the 8 K segments of the output projection ARE the heads (K = n_head * head_dim, a segment =
// head_dim elements): the serial chain of segment c only reads head c of the attention output, and the row's result is
// the adjacent-pair tree over the 8 chains.  So the workgroup that merges (head, row j) can run that head's chain
// for a slice of the E output rows straight from LDS, and slab `head` of 8 receives the chain sums: the consumer (the
// row kernel, dparts = 8) adds the slabs in the tree's order, bit for bit what lg_k_mm computes from the q8 row.
// Unit = (row j, head, slice s of the output rows in chunks of 64); the merge is repeated by the slices of a (head, row),
// which costs less than the kernel boundary it replaces.  Workgroup id = j * (8 * slices) + head * slices + s: the units
// that read the same weights differ by a multiple of 8 and run on one XCD (one trip from HBM, the others hit its L2).
// Weights: the projection tiled by row blocks (tile (64-row chunk, K block): lane r = row 64 * chunk + r), where the
// tiles of a head are consecutive.  Lane r of wavefront w runs the chains of the rows r of the unit's chunks w, w + 4, ...
// NIT = head_dim / 32 blocks per chain; RPL = most chunks per wavefront.
struct MergeOArgs {
    MergeArgs      g;           // g.xq unused; g.xf optional
    const uint8_t *w;           // row-block tiles of attn_output [E][n_head * head_dim]
    float         *slabs;       // [8][M][E]
    int            E, slices, rows;
};
#define LG_MERGEO_FIELDS(X, v) X(const float *, pm, g.pm, v) X(const float *, pl, g.pl, v) X(const float *, pacc, g.pacc, v) X(int, tiles_max, g.tiles_max, v) \
    X(int, H, g.H, v) X(int, hd, g.hd, v) X(int, window, g.window, v) X(int, pos_off, g.pos_off, v) X(const uint8_t *, w, w, v) X(int, E, E, v) X(int, slices, slices, v) \
    X(int, rows, rows, v) X(float *, slabs, slabs, v) X(float *, xf, g.xf, v)
template <int NIT, int RPL>
__global__ __launch_bounds__(LG_WG) void lg_k_merge_o(const StepCtl *ctl, LG_MERGEO_FIELDS(LG_XP, _) int p_end_) {
    MergeOArgs a; LG_MERGEO_FIELDS(LG_XI, a)
    a.g.xq = nullptr;
    __shared__ float wts[512], pls[512], wmx[LG_WG / 64];
    __shared__ __align__(16) int8_t hq[NIT * 32];             // the merged head as q8, natural order
    __shared__ float2 hds[NIT];
    const int W = a.g.H * a.slices, id = blockIdx.x;
    const int j = id / W, wi = id - j * W, head = wi / a.slices, s = wi - head * a.slices;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nb = a.g.H * NIT, n64 = (a.E >> 6) / a.slices, chunk0 = s * n64;
    uint4 wq[RPL][NIT];
    uint16_t wsc[RPL][NIT];
    const int qd = a.g.H * a.g.hd;
    lg_attn_merge_body(ctl, a.g, head, j, (int)threadIdx.x, wts, pls, wmx, [&] {
        #pragma unroll
        for (int r = 0; r < RPL; ++r) {
            const int c = wave + 4 * r < n64 ? wave + 4 * r : n64 - 1;     // past the unit's chunks: its last one again, unused
            const uint8_t *tb = a.w + ((size_t)(chunk0 + c) * nb + (size_t)head * NIT) * LG_TILE;
            #pragma unroll
            for (int it = 0; it < NIT; ++it) { wq[r][it] = lg_ldt16(tb, it, lane); wsc[r][it] = lg_ldt2(tb, it, lane); }
        }
    }, [&](int d, float r, int q, float dq, int sum) {
        hq[d] = (int8_t)q;
        if ((d & 31) == 0) hds[d >> 5] = make_float2(dq, __int_as_float(sum));
        if (a.g.xf && s == 0) a.g.xf[(size_t)j * qd + head * a.g.hd + d] = r;
    });
    __syncthreads();
    #pragma unroll
    for (int r = 0; r < RPL; ++r) {
        if (wave + 4 * r >= n64) break;
        float acc = 0.0f;
        #pragma unroll
        for (int it = 0; it < NIT; ++it) {
            const float2 ds = hds[it];
            const int4 a0 = *(const int4 *)(hq + it * 32), a1 = *(const int4 *)(hq + it * 32 + 16);
            const int dot = lg_block_dot(wq[r][it], a0, a1, __float_as_int(ds.y));
            acc = lg_fmaf(ds.x * lg_h2f(wsc[r][it]), (float)dot, acc);
        }
        a.slabs[((size_t)head * a.rows + j) * a.E + (size_t)(chunk0 + wave + 4 * r) * 64 + lane] = acc;
    }
}
