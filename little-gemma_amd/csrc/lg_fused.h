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
template <int M, int NV, int NW>
__global__ __launch_bounds__(LG_WG) void lg_k_rows_mm(RowsMmArgs a) {
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
__global__ __launch_bounds__(128 * KP) void lg_k_mm_ks(MmArgs a) {
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
    uint4 wq[TMAX]; uint32_t ws[TMAX];
    #pragma unroll
    for (int u = 0; u < TMAX; ++u) {
        const int it = it_lo + u < nit ? it_lo + u : nit - 1;
        wq[u] = *(const uint4 *)(wg + (size_t)it * LG_TILE + lane * 16);
        ws[u] = *(const uint16_t *)(wg + (size_t)it * LG_TILE + 1024 + lane * 2);
    }
    lg_load_q8<M>(a.q_in, k, lq);
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
