// lg_xtail.h — the narrow end of a layer as ONE launch that runs on ONE XCD (verify blocks, models with per-layer inputs).
//
// After ffn_down a layer with per-layer inputs still has three dependent steps, each of them a handful of workgroups
// and a kernel of its own when launched separately:
//   1  rows + PLE gate   x += rmsnorm(ffn_down) * w ; q8(x) ; gelu(inp_gate . q8(x)) * per-layer input ; q8    (ple/32 x M workgroups)
//   2  PLE projection    proj . that q8 row: [E] outputs of K = ple                                              (E x ple weights: 0.37 MB)
//   3  rows              x = (x + rmsnorm(2) * w) * out_scale ; q8(rmsnorm(x) * next norm weight)               (M rows)
// None of them can use the chip: what they cost is a kernel boundary each (the gap to the predecessor's end plus the
// first trip of the predecessor's data through the memory-side cache).  The workgroups of one XCD share an L2, and a
// hand-over through it costs a fraction of a boundary (lg_xcd.h).  So the three run as the phases of one kernel on the
// U = ple/32 x M workgroups i of the launch with i % 8 == 0 (the dispatcher deals workgroups to the XCDs in turn: one
// XCD gets them all; the other 7U workgroups of the launch leave at once):
//   phase 1 is lg_k_rows_plegate's body for unit (gate block, row); the unit keeps the updated residual row in registers;
//   hand-over (the M x ple q8 values: 1.6 KB) ;
//   phase 2: the E/8 row groups of the projection dealt over the 4U wavefronts, weights requested at kernel start
//   (they depend on nothing and are in registers long before the hand-over);
//   hand-over (the [M][E] f32 outputs) ;
//   phase 3: lg_k_rows' work for row j, by the units (v, j) of the row's first E/1024 gate blocks: each forms the row's
//   sums and stores and quantizes the float4s t + 256 v of every lane (the slices of lg_k_rows).
// Sums and quantization are the ones of the separate kernels, lane for lane: the results are bit-identical.
// The flags carry the writer's XCD id; a unit that sees another id, or gives up a bounded wait, reports it in
// StepCtl.err and goes on, so the kernel always ends and the host refuses the step.
#pragma once
#include "lg_kernels.h"
#include "lg_xcd.h"
#include "lg_xffn.h"

#define LG_XTAIL_UNITS 64           // most units of a launch (lane i of a wavefront polls flag i)
struct XtailSync {
    uint32_t gen;                   // launches so far (advanced by unit 0 at the end of a launch); epochs 2 gen + 1, + 2
    uint32_t pad[31];
    uint32_t flags[2][LG_XTAIL_UNITS];
};

struct XtailArgs {
    RowsPleGateArgs r;              // phase 1 (x_out is not written: the row stays in registers)
    const uint8_t *pw;              // phase 2: tiled projection weights [E][ple]
    float         *pout;            // [M][E] its output (the XCD's L2 hands it from phase 2 to phase 3)
    const float   *w_post2, *os;    // phase 3: norm weight for pout, layer output scale (or nullptr)
    const float   *w_pre;           // norm weight applied before quantization
    float         *x_out, *h_out;   // [M][E] new residual; normed rows before quantization, or nullptr
    int8_t        *q;               // q8 activation buffer of the result
    int            q_units;         // 0: rows in the order of lg_act_layout; 2: the 80-dword blocks of lg_k_geglu_m
    XtailSync     *sync;
    int            spin_limit;
    unsigned long long *stamps;     // nullptr, or [LG_XTAIL_UNITS][8] device wall-clock ticks at the phase boundaries of every unit (measurement runs)
    float         *gf;              // lg_k_ple_tail_s: [M][ple] the gated values as floats (handed from phase 1 to phase 2 through the XCD's L2)
};
#define LG_XTAIL_FIELDS(X, v) X(const float *, x, r.x, v) X(const float *, dout, r.dout, v) X(const float *, w_post, r.w_post, v) X(const uint8_t *, gw, r.g.w, v) \
    X(int, gk, r.g.k, v) X(int, gple, r.g.ple, v) X(int, dparts, r.dparts, v) X(XtailSync *, sync, sync, v) X(const float *, gipl, r.g.ipl, v) X(int, glayer, r.g.layer, v) \
    X(int, gnl, r.g.n_layer, v) X(int8_t *, gpq, r.g.pq, v) X(const uint8_t *, pw, pw, v) X(const float *, w_post2, w_post2, v) X(const float *, w_pre, w_pre, v) \
    X(const float *, os, os, v) X(float *, pout, pout, v) X(float *, x_out, x_out, v) X(float *, h_out, h_out, v) X(int8_t *, q, q, v) X(int, q_units, q_units, v) \
    X(float, eps, r.eps, v) X(int, spin_limit, spin_limit, v) X(unsigned long long *, stamps, stamps, v) X(float *, gf, gf, v)

__device__ __forceinline__ void lg_ld4_wait1(lg_x4u &a) { asm volatile("s_waitcnt vmcnt(0)" : "+v"(a) :: "memory"); }

// G: most projection row groups per wavefront (E/8 groups over 4U wavefronts).
template <int M, int G>
__global__ __launch_bounds__(LG_WG) void lg_k_ple_tail(StepCtl *ctl, LG_XTAIL_FIELDS(LG_XP, _) int p_end_) {
    if (blockIdx.x & (LG_XCDS - 1)) return;
    XtailArgs a; LG_XTAIL_FIELDS(LG_XI, a)
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float gbuf[32], red[3][4];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int E = a.r.g.k, ple = a.r.g.ple, nblk = ple >> 5, U = nblk * M, nq = E >> 2;
    const int u = blockIdx.x >> 3, gb = u % nblk, j = u / nblk;
    const uint32_t gen = a.sync->gen;
    auto stamp = [&](int i) { if (a.stamps && t == 0) a.stamps[(size_t)u * 8 + i] = wall_clock64(); };
    stamp(0);
    const int xcc = lg_xcc_id();
    // ---- phase 1, with this kernel's later loads requested behind its own ----
    const int groups = E >> 3, waves = 4 * U, gw = u * 4 + wave;
    const uint8_t *wgp[G];
    int row[G];
    bool live[G];
    #pragma unroll
    for (int g = 0; g < G; ++g) {
        const int gi = gw + g * waves;
        live[g] = gi < groups;
        const int gc = live[g] ? gi : groups - 1;
        wgp[g] = a.pw + (size_t)gc * LG_TILE;                  // K = ple = 256: one tile per group of 8 rows
        row[g] = gc * 8 + (lane >> 3);
    }
    WChunk<G, 1> pwt;
    float4 wpost2[LG_ROWV], wpre[LG_ROWV];
    float osv = 1.0f;
    float4 xv[LG_ROWV];
    lg_rows_plegate_body<M>(a.r, gb, j, smem, gbuf, red[0], xv, false, [&] {
        lg_mm_fetch<G, 1>(pwt, wgp, 0, 1, lane);
        const float4 *w2 = (const float4 *)a.w_post2, *w3 = (const float4 *)a.w_pre;
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) { wpost2[v] = w2[t + 256 * v]; wpre[v] = w3[t + 256 * v]; }
        if (a.os) osv = a.os[0];
    });
    stamp(1);
    // ---- hand-over: every unit's 32 gated values of its row are in the XCD's L2 ----
    int8_t *lq2 = (int8_t *)(smem + (size_t)E * 5 / 4);       // [M][ple] int8, [M][ple/32] {scale, sum}
    lg_wait_vm();
    __syncthreads();
    if (wave == 0) {
        const int err = lg_xcd_arrive_wait(a.sync->flags[0], u, true, U, 2 * gen + 1, xcc, a.spin_limit);
        if (err && lane == 0) atomicOr(&ctl->err, err);
    }
    __syncthreads();
    stamp(2);
    {
        const int n16 = M * ple * 5 / 64;                      // 16-byte units of the q8 rows
        for (int i = t; i < n16; i += LG_WG) {
            lg_x4u v = lg_ld4_sc_issue<2>(a.r.g.pq + (size_t)i * 16);
            lg_ld4_wait1(v);
            *(lg_x4u *)(lq2 + (size_t)i * 16) = v;
        }
    }
    __syncthreads();
    stamp(3);
    // ---- phase 2: this wavefront's row groups of the projection ----
    {
        float acc[G][M];
        lg_mm_groups<M, 8, G, false, 1>(wgp, pwt, 1, lq2, lg_q8_ds<M>(lq2, ple), ple, acc, lane, nullptr, E, row);
        const int c = lane & 7;
        if (c < M) {
            #pragma unroll
            for (int g = 0; g < G; ++g) if (live[g]) a.pout[(size_t)c * E + row[g]] = lg_pick<M>(acc[g], c);
        }
    }
    // ---- hand-over: the projection's [M][E] is in the XCD's L2 ----
    const int slices = (E + 1023) >> 10;
    stamp(4);
    lg_wait_vm();
    __syncthreads();
    if (gb >= slices) {                                        // this unit has no share of the row work: it arrives and leaves
        if (t == 0) lg_st_sc<0>(a.sync->flags[1] + u, ((2 * gen + 2) << 4) | (uint32_t)xcc);
        return;
    }
    if (wave == 0) {
        const int err = lg_xcd_arrive_wait(a.sync->flags[1], u, true, U, 2 * gen + 2, xcc, a.spin_limit);
        if (err && lane == 0) atomicOr(&ctl->err, err);
    }
    __syncthreads();
    stamp(5);
    // ---- phase 3: the row work of row j, this unit storing and quantizing slice gb ----
    float4 dv[LG_ROWV];
    {
        lg_x4u d0 = lg_x4u{ 0, 0, 0, 0 }, d1 = d0, d2 = d0, d3 = d0;
        const float *pr = a.pout + (size_t)j * E;
        const int last = nq - 1;
        d0 = lg_ld4_sc_issue<2>(pr + 4 * min(t, last));
        d1 = lg_ld4_sc_issue<2>(pr + 4 * min(t + 256, last));
        d2 = lg_ld4_sc_issue<2>(pr + 4 * min(t + 512, last));
        d3 = lg_ld4_sc_issue<2>(pr + 4 * min(t + 768, last));
        lg_ld4_wait(d0, d1, d2, d3);
        const lg_x4u d[4] = { d0, d1, d2, d3 };
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) dv[v] = make_float4(__uint_as_float(d[v].x), __uint_as_float(d[v].y), __uint_as_float(d[v].z), __uint_as_float(d[v].w));
    }
    stamp(6);
    {
        float ss = 0.0f;
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) ss = lg_sumsq4(dv[v], ss);
        ss = lg_block_sum256(ss, red[1]);
        const float sc = 1.0f / sqrtf(ss / (float)E + a.r.eps);
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) {
            const float4 w = wpost2[v];
            float4 r;
            r.x = xv[v].x + dv[v].x * sc * w.x;  r.y = xv[v].y + dv[v].y * sc * w.y;
            r.z = xv[v].z + dv[v].z * sc * w.z;  r.w = xv[v].w + dv[v].w * sc * w.w;
            if (a.os) { r.x = r.x * osv; r.y = r.y * osv; r.z = r.z * osv; r.w = r.w * osv; }
            xv[v] = r;
        }
    }
    {
        float4 *xo = (float4 *)(a.x_out + (size_t)j * E);
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq && v == gb) xo[t + 256 * v] = xv[v];
    }
    {
        float ss = 0.0f;
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) ss = lg_sumsq4(xv[v], ss);
        ss = lg_block_sum256(ss, red[2]);
        const float sc = 1.0f / sqrtf(ss / (float)E + a.r.eps);
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) {
            const float4 w = wpre[v];
            xv[v] = make_float4(xv[v].x * sc * w.x, xv[v].y * sc * w.y, xv[v].z * sc * w.z, xv[v].w * sc * w.w);
        }
    }
    if (a.h_out) {
        float4 *ho = (float4 *)(a.h_out + (size_t)j * E);
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq && v == gb) ho[t + 256 * v] = xv[v];
    }
    float2 *dsb = lg_q8_ds<M>(a.q, E);
    #pragma unroll
    for (int v = 0; v < LG_ROWV; ++v) {
        if (t + 256 * v >= nq || v != gb) continue;
        float d; int sum;
        const uint32_t packed = lg_quant4_8lanes(xv[v], &d, &sum);
        const int quad = t + 256 * v;
        if (a.q_units == 2) {
            uint32_t *blk = (uint32_t *)a.q + (size_t)(quad >> 3) * LG_MU_DWORDS;
            const int dw = quad & 7;
            blk[j * 8 + ((dw & 1) | ((dw & 2) << 1) | ((dw & 4) >> 1))] = packed;
            if ((t & 7) == 0) *(float2 *)(blk + 64 + 2 * j) = make_float2(d, 12582912.0f + (float)(8 * sum));
        } else {
            *(uint32_t *)(a.q + lg_q8_off<M>(E, j, quad >> 2, (quad & 3) * 4)) = packed;
            if ((t & 7) == 0) dsb[lg_q8_ds_idx<M>(E, j, quad >> 3)] = make_float2(d, __int_as_float(sum));
        }
    }
    stamp(7);
    if (u == 0 && t == 0) a.sync->gen = gen + 1;
}

// the sum over the 256 lanes of wavefronts 0..3 (order of lg_block_sum256) in a workgroup of 8 wavefronts that all call it
__device__ __forceinline__ float lg_block_sum256_of512(float v, float *scratch8) {
    v = lg_wave_sum64(v);
    if ((threadIdx.x & 63) == 0) scratch8[threadIdx.x >> 6] = v;
    __syncthreads();
    return (scratch8[0] + scratch8[1]) + (scratch8[2] + scratch8[3]);
}

// The same tail for blocks of 5..8 rows, where ple/32 x M units no longer fit one per CU of the XCD (at 5 rows 8 CUs held
// two units, pulled twice the bytes through their one memory path and kept every other unit waiting at the first
// hand-over).  Here the launch has W = M * P units, P = 32 / M per row (30, 30, 28, 32 units at 5..8 rows), each a workgroup
// of 8 wavefronts.  Unit (row j, part p):
//   phase 1: wavefronts 0..3 do the row's update and q8 exactly as lg_k_rows_plegate does (every part of a row repeats
//   it), then wavefront w runs gate row group g0 + w (8 gate rows) of the part's share g0 .. g0 + cnt - 1 of the ple/8
//   groups (cnt = 5 or 6 at 5 rows, 8 at 8 rows); the gated values go out as floats: a part's rows do not line up
//   with the q8 blocks of 32;
//   hand-over; every unit quantizes the M x ple floats into its LDS (the blocks, scales and sums of lg_k_rows_plegate);
//   phase 2 and 3 as in lg_k_ple_tail, the projection's row groups dealt over 8 W wavefronts, the row work of row j by
//   its parts 0 .. E/1024 - 1 (wavefronts 0..3).
template <int M, int G>
__global__ __launch_bounds__(512) void lg_k_ple_tail_s(StepCtl *ctl, LG_XTAIL_FIELDS(LG_XP, _) int p_end_) {
    if (blockIdx.x & (LG_XCDS - 1)) return;
    XtailArgs a; LG_XTAIL_FIELDS(LG_XI, a)
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float red[3][8];
    constexpr int P = 32 / M;
    const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const bool rowt = t < 256;                                 // the threads of the row work (lane order of lg_k_rows)
    const int E = a.r.g.k, ple = a.r.g.ple, W = M * P, nq = E >> 2, nit = E >> 8;
    const int u = blockIdx.x >> 3, j = u / P, p = u - j * P;
    const int ngr = ple >> 3, gbase = ngr / P, gextra = ngr - gbase * P;
    const int cnt = gbase + (p < gextra ? 1 : 0), g0 = p * gbase + (p < gextra ? p : gextra);
    const bool gatew = wave < cnt;
    const int gg = g0 + (gatew ? wave : 0);                    // this wavefront's gate row group
    const uint32_t gen = a.sync->gen;
    auto stamp = [&](int i) { if (a.stamps && t == 0) a.stamps[(size_t)u * 8 + i] = wall_clock64(); };
    stamp(0);
    const int xcc = lg_xcc_id();
    int8_t *lq = (int8_t *)smem;                               // the row: [E] int8, then [E/32] {scale, sum}
    float2 *lds = (float2 *)(smem + (size_t)E);
    int8_t *lq2 = (int8_t *)(smem + (size_t)E * 5 / 4);        // [M][ple] int8, [M][ple/32] {scale, sum}
    // ---- every load of phase 1 up front, the row's first; then what the later phases need ----
    float4 xv[LG_ROWV], dv[LG_ROWV], wp[LG_ROWV];
    if (rowt) {
        const float4 *wr = (const float4 *)a.r.w_post, *xr = (const float4 *)(a.r.x + (size_t)j * E), *dr = (const float4 *)(a.r.dout + (size_t)j * E);
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) { xv[v] = xr[t + 256 * v]; dv[v] = dr[t + 256 * v]; wp[v] = wr[t + 256 * v]; }
        if (a.r.dparts == 4) {                                 // the top two levels of the tree of an ffn_down cut by K quarter
            const size_t slab = (size_t)M * nq;
            #pragma unroll
            for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) {
                const float4 p1 = dr[slab + t + 256 * v], p2 = dr[2 * slab + t + 256 * v], p3 = dr[3 * slab + t + 256 * v], p0 = dv[v];
                dv[v] = make_float4((p0.x + p1.x) + (p2.x + p3.x), (p0.y + p1.y) + (p2.y + p3.y),
                                    (p0.z + p1.z) + (p2.z + p3.z), (p0.w + p1.w) + (p2.w + p3.w));
            }
        }
        if (a.r.dparts == 8) {                                 // the top three levels of the K-segment tree of an ffn_down cut over the 8 XCDs
            const size_t slab = (size_t)M * nq;
            #pragma unroll
            for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) {
                const float4 *b = dr + t + 256 * v;
                const float4 p1 = b[slab], p2 = b[2 * slab], p3 = b[3 * slab], p4 = b[4 * slab], p5 = b[5 * slab], p6 = b[6 * slab], p7 = b[7 * slab], p0 = dv[v];
                dv[v] = make_float4(((p0.x + p1.x) + (p2.x + p3.x)) + ((p4.x + p5.x) + (p6.x + p7.x)), ((p0.y + p1.y) + (p2.y + p3.y)) + ((p4.y + p5.y) + (p6.y + p7.y)),
                                    ((p0.z + p1.z) + (p2.z + p3.z)) + ((p4.z + p5.z) + (p6.z + p7.z)), ((p0.w + p1.w) + (p2.w + p3.w)) + ((p4.w + p5.w) + (p6.w + p7.w)));
            }
        }
    }
    uint4 wq[LG_MAXV]; uint32_t wsc[LG_MAXV];
    {
        const uint8_t *wg0 = a.r.g.w + (size_t)gg * nit * LG_TILE;
        #pragma unroll
        for (int k = 0; k < LG_MAXV; ++k) {
            const int it = k < nit ? k : nit - 1;
            wq[k] = *(const uint4 *)(wg0 + (size_t)it * LG_TILE + lane * 16);
            wsc[k] = *(const uint16_t *)(wg0 + (size_t)it * LG_TILE + 1024 + lane * 2);
        }
    }
    const float iplv = a.r.g.ipl[(size_t)j * a.r.g.n_layer * ple + (size_t)a.r.g.layer * ple + gg * 8 + (lane >> 3)];   // of this lane's gate column
    const int groups = E >> 3, waves = 8 * W, gw = u * 8 + wave;
    const uint8_t *wgp[G];
    int row[G];
    bool live[G];
    #pragma unroll
    for (int g = 0; g < G; ++g) {
        const int gi = gw + g * waves;
        live[g] = gi < groups;
        const int gc = live[g] ? gi : groups - 1;
        wgp[g] = a.pw + (size_t)gc * LG_TILE;                  // K = ple = 256: one tile per group of 8 rows
        row[g] = gc * 8 + (lane >> 3);
    }
    WChunk<G, 1> pwt;
    lg_mm_fetch<G, 1>(pwt, wgp, 0, 1, lane);
    float4 wpost2[LG_ROWV], wpre[LG_ROWV];
    float osv = 1.0f;
    if (rowt) {
        const float4 *w2 = (const float4 *)a.w_post2, *w3 = (const float4 *)a.w_pre;
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) { wpost2[v] = w2[t + 256 * v]; wpre[v] = w3[t + 256 * v]; }
        if (a.os) osv = a.os[0];
    }
    // ---- phase 1: the row, then this wavefront's gate rows ----
    {
        float ss = 0.0f;
        if (rowt) {
            #pragma unroll
            for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) ss = lg_sumsq4(dv[v], ss);
        }
        ss = lg_block_sum256_of512(ss, red[0]);
        const float sc = 1.0f / sqrtf(ss / (float)E + a.r.eps);
        if (rowt) {
            #pragma unroll
            for (int v = 0; v < LG_ROWV; ++v) {
                if (t + 256 * v < nq) {                        // nq is a multiple of 64: whole wavefronts
                    const float4 w = wp[v], d = dv[v];
                    float4 x = xv[v];
                    x.x = x.x + d.x * sc * w.x;  x.y = x.y + d.y * sc * w.y;
                    x.z = x.z + d.z * sc * w.z;  x.w = x.w + d.w * sc * w.w;
                    xv[v] = x;
                    float dq; int sum;
                    const uint32_t packed = lg_quant4_8lanes(x, &dq, &sum);
                    const int quad = t + 256 * v;
                    *(uint32_t *)(lq + lg_q8_off<1>(E, 0, quad >> 2, (quad & 3) * 4)) = packed;
                    if ((t & 7) == 0) lds[lg_q8_ds_idx<1>(E, 0, quad >> 3)] = make_float2(dq, __int_as_float(sum));
                }
            }
        }
    }
    __syncthreads();
    if (gatew) {
        const int c = lane & 7;
        float pr = 0.0f;
        #pragma unroll
        for (int k = 0; k < LG_MAXV; ++k) {
            if (k < nit) {                                     // (a guard, not a break: the arrays stay in registers)
                const float2 ds = lds[k * 8 + c];
                const int8_t *au = lq + (size_t)(k * 16 + c) * 16;
                const int dot = lg_block_dot(wq[k], *(const int4 *)au, *(const int4 *)(au + 8 * 16), __float_as_int(ds.y));
                pr = lg_fmaf(ds.x * lg_h2f((uint16_t)wsc[k]), (float)dot, pr);
            }
        }
        pr = lg_sum_seg<8>(pr);
        if (c == 0) a.gf[(size_t)j * ple + gg * 8 + (lane >> 3)] = lg_gelu(pr) * iplv;
    }
    stamp(1);
    // ---- hand-over: every part's gated values of its row are in the XCD's L2 ----
    lg_wait_vm();
    __syncthreads();
    if (wave == 0) {
        const int err = lg_xcd_arrive_wait(a.sync->flags[0], u, true, W, 2 * gen + 1, xcc, a.spin_limit);
        if (err && lane == 0) atomicOr(&ctl->err, err);
    }
    __syncthreads();
    stamp(2);
    if (wave < M) {                                            // wavefront r = row r: a float4 per lane, 8 lanes a block of 32
        constexpr int PLE = 256;                               // (the launch is made for ple == 256 only: constant layout arithmetic)
        lg_x4u v = lg_ld4_sc_issue<2>(a.gf + 4 * t);
        lg_ld4_wait1(v);
        const int r = wave, blk = lane >> 3, l8 = lane & 7;
        float d; int sum;
        const uint32_t packed = lg_quant4_8lanes(make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w)), &d, &sum);
        const ActLayout lay = lg_act_layout(PLE);
        *(uint32_t *)(lq2 + (size_t)r * PLE + lg_act_unit(lay, blk * 2 + (l8 >> 2)) * 16 + (l8 & 3) * 4) = packed;
        if (l8 == 0) lg_q8_ds<M>(lq2, PLE)[(size_t)r * (PLE >> 5) + lg_act_block(lay, blk)] = make_float2(d, __int_as_float(sum));
    }
    __syncthreads();
    stamp(3);
    // ---- phase 2: this wavefront's row groups of the projection ----
    {
        float acc[G][M];
        lg_mm_groups<M, 8, G, false, 1>(wgp, pwt, 1, lq2, lg_q8_ds<M>(lq2, ple), ple, acc, lane, nullptr, E, row);
        const int c = lane & 7;
        if (c < M) {
            #pragma unroll
            for (int g = 0; g < G; ++g) if (live[g]) a.pout[(size_t)c * E + row[g]] = lg_pick<M>(acc[g], c);
        }
    }
    // ---- hand-over: the projection's [M][E] is in the XCD's L2 ----
    const int slices = (E + 1023) >> 10;
    stamp(4);
    lg_wait_vm();
    __syncthreads();
    if (p >= slices) {                                         // this unit has no share of the row work: it arrives and leaves
        if (t == 0) lg_st_sc<0>(a.sync->flags[1] + u, ((2 * gen + 2) << 4) | (uint32_t)xcc);
        return;
    }
    if (wave == 0) {
        const int err = lg_xcd_arrive_wait(a.sync->flags[1], u, true, W, 2 * gen + 2, xcc, a.spin_limit);
        if (err && lane == 0) atomicOr(&ctl->err, err);
    }
    __syncthreads();
    stamp(5);
    // ---- phase 3: the row work of row j, this unit storing and quantizing slice p (wavefronts 0..3; the others only
    //      take part in the workgroup's barriers) ----
    if (rowt) {
        lg_x4u d0 = lg_x4u{ 0, 0, 0, 0 }, d1 = d0, d2 = d0, d3 = d0;
        const float *pr = a.pout + (size_t)j * E;
        const int last = nq - 1;
        d0 = lg_ld4_sc_issue<2>(pr + 4 * min(t, last));
        d1 = lg_ld4_sc_issue<2>(pr + 4 * min(t + 256, last));
        d2 = lg_ld4_sc_issue<2>(pr + 4 * min(t + 512, last));
        d3 = lg_ld4_sc_issue<2>(pr + 4 * min(t + 768, last));
        lg_ld4_wait(d0, d1, d2, d3);
        const lg_x4u d[4] = { d0, d1, d2, d3 };
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) dv[v] = make_float4(__uint_as_float(d[v].x), __uint_as_float(d[v].y), __uint_as_float(d[v].z), __uint_as_float(d[v].w));
    }
    stamp(6);
    {
        float ss = 0.0f;
        if (rowt) {
            #pragma unroll
            for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) ss = lg_sumsq4(dv[v], ss);
        }
        ss = lg_block_sum256_of512(ss, red[1]);
        const float sc = 1.0f / sqrtf(ss / (float)E + a.r.eps);
        if (rowt) {
            #pragma unroll
            for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) {
                const float4 w = wpost2[v];
                float4 r;
                r.x = xv[v].x + dv[v].x * sc * w.x;  r.y = xv[v].y + dv[v].y * sc * w.y;
                r.z = xv[v].z + dv[v].z * sc * w.z;  r.w = xv[v].w + dv[v].w * sc * w.w;
                if (a.os) { r.x = r.x * osv; r.y = r.y * osv; r.z = r.z * osv; r.w = r.w * osv; }
                xv[v] = r;
            }
        }
    }
    if (rowt) {
        float4 *xo = (float4 *)(a.x_out + (size_t)j * E);
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq && v == p) xo[t + 256 * v] = xv[v];
    }
    {
        float ss = 0.0f;
        if (rowt) {
            #pragma unroll
            for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) ss = lg_sumsq4(xv[v], ss);
        }
        ss = lg_block_sum256_of512(ss, red[2]);
        const float sc = 1.0f / sqrtf(ss / (float)E + a.r.eps);
        if (rowt) {
            #pragma unroll
            for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) {
                const float4 w = wpre[v];
                xv[v] = make_float4(xv[v].x * sc * w.x, xv[v].y * sc * w.y, xv[v].z * sc * w.z, xv[v].w * sc * w.w);
            }
        }
    }
    if (rowt) {
        if (a.h_out) {
            float4 *ho = (float4 *)(a.h_out + (size_t)j * E);
            #pragma unroll
            for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq && v == p) ho[t + 256 * v] = xv[v];
        }
        float2 *dsb = lg_q8_ds<M>(a.q, E);
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) {
            if (t + 256 * v >= nq || v != p) continue;
            float d; int sum;
            const uint32_t packed = lg_quant4_8lanes(xv[v], &d, &sum);
            const int quad = t + 256 * v;
            if (a.q_units == 2) {
                uint32_t *blk = (uint32_t *)a.q + (size_t)(quad >> 3) * LG_MU_DWORDS;
                const int dw = quad & 7;
                blk[j * 8 + ((dw & 1) | ((dw & 2) << 1) | ((dw & 4) >> 1))] = packed;
                if ((t & 7) == 0) *(float2 *)(blk + 64 + 2 * j) = make_float2(d, 12582912.0f + (float)(8 * sum));
            } else {
                *(uint32_t *)(a.q + lg_q8_off<M>(E, j, quad >> 2, (quad & 3) * 4)) = packed;
                if ((t & 7) == 0) dsb[lg_q8_ds_idx<M>(E, j, quad >> 3)] = make_float2(d, __int_as_float(sum));
            }
        }
    }
    stamp(7);
    if (u == 0 && t == 0) a.sync->gen = gen + 1;
}

// A second form was built and measured, and is not kept: 32 units of 8 gate rows and 8 wavefronts whatever the block
// width (so that no CU holds two units from 5 rows up), the row update as a phase of its own ahead of the gate (units
// (slice, row), q8 rows handed over), the gated rows handed over as floats and quantized by every unit.  Bit-identical,
// three hand-overs instead of two, and slower at every width: E4B shape, 5 rows 11.2 against 10.6 us per launch (step
// 2.231 against 2.210 ms), 6 rows 2.326 against 2.303 ms, 8 rows 2.494 against 2.477 ms.  A hand-over costs about 1 us
// once the wait for the stores and the load of what was handed over are counted, more than the lighter phases save.


// ---------------------------------------------------------------------------------------------------------
// Measured at the E4B shape (5 rows): 12.3 us per launch against 4.3 + 4.1 + 4.5 for the three kernels it replaces, and the
// step 2.219 against 2.203 ms: not a gain, so the option is off by default.  By the stamps: merges 4.3-4.8 us (the same chain of
// round trips as the separate kernel: the partials come from other XCDs), hand-over 0.45, copy of the merged rows 0.5, the
// projection 2.1 (bound by the vector instructions around the MFMA: 640 chains x 8 steps x ~20 instructions on one XCD's
// 128 SIMDs), hand-over 0.55, row work 1.7; the three separate kernels hide their launch gaps under each other's tails, the
// phases of one launch cannot.
// The narrow end of the attention half the same way: merge -> output projection -> row work, one launch on one XCD.
//   1  merge of the tile partials of every (head, row), two of them at a time per unit (a unit is 8 wavefronts, a merge
//      takes 4); the q8 of the merged head goes to the XCD's L2 in the matrix-core block order (80 dwords per block of 32:
//      8 row slots of 32 bytes, then 8 x {scale, 12582912 + 8 * sum});
//      hand-over;
//   2  the output projection on the matrix cores: a chain = (block of 32 output rows, K segment); wavefront w of unit u
//      runs segment w of the row blocks u, u + 32, ...: per block of the segment one v_mfma_i32_32x32x32_i8 (A = the
//      block's activations in 8 row slots, B = the 32 rows' nibbles) and four fma per lane, p = fma(xd * dw, (float)dot, p),
//      the chain of lg_k_mm; the 8 segment sums of a row meet in LDS in the adjacent-pair tree.  The weights (E x K / 32
//      units = 92 KB per unit at the E4B shape) are requested at kernel start and arrive under the merge: a lone XCD pulls
//      3 MB from HBM in about 2 us.  On v_dot4 the same projection would keep the XCD's 128 SIMDs busy for 4.5 us;
//      hand-over;
//   3  the row work ahead of gate/up (residual update, ffn norm, q8 in the order the gate/up kernel reads) by units (slice, row).
// Weights: per chain the stream layout of lg_xffn.h (pairs of blocks: [pair][half h][row n] 8 + 8 nibble bytes, then
// [pair][row n] the two f16 scales), chains ordered [row block][segment].
struct XattnTailArgs {
    MergeArgs      g;            // g.xq, g.xf unused
    const uint8_t *wo;           // chains of attn_output
    uint32_t      *aq;           // [K / 32][80] the merged rows as matrix-core blocks
    float         *pout;         // [M][E]
    const float   *x, *w_post, *w_pre;
    float         *x_out;
    int8_t        *q;
    int            q_units;      // 2: blocks of lg_k_geglu_m (4..8 rows), 1: units of lg_k_geglu_t (up to 3 rows)
    int            E;
    float          eps;
    XtailSync     *sync;
    int            spin_limit;
    unsigned long long *stamps;
};
#define LG_XATTN_FIELDS(X, v) X(const float *, pm, g.pm, v) X(const float *, pl, g.pl, v) X(const float *, pacc, g.pacc, v) X(int, tiles_max, g.tiles_max, v) \
    X(int, H, g.H, v) X(int, hd, g.hd, v) X(int, window, g.window, v) X(int, pos_off, g.pos_off, v) X(const uint8_t *, wo, wo, v) X(XtailSync *, sync, sync, v) \
    X(const float *, x, x, v) X(const float *, w_post, w_post, v) X(const float *, w_pre, w_pre, v) X(uint32_t *, aq, aq, v) X(float *, pout, pout, v) \
    X(float *, x_out, x_out, v) X(int8_t *, q, q, v) X(int, q_units, q_units, v) X(int, E, E, v) X(float, eps, eps, v) X(int, spin_limit, spin_limit, v) \
    X(unsigned long long *, stamps, stamps, v)

// Row blocks of a unit whose weights are requested with the merge's partials; the rest after the merge.  All of them early
// is the faster choice: requested after the merge they delay the first hand-over, whose store wait also waits for them
// (the merge phase 4.3-4.8 us either way, the whole launch 10.1 against 11.0 us).
#ifndef LG_XATTN_EARLY
#define LG_XATTN_EARLY 8
#endif
// M: rows; NP: pairs of blocks per chain (K / 32 / 8 / 2); RB: most row blocks per unit (E / 32 over 32 units).
template <int M, int NP, int RB>
__global__ __launch_bounds__(512) void lg_k_attn_tail(StepCtl *ctl, LG_XATTN_FIELDS(LG_XP, _) int p_end_) {
    if (blockIdx.x & (LG_XCDS - 1)) return;
    XattnTailArgs a; LG_XATTN_FIELDS(LG_XI, a)
    a.g.xq = nullptr; a.g.xf = nullptr;
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float wts[2][512], pls[2][512], wmx[2][4], red3[2][8];
    __shared__ __align__(16) int8_t hq[2][512];
    __shared__ float2 hds[2][16];
    const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6), half = wave >> 2, tid = t & 255;
    const int n = lane & 31, h = lane >> 5;
    const int E = a.E, nq = E >> 2, hd = a.g.hd, nbh = hd >> 5, nit = 2 * NP, nb = 8 * nit;
    const int U = LG_XCD_WGS, u = blockIdx.x >> 3;
    const int slices = (E + 1023) >> 10, nrow = slices * M;
    const bool rowunit = u < nrow, rowlane = t < LG_WG;
    const int v_ = u / M, jr = u - v_ * M;
    const uint32_t gen = a.sync->gen;
    const int xcc = lg_xcc_id();
    auto stamp = [&](int i) { if (a.stamps && t == 0) a.stamps[(size_t)u * 8 + i] = wall_clock64(); };
    stamp(0);
    lg_v16i magic;
    #pragma unroll
    for (int i = 0; i < 16; ++i) magic[i] = 0x4B400000;
    asm volatile("" : "+v"(magic));
    // ---- phase 1: the merges (tasks u and u + 32), with everything else this unit reads requested behind their partials ----
    const int ntasks = a.g.H * M, task = u + U * half;
    const bool on = task < ntasks;
    const int tk = on ? task : ntasks - 1, head = tk % a.g.H, j = tk / a.g.H;
    struct Pair { lg_x4u q; uint32_t sw; };
    Pair wq[RB][NP];
    bool live[RB];
    float4 xv[LG_ROWV], wpost[LG_ROWV], wpre[LG_ROWV];
    const int nrb = E >> 5;
    auto fetch_w = [&](int k0, int k1) {
        #pragma unroll
        for (int k = 0; k < RB; ++k) {
            if (k < k0 || k >= k1) continue;
            const int rb = u + U * k;
            live[k] = rb < nrb;
            const uint8_t *cb = a.wo + ((size_t)(live[k] ? rb : 0) * 8 + wave) * ((size_t)nit * 576);    // (no such row block: the first one's weights, never stored)
            #pragma unroll
            for (int jp = 0; jp < NP; ++jp) {
                wq[k][jp].q = __builtin_nontemporal_load((const lg_x4u *)(cb + (size_t)((jp * 2 + h) * 32 + n) * 16));
                wq[k][jp].sw = __builtin_nontemporal_load((const uint32_t *)(cb + (size_t)nit * 512 + (size_t)(jp * 32 + n) * 4));
            }
        }
    };
    lg_attn_merge_body<false>(ctl, a.g, head, j, tid, wts[half], pls[half], wmx[half], [&] { fetch_w(0, LG_XATTN_EARLY); }, [&](int d, float r, int q, float dq, int sum) {
        hq[half][d] = (int8_t)q;
        if ((d & 31) == 0) hds[half][d >> 5] = make_float2(dq, 12582912.0f + (float)(8 * sum));
    });
    fetch_w(LG_XATTN_EARLY, RB);
    __syncthreads();
    if (on && tid < (hd >> 2)) {                               // dword tid of the merged head: block tid / 8, dword tid % 8 of it
        const int b = tid >> 3, dw = tid & 7;
        uint32_t *blk = a.aq + (size_t)(head * nbh + b) * LG_MU_DWORDS;
        blk[j * 8 + ((dw & 1) | ((dw & 2) << 1) | ((dw & 4) >> 1))] = *(const uint32_t *)(hq[half] + 4 * tid);
        if (dw == 0) *(float2 *)(blk + 64 + 2 * j) = hds[half][b];
    }
    stamp(1);
    // ---- hand-over: the merged rows are in the XCD's L2 ----
    const int nmerge = ntasks < U ? ntasks : U;                 // units that ran a merge
    lg_wait_vm();
    __syncthreads();
    if (wave == 0) {
        const int err = lg_xcd_arrive_wait(a.sync->flags[0], u, u < nmerge, nmerge, 2 * gen + 1, xcc, a.spin_limit);
        if (err && lane == 0) atomicOr(&ctl->err, err);
    }
    __syncthreads();
    stamp(2);
    unsigned char *la = smem;                                  // [nb][320]
    float *red = (float *)(smem + (size_t)nb * LG_MU_DWORDS * 4);          // [8 segments][RB][8 row slots][32]
    {
        const int n16 = nb * LG_MU_DWORDS / 4;                 // 16-byte units
        for (int i0 = t; i0 < n16; i0 += 4 * 512) {
            const int i1 = min(i0 + 512, n16 - 1), i2 = min(i0 + 1024, n16 - 1), i3 = min(i0 + 1536, n16 - 1);
            lg_x4u v0 = lg_ld4_sc_issue<2>((const unsigned char *)a.aq + (size_t)i0 * 16), v1 = lg_ld4_sc_issue<2>((const unsigned char *)a.aq + (size_t)i1 * 16);
            lg_x4u v2 = lg_ld4_sc_issue<2>((const unsigned char *)a.aq + (size_t)i2 * 16), v3 = lg_ld4_sc_issue<2>((const unsigned char *)a.aq + (size_t)i3 * 16);
            lg_ld4_wait(v0, v1, v2, v3);
            *(lg_x4u *)(la + (size_t)i0 * 16) = v0; *(lg_x4u *)(la + (size_t)i1 * 16) = v1;
            *(lg_x4u *)(la + (size_t)i2 * 16) = v2; *(lg_x4u *)(la + (size_t)i3 * 16) = v3;
        }
    }
    __syncthreads();
    stamp(3);
    // (what phase 3 needs besides the projection is requested here: behind the loads this phase waits for, with a phase's
    // time to arrive, and not occupying registers during the merge)
    if (rowunit && rowlane) {
        const float4 *xr = (const float4 *)(a.x + (size_t)jr * E), *w1 = (const float4 *)a.w_post, *w2 = (const float4 *)a.w_pre;
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) { xv[v] = xr[t + 256 * v]; wpost[v] = w1[t + 256 * v]; wpre[v] = w2[t + 256 * v]; }
    }
    // ---- phase 2: segment `wave` of the unit's row blocks ----
    {
        const int arow = n < 8 ? n : 7;
        float p[RB][4];
        #pragma unroll
        for (int k = 0; k < RB; ++k)
            #pragma unroll
            for (int i = 0; i < 4; ++i) p[k][i] = 0.0f;
        #pragma unroll
        for (int jp = 0; jp < NP; ++jp) {
            #pragma unroll
            for (int e = 0; e < 2; ++e) {
                const XffnAct ac = lg_xffn_act(la + (size_t)(wave * nit + 2 * jp + e) * (LG_MU_DWORDS * 4), arow, h);
                #pragma unroll
                for (int k = 0; k < RB; ++k) {
                    lg_v2u q; q.x = e ? wq[k][jp].q.z : wq[k][jp].q.x; q.y = e ? wq[k][jp].q.w : wq[k][jp].q.y;
                    lg_xffn_step(ac.av, ac.xd, ac.cf, q, lg_h2f((uint16_t)(e ? wq[k][jp].sw >> 16 : wq[k][jp].sw)), magic, p[k]);
                }
            }
        }
        #pragma unroll
        for (int k = 0; k < RB; ++k)
            #pragma unroll
            for (int i = 0; i < 4; ++i) red[((size_t)(wave * RB + k) * 8 + 4 * h + i) * 32 + n] = p[k][i];      // (all 8 row slots: the tree reads the first M)
    }
    __syncthreads();
    for (int idx = t; idx < RB * M * 32; idx += 512) {         // the adjacent-pair tree over the 8 segments
        const int k = idx / (M * 32), rem = idx - k * (M * 32), jj = rem >> 5, nn = rem & 31, rb = u + U * k;
        if (rb < nrb) {
            const float *b = red + ((size_t)k * 8 + jj) * 32 + nn;
            const size_t sg = (size_t)RB * 8 * 32;
            a.pout[(size_t)jj * E + rb * 32 + nn] = ((b[0] + b[sg]) + (b[2 * sg] + b[3 * sg])) + ((b[4 * sg] + b[5 * sg]) + (b[6 * sg] + b[7 * sg]));
        }
    }
    stamp(4);
    // ---- hand-over: the projection's [M][E] is in the XCD's L2 ----
    lg_wait_vm();
    __syncthreads();
    if (!rowunit) {
        if (t == 0) lg_st_sc<0>(a.sync->flags[1] + u, ((2 * gen + 2) << 4) | (uint32_t)xcc);
        return;
    }
    if (wave == 0) {
        const int err = lg_xcd_arrive_wait(a.sync->flags[1], u, true, U, 2 * gen + 2, xcc, a.spin_limit);
        if (err && lane == 0) atomicOr(&ctl->err, err);
    }
    __syncthreads();
    stamp(5);
    // ---- phase 3: the row work of row jr, this unit storing and quantizing slice v_ ----
    float4 dv[LG_ROWV];
    if (rowlane) {
        lg_x4u d0, d1, d2, d3;
        const float *pr = a.pout + (size_t)jr * E;
        const int last = nq - 1;
        d0 = lg_ld4_sc_issue<2>(pr + 4 * min(t, last));
        d1 = lg_ld4_sc_issue<2>(pr + 4 * min(t + 256, last));
        d2 = lg_ld4_sc_issue<2>(pr + 4 * min(t + 512, last));
        d3 = lg_ld4_sc_issue<2>(pr + 4 * min(t + 768, last));
        lg_ld4_wait(d0, d1, d2, d3);
        const lg_x4u d[4] = { d0, d1, d2, d3 };
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) dv[v] = make_float4(__uint_as_float(d[v].x), __uint_as_float(d[v].y), __uint_as_float(d[v].z), __uint_as_float(d[v].w));
    }
    stamp(6);
    {
        float ss = 0.0f;
        if (rowlane) {
            #pragma unroll
            for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) ss = lg_sumsq4(dv[v], ss);
        }
        ss = lg_block_sum256_of512(ss, red3[0]);
        if (rowlane) {
            const float sc = 1.0f / sqrtf(ss / (float)E + a.eps);
            #pragma unroll
            for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) {
                const float4 w = wpost[v];
                float4 r;
                r.x = xv[v].x + dv[v].x * sc * w.x;  r.y = xv[v].y + dv[v].y * sc * w.y;
                r.z = xv[v].z + dv[v].z * sc * w.z;  r.w = xv[v].w + dv[v].w * sc * w.w;
                xv[v] = r;
            }
            float4 *xo = (float4 *)(a.x_out + (size_t)jr * E);
            #pragma unroll
            for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq && v == v_) xo[t + 256 * v] = xv[v];
        }
    }
    {
        float ss = 0.0f;
        if (rowlane) {
            #pragma unroll
            for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) ss = lg_sumsq4(xv[v], ss);
        }
        ss = lg_block_sum256_of512(ss, red3[1]);
        if (rowlane) {
            const float sc = 1.0f / sqrtf(ss / (float)E + a.eps);
            #pragma unroll
            for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) {
                const float4 w = wpre[v];
                xv[v] = make_float4(xv[v].x * sc * w.x, xv[v].y * sc * w.y, xv[v].z * sc * w.z, xv[v].w * sc * w.w);
            }
        }
    }
    if (rowlane) {
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) {
            if (t + 256 * v >= nq || v != v_) continue;
            float d; int sum;
            const uint32_t packed = lg_quant4_8lanes(xv[v], &d, &sum);
            const int quad = t + 256 * v;
            if (a.q_units == 2) {
                uint32_t *blk = (uint32_t *)a.q + (size_t)(quad >> 3) * LG_MU_DWORDS;
                const int dw = quad & 7;
                blk[jr * 8 + ((dw & 1) | ((dw & 2) << 1) | ((dw & 4) >> 1))] = packed;
                if ((t & 7) == 0) *(float2 *)(blk + 64 + 2 * jr) = make_float2(d, 12582912.0f + (float)(8 * sum));
            } else {
                uint32_t *unit = (uint32_t *)a.q + ((size_t)(quad >> 3) * ((M + 2) / 3) + jr / 3) * 32;
                unit[(jr % 3) * 8 + (quad & 7)] = packed;
                if ((t & 7) == 0) *(float2 *)(unit + 24 + 2 * (jr % 3)) = make_float2(d, __int_as_float(sum));
            }
        }
    }
    stamp(7);
    if (u == 0 && t == 0) a.sync->gen = gen + 1;
}
