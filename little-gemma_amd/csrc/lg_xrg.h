// lg_xrg.h — the row work ahead of gate/up and gate/up + GeGLU as ONE launch (verify blocks of 4..8 rows).
//
// Launched one after the other, lg_k_rows (a handful of workgroups: residual update, ffn norm, q8) and lg_k_geglu_m
// (the largest weight stream of a layer) each pay a kernel boundary, and the weight stream cannot start before the
// rows are done although it does not depend on them.  Here the first P = M x slices workgroups of the launch do the
// row work (lg_k_rows' arithmetic, lane for lane) and every other workgroup is a gate/up workgroup of lg_k_geglu_m
// that requests ALL of its weights first (a K segment per wavefront: NIT tiles of 16 + 2 bytes per lane, in
// registers), then waits for the P row workgroups, then copies its activations and runs its chains.  The weights
// travel while the rows are being made.
//
// The row workgroups sit on whatever XCDs the dispatcher gives them and the gate/up workgroups on all of them, so
// the hand-over crosses XCDs: the q8 blocks are stored write-through (sc1), the stores waited for, then a flag per
// row workgroup is stored the same way (in 32 copies, a line each); a gate/up workgroup polls one copy of the P flags
// with sc1 loads and then reads its activations with plain loads (its XCD's L2 holds nothing of that buffer: it was
// emptied at the kernel boundary, and nothing on the XCD reads the buffer before the flags are up).  The row workgroups
// have the lowest workgroup ids: they are dispatched first and wait for nobody, so the launch cannot deadlock
// whatever the residency of the others; a gate/up workgroup that gives up its bounded wait reports it in
// StepCtl.err and goes on, so the kernel always ends and the host refuses the step.
//
// Measured (E4B shape, 5 rows; stamps of a launch, microseconds since its first workgroup's start): the row workgroups
// have their row at 1.7-2.8, their stores out at 4.5-5.1 and acknowledged at 4.8-5.6 (alone, lg_k_rows ends 3 us after
// its start: beside some hundred workgroups that pull 29 MB every memory round trip of the rows is longer); the
// gate/up workgroups have their weights at 2.7-4.8, see the flags at 6.3-6.5, have their activations at 6.6-7.0, their
// chains done at 8.5-9.9 and end at 9.3-11.2.  12.3 us per launch against 4.4 + 8.6 for the two kernels, and the step
// 2.188 against 2.168 ms (12B shape: 19.5 against 4.3 + 13.0 us, 3.53 against 3.42 ms): the signal through memory
// (acknowledged stores, flag, poll, load: four round trips) costs more than the kernel boundary it replaces, whose
// launch gap the graph hides anyway.  Bit-identical; kept as an option, off (`rows_geglu`).
//
// A flag holds an epoch that no earlier launch has used: base + seq + 1, where `base` is advanced once per step by
// the step's first kernel (the embedding rows: RowArgs.bump) and seq is the launch's number inside the step (the
// layer).  Nothing changes `base` while a step's launches run, so every workgroup of a launch computes the same
// epoch whenever it starts.
#pragma once
#include "lg_kernels.h"
#include "lg_xcd.h"
#include "lg_xffn.h"
#include "lg_xtail.h"

#define LG_RG_MAXP 32               // most row workgroups of a launch (lane i of a wavefront polls flag i)
#define LG_RG_COPIES 32             // copies of the flags, a 128-byte line each: a gate/up workgroup polls copy (id % 32), so that
                                    // the polls of some hundred workgroups do not all queue at one memory channel
struct RgSync {
    uint32_t base;
    uint32_t pad[31];
    uint32_t flags[LG_RG_COPIES][LG_RG_MAXP];
};
struct RowsGegluArgs {
    const float   *x, *dout, *w_post, *w_pre;   // [M][E] residual, [M][E] (x dparts) previous output, its norm weight, the ffn norm weight
    float         *x_out;                       // [M][E] updated residual
    int8_t        *hq;                          // the rows' q8 as 80-dword blocks (written by the row workgroups, read by the others)
    int            E, dparts, slices;           // dparts: 1, or 4 slabs of partial sums added as (p0+p1)+(p2+p3)
    float          eps;
    const uint8_t *w;                           // tiled ffn_gate_up [n_ff/32 tiles of 64 rows][E/32]
    int            n_ff;
    int8_t        *gq;                          // q8 of gelu(gate) * up
    int            gq_units;                    // as GegluArgs
    RgSync        *sync;
    int            seq;                         // number of this launch inside the step
    int            spin_limit;
    unsigned long long *stamps;                 // nullptr, or [64][8] device wall-clock ticks: units 0..P-1 the row workgroups, 32.. some gate/up workgroups (measurement runs)
};
#define LG_RG_FIELDS(X, v) X(const float *, x, x, v) X(const float *, dout, dout, v) X(const float *, w_post, w_post, v) X(const uint8_t *, w, w, v) \
    X(int, E, E, v) X(int, dparts, dparts, v) X(int, slices, slices, v) X(RgSync *, sync, sync, v) X(int, seq, seq, v) X(const float *, w_pre, w_pre, v) \
    X(float *, x_out, x_out, v) X(int8_t *, hq, hq, v) X(float, eps, eps, v) X(int, n_ff, n_ff, v) X(int8_t *, gq, gq, v) X(int, gq_units, gq_units, v) \
    X(int, spin_limit, spin_limit, v) X(unsigned long long *, stamps, stamps, v)

// NIT: tiles of a wavefront's K segment (E / 256): the whole segment is held in registers.
template <int M, int NIT>
__global__ __launch_bounds__(512, 4) void lg_k_rows_geglu(StepCtl *ctl, LG_RG_FIELDS(LG_XP, _) int p_end_) {
    RowsGegluArgs a; LG_RG_FIELDS(LG_XI, a)
    extern __shared__ __align__(16) unsigned char smem[];     // gate/up workgroups: [8 segments][NIT][80 dwords]
    __shared__ float red[8][LG_HIP_MAX_ROWS_DEV][64];
    const int P = M * a.slices;
    const uint32_t epoch = a.sync->base + (uint32_t)a.seq + 1u;
    const int E = a.E;
    if ((int)blockIdx.x < P) {
        // ---- a row workgroup: row j, storing and quantizing the float4s t + 256 vs of every lane (lg_k_rows with a
        //      previous output, no output scale, a norm weight and the block order of lg_k_geglu_m); wavefronts 4..7
        //      only take part in the workgroup's barriers
        float *scr = &red[0][0][0];
        const int t = threadIdx.x, j = (int)blockIdx.x / a.slices, vs = (int)blockIdx.x - j * a.slices, nq = E >> 2;
        const bool rowt = t < 256;
        auto stamp = [&](int i) { if (a.stamps && t == 0) a.stamps[(size_t)blockIdx.x * 8 + i] = wall_clock64(); };
        stamp(0);
        float4 xv[LG_ROWV], dv[LG_ROWV], wpost[LG_ROWV], wpre[LG_ROWV];
        if (rowt) {
            const float4 *xr = (const float4 *)(a.x + (size_t)j * E), *dr = (const float4 *)(a.dout + (size_t)j * E);
            const float4 *wr = (const float4 *)a.w_post, *w2 = (const float4 *)a.w_pre;
            #pragma unroll
            for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) { xv[v] = xr[t + 256 * v]; dv[v] = dr[t + 256 * v]; wpost[v] = wr[t + 256 * v]; }
            if (a.dparts == 4) {
                const size_t slab = (size_t)M * nq;
                #pragma unroll
                for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) {
                    const float4 p1 = dr[slab + t + 256 * v], p2 = dr[2 * slab + t + 256 * v], p3 = dr[3 * slab + t + 256 * v], p0 = dv[v];
                    dv[v] = make_float4((p0.x + p1.x) + (p2.x + p3.x), (p0.y + p1.y) + (p2.y + p3.y),
                                        (p0.z + p1.z) + (p2.z + p3.z), (p0.w + p1.w) + (p2.w + p3.w));
                }
            }
            #pragma unroll
            for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) wpre[v] = w2[t + 256 * v];
        }
        {
            float ss = 0.0f;
            if (rowt) {
                #pragma unroll
                for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) ss = lg_sumsq4(dv[v], ss);
            }
            ss = lg_block_sum256_of512(ss, scr);
            stamp(1);
            const float sc = 1.0f / sqrtf(ss / (float)E + a.eps);
            if (rowt) {
                #pragma unroll
                for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) {
                    const float4 w = wpost[v];
                    float4 r;
                    r.x = xv[v].x + dv[v].x * sc * w.x;  r.y = xv[v].y + dv[v].y * sc * w.y;
                    r.z = xv[v].z + dv[v].z * sc * w.z;  r.w = xv[v].w + dv[v].w * sc * w.w;
                    xv[v] = r;
                }
                float4 *xo = (float4 *)(a.x_out + (size_t)j * E);
                #pragma unroll
                for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq && v == vs) xo[t + 256 * v] = xv[v];
            }
        }
        {
            float ss = 0.0f;
            if (rowt) {
                #pragma unroll
                for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) ss = lg_sumsq4(xv[v], ss);
            }
            ss = lg_block_sum256_of512(ss, scr + 8);
            const float sc = 1.0f / sqrtf(ss / (float)E + a.eps);
            if (rowt) {
                #pragma unroll
                for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) {
                    const float4 w = wpre[v];
                    xv[v] = make_float4(xv[v].x * sc * w.x, xv[v].y * sc * w.y, xv[v].z * sc * w.z, xv[v].w * sc * w.w);
                }
                #pragma unroll
                for (int v = 0; v < LG_ROWV; ++v) {
                    if (t + 256 * v >= nq || v != vs) continue;     // (nq is a multiple of 64: whole wavefronts)
                    float d; int sum;
                    const uint32_t packed = lg_quant4_8lanes(xv[v], &d, &sum);
                    const int quad = t + 256 * v;
                    uint32_t *blk = (uint32_t *)a.hq + (size_t)(quad >> 3) * LG_MU_DWORDS;
                    const int dw = quad & 7;
                    lg_st_sc<2>(blk + j * 8 + ((dw & 1) | ((dw & 2) << 1) | ((dw & 4) >> 1)), packed);
                    if ((t & 7) == 0) {
                        lg_st_sc<2>(blk + 64 + 2 * j, __float_as_uint(d));
                        lg_st_sc<2>(blk + 64 + 2 * j + 1, __float_as_uint(12582912.0f + (float)(8 * sum)));
                    }
                }
            }
        }
        stamp(2);
        lg_wait_vm();                                         // every store of this workgroup has reached memory
        __syncthreads();
        stamp(3);
        if (t < LG_RG_COPIES) lg_st_sc<2>(a.sync->flags[t] + blockIdx.x, epoch);
        return;
    }
    // ---- a gate/up workgroup: lg_k_geglu_m with the whole K segment's weights requested before anything else
    const int lane = threadIdx.x & 63, n = lane & 31, h = lane >> 5;
    const int s = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));      // K segment of this wavefront
    const int t = (int)blockIdx.x - P, nb = E >> 5;
    const uint8_t *wt = a.w + ((size_t)t * nb + (size_t)s * NIT) * LG_TILE;
    const int su = t == 0 ? 32 : t == 1 ? 33 : t == 160 ? 34 : t == 319 ? 35 : -1;
    auto stamp = [&](int i) { if (a.stamps && su >= 0 && threadIdx.x == 0) a.stamps[(size_t)su * 8 + i] = wall_clock64(); };
    stamp(0);
    uint4 wq[NIT]; uint32_t wd[NIT];
    {
        const __amdgpu_buffer_rsrc_t rw = lg_buffer_rsrc(wt);
        #pragma unroll
        for (int u = 0; u < NIT; ++u) { wq[u] = lg_ldt16b(rw, u, lane); wd[u] = lg_ldt2b(rw, u, lane); }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (s == 0) {                                             // the rows are ready when every row workgroup's flag holds this launch's epoch
        int err = LG_XFFN_ERR_WAIT;
        for (int spins = 0; spins < a.spin_limit; ++spins) {
            if (spins == 1) stamp(1);
            const uint32_t f = lane < P ? lg_ld_sc<2>(a.sync->flags[blockIdx.x % LG_RG_COPIES] + lane) : epoch;
            if (__all(f == epoch)) { err = 0; break; }
        }
        if (err && lane == 0) atomicOr(&ctl->err, err);
        stamp(2);
    }
    __syncthreads();
    unsigned char *la = smem + (size_t)s * NIT * (LG_MU_DWORDS * 4);
    {   // this wavefront's K segment of the rows, four loads in flight per lane.  Plain loads: the caches were emptied of
        // this buffer at the kernel boundary and nothing on this XCD has read it since, so the first workgroup to ask
        // brings a line from memory (where the write-through stores put it before the flag) and the others share it
        const uint4 *src = (const uint4 *)((const unsigned char *)a.hq + (size_t)s * NIT * (LG_MU_DWORDS * 4));
        constexpr int nu = NIT * (LG_MU_DWORDS / 4);
        for (int i0 = lane; i0 < nu; i0 += 256) {
            const int i1 = min(i0 + 64, nu - 1), i2 = min(i0 + 128, nu - 1), i3 = min(i0 + 192, nu - 1);
            const uint4 t0 = src[i0], t1 = src[i1], t2 = src[i2], t3 = src[i3];
            __builtin_amdgcn_sched_barrier(0);
            ((uint4 *)la)[i0] = t0; ((uint4 *)la)[i1] = t1; ((uint4 *)la)[i2] = t2; ((uint4 *)la)[i3] = t3;
        }
        // read back below by other lanes of this wavefront only
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    stamp(3);
    float pg[4] = { 0.0f, 0.0f, 0.0f, 0.0f }, pu[4] = { 0.0f, 0.0f, 0.0f, 0.0f };
    // The integer dots are turned into floats as in lg_k_geglu_m (the bit pattern of 1.5 * 2^23 plus the dot, read as a
    // float, minus the stored 12582912 + 8*sum: exact), with the constant added after the matrix instruction instead of
    // sitting in its 16 accumulator registers, and the gate and the up product one after the other through the same
    // 16 result registers: beside the segment's weights the registers of a workgroup of two per CU hold no more.
    lg_v16i zero;
    #pragma unroll
    for (int i = 0; i < 16; ++i) zero[i] = 0;
    const int arow = n < 8 ? n : 7;
    #pragma unroll
    for (int c = 0; c < NIT; ++c) {
        const unsigned char *lb = la + (size_t)c * (LG_MU_DWORDS * 4);
        const lg_v4i av = *(const lg_v4i *)(lb + arow * 32 + h * 16);
        const int4 sc0 = *(const int4 *)(lb + 256 + h * 32), sc1 = *(const int4 *)(lb + 256 + h * 32 + 16);
        const uint4 q = wq[c];
        const lg_v2u s0 = __builtin_amdgcn_permlane32_swap(q.x, q.z, false, false);
        const lg_v2u s1 = __builtin_amdgcn_permlane32_swap(q.y, q.w, false, false);
        const lg_v2u sd = __builtin_amdgcn_permlane32_swap(wd[c], wd[c], false, false);
        const float dg = lg_h2f((uint16_t)sd.x), du = lg_h2f((uint16_t)sd.y);
        const float xd[4] = { __int_as_float(sc0.x), __int_as_float(sc0.z), __int_as_float(sc1.x), __int_as_float(sc1.z) };
        const float cf[4] = { __int_as_float(sc0.y), __int_as_float(sc0.w), __int_as_float(sc1.y), __int_as_float(sc1.w) };
        {
            lg_v4i bg;
            bg.x = s0.x & 0x0F0F0F0F; bg.y = s1.x & 0x0F0F0F0F; bg.z = (s0.x >> 4) & 0x0F0F0F0F; bg.w = (s1.x >> 4) & 0x0F0F0F0F;
            const lg_v16i d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, bg, zero, 0, 0, 0);
            #pragma unroll
            for (int i = 0; i < 4; ++i) pg[i] = lg_fmaf(xd[i] * dg, __int_as_float(d0[i] + 0x4B400000) - cf[i], pg[i]);
            // (the sums are pinned here: left alone, the compiler runs all the matrix instructions first and parks their results in scratch memory)
            asm volatile("" : "+v"(pg[0]), "+v"(pg[1]), "+v"(pg[2]), "+v"(pg[3]));
        }
        __builtin_amdgcn_sched_barrier(0);
        {
            lg_v4i bu;
            bu.x = s0.y & 0x0F0F0F0F; bu.y = s1.y & 0x0F0F0F0F; bu.z = (s0.y >> 4) & 0x0F0F0F0F; bu.w = (s1.y >> 4) & 0x0F0F0F0F;
            const lg_v16i d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, bu, zero, 0, 0, 0);
            #pragma unroll
            for (int i = 0; i < 4; ++i) pu[i] = lg_fmaf(xd[i] * du, __int_as_float(d1[i] + 0x4B400000) - cf[i], pu[i]);
            asm volatile("" : "+v"(pu[0]), "+v"(pu[1]), "+v"(pu[2]), "+v"(pu[3]));
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    stamp(4);
    #pragma unroll
    for (int i = 0; i < 4; ++i) { red[s][4 * h + i][n] = pg[i]; red[s][4 * h + i][32 + n] = pu[i]; }
    __syncthreads();
    stamp(5);
    for (int j = threadIdx.x >> 5; j < M; j += 16) {         // half-wavefront per row, one FFN column per lane
        const int i = threadIdx.x & 31;
        float g[8], u[8];
        #pragma unroll
        for (int c = 0; c < 8; ++c) { g[c] = red[c][j][i]; u[c] = red[c][j][32 + i]; }
        const float gate = ((g[0] + g[1]) + (g[2] + g[3])) + ((g[4] + g[5]) + (g[6] + g[7]));
        const float up = ((u[0] + u[1]) + (u[2] + u[3])) + ((u[4] + u[5]) + (u[6] + u[7]));
        float d; int sum;
        const int q = lg_quant1_32lanes(lg_gelu(gate) * up, &d, &sum);
        if (a.gq_units == 2) {                                // block t of 80 dwords: row slot j's 32 bytes, dwords in the order 0 1 4 5 2 3 6 7
            int8_t *blk = a.gq + (size_t)t * (LG_MU_DWORDS * 4);
            const int dw = i >> 2;
            blk[(j * 8 + ((dw & 1) | ((dw & 2) << 1) | ((dw & 4) >> 1))) * 4 + (i & 3)] = (int8_t)q;
            if (i == 0) *(float2 *)(blk + 256 + 8 * j) = make_float2(d, 12582912.0f + (float)(8 * sum));
            continue;
        }
        const ActLayout lay = lg_act_layout(a.n_ff);          // order the ffn_down matmul reads
        a.gq[(size_t)j * a.n_ff + lg_act_unit(lay, t * 2 + (i >> 4)) * 16 + (i & 15)] = (int8_t)q;
        if (i == 0) lg_q8_ds<M>(a.gq, a.n_ff)[(size_t)j * (a.n_ff >> 5) + lg_act_block(lay, t)] = make_float2(d, __int_as_float(sum));
    }
    stamp(6);
}
