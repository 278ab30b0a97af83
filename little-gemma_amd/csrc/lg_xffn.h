// lg_xffn.h — the feed-forward half of a layer as ONE launch, partitioned by XCD (verify blocks of 4..8 rows).
//
// As separate kernels the half is  rows (post-attention add-norm, ffn norm, q8) -> gate/up + GeGLU (+ q8) -> ffn_down:
// three launches, two chip-wide hand-overs through memory, and at every kernel start a chip that has no weight in
// flight.  Here the 256 workgroups of one launch (one per CU, workgroup i on XCD i % 8) form 8 groups of 32, and XCD x
// does, for its eighth of the FFN columns [x*FF/8, (x+1)*FF/8):
//   A  the row work of all M rows, one row per workgroup (ranks 0..M-1), redundantly per XCD: the q8 rows land in the
//      XCD's L2 (plain stores), the workgroups of XCD 0 also write the new residual;
//   B  gate/up for the XCD's columns, FF/256 columns per workgroup, all 8 K segments of a column in one workgroup, so
//      the segment tree and the GeGLU are local; gelu(gate)*up goes to the XCD's L2 as f32;
//   C  the XCD's K share of ffn_down (whole K segments: lg_segments(FF)/8 of them) for all E output rows, E/32 rows per
//      workgroup: every workgroup quantizes the XCD's FF/8 activations itself (same q8 as the GeGLU epilogue of
//      lg_k_geglu_m: amax, d = amax/127, ties-even), runs the serial chains of its segments and adds them in
//      adjacent-pair order: the bottom levels of the row's segment tree.  Slab x of 8 receives the partial sums; the
//      consumer adds the 8 slabs with the top three levels of the same tree, so every sum keeps its defined order.
// A -> B and B -> C are hand-overs inside the XCD (flags in the XCD's L2, L1-bypassing loads: lg_xcd.h).  A workgroup
// is 8 compute wavefronts (one K segment of gate/up each) and 4 more that do the row work (in the M workgroups that have
// a row), the first of which also serves the hand-overs: a wavefront's loads return in the order they were requested
// and a store is known to have landed only when everything requested before it has (s_waitcnt vmcnt), so a wavefront
// with a segment of weights in flight can neither publish data nor poll a flag without waiting for its weights; the
// hand-over wavefront has nothing in flight, takes what is to be published from LDS, stores it, waits, raises the flag
// and polls.  The compute wavefronts stream their weights in pairs of blocks (a few KB in flight per wavefront: the
// first pair is requested before the hand-over is waited for, every next one while the current one is multiplied).
// More in flight is slower, not faster: a wavefront's loads return in order, what arrives early waits in the CU's
// 32 KB L1, and beyond that lines are evicted before they are delivered (with a whole K segment per wavefront
// requested at once the same kernel took twice as long); and parking the weights in LDS first makes the dots wait
// for the LDS pipe, which the activation operands already keep busy.
// The 4 row-work wavefronts also do everything else that goes through memory for a hand-over: they copy the group's q8
// rows into LDS for the compute wavefronts, do the segment tree and the GeGLU, publish the result, fetch the group's
// activations and quantize them into LDS.  The compute wavefronts only stream weights and multiply.  The two kinds run
// separate branches (so the registers of neither add to the other's) that meet at workgroup barriers; among themselves
// the row-work wavefronts synchronise through a counter in LDS, which the compute wavefronts never wait for.  Every wait is bounded: a workgroup that gives up sets
// StepCtl.err and goes on, so the kernel always ends.
// The groups are the workgroups i with the same i % 8; which XCD a group runs on may differ from launch to launch
// (the dispatcher goes on dealing where the previous launch stopped), so every flag carries its writer's XCD id and a
// reader on another XCD reports it instead of using stale data.
//
// Weights come from per-workgroup streams built at upload (xffn_pack_*): what a workgroup reads is contiguous, in
// matrix-core operand order (lane (n, h) of an operand of 32 weight rows holds bytes 8h..8h+7 of row n's q4_0 block,
// i.e. K = 8h..8h+7 and 16+8h..16+8h+7: no lane exchange), two consecutive blocks of a K segment per 16-byte load, and
// the two blocks' f16 scales as one dword per lane (a segment with an odd number of blocks is padded with a zero block).
#pragma once
#include "lg_kernels.h"
#include "lg_xcd.h"

struct XcdSync {
    uint32_t gen[LG_XCDS];                       // per group: launches so far (advanced by rank 0 at the end of a launch)
    uint32_t flags[LG_XCDS][2][LG_XCD_WGS];      // per group and hand-over: (epoch << 4 | XCD id) of each rank's last arrival; epoch = 2 * gen + 1, + 2
};

struct XffnGeo {
    int E, FF;
    int nb, nit, nitp;        // gate/up: blocks per row, per K segment (8 segments), the latter rounded up to even
    int CW, R2, ops;          // per workgroup: FFN columns, weight rows (gate then up), operands of 32 rows
    int C, CB;                // per XCD: FFN columns, q8 blocks
    int RW, groups;           // ffn_down: output rows per workgroup, operands of 32 rows
    int SX, nitd, nitdp;      // ffn_down: K segments per XCD, blocks per segment, rounded up to even
    int units;                // groups * SX (operand, segment) chains per workgroup
    int rb, rbd;              // stream bytes per weight row and segment: 18 per block of the (padded) even count
    size_t gu_seg, gu_bytes, dn_bytes;           // stream bytes per gate/up segment, per workgroup: gate/up, down
    bool ok;
    // LDS of a workgroup for blocks of M rows: the q8 rows of gate/up (before that, this workgroup's row on its way out),
    // the segment sums of gate/up, the q8 activations of ffn_down, this workgroup's gelu(gate)*up, the chain sums
    __host__ __device__ size_t lds(int M) const {
        return (size_t)nb * 320 + (size_t)8 * M * ops * 32 * 4 + (size_t)SX * nitd * 320 + (size_t)M * CW * 4 + (size_t)units * M * 32 * 4;
    }
};
__host__ __device__ static inline XffnGeo lg_xffn_geo(int E, int FF) {
    XffnGeo g{};
    g.E = E; g.FF = FF;
    g.ok = E >= 256 && E % 256 == 0 && E <= 4096 && FF >= 256 && FF % 256 == 0;
    if (!g.ok) return g;
    g.nb = E >> 5; g.nit = g.nb >> 3; g.nitp = (g.nit + 1) & ~1;
    g.CW = FF >> 8; g.R2 = 2 * g.CW; g.ops = (g.R2 + 31) >> 5;
    g.C = FF >> 3; g.CB = g.C >> 5;
    g.RW = E >> 5; g.groups = (g.RW + 31) >> 5;
    const int sd = lg_segments(FF);
    g.SX = sd / LG_XCDS; g.nitd = (FF >> 5) / sd; g.nitdp = (g.nitd + 1) & ~1;
    g.ok = (FF >> 5) % sd == 0;
    g.units = g.groups * g.SX;
    g.rb = 18 * g.nitp; g.rbd = 18 * g.nitdp;
    g.gu_seg = (size_t)g.R2 * g.rb; g.gu_bytes = 8 * g.gu_seg;
    g.dn_bytes = (size_t)g.RW * g.SX * g.rbd;
    return g;
}

// (arguments one by one, the most urgent first: the leading ones arrive in scalar registers at launch, see LG_XP)
struct XffnArgs {
    const uint8_t *wgu, *wdn;      // per-workgroup weight streams: [256][gu_bytes], [256][dn_bytes]
    const float *x, *dout;         // [M][E] residual and attention output projection
    const float *w_post, *w_pre;   // [E] post-attention norm, ffn norm
    float *x_out;                  // [M][E] new residual
    float *slabs;                  // [8][M][E] partial sums of ffn_down
    uint32_t *xq;                  // [8][E/32][80] q8 rows of A, per group (matrix-core block order of lg_k_rows, q_units 2)
    float *act;                    // [8][M][FF/8] gelu(gate)*up, per group
    XcdSync *sync;
    StepCtl *ctl;
    int E, FF;
    float eps;
    int spin_limit;
    int delay_w;                   // the compute wavefronts sleep this many units of 64 clocks before they request their weights (the rows' loads go first)
    unsigned long long *stamps;    // nullptr, or [256][LG_XFFN_STAMPS] device wall-clock ticks at the phase boundaries of every workgroup (measurement runs)
};
#define LG_XFFN_FIELDS(X, v) X(const uint8_t *, wgu, wgu, v) X(const float *, x, x, v) X(const float *, dout, dout, v) X(const float *, w_post, w_post, v) X(const float *, w_pre, w_pre, v) X(int, E, E, v) X(int, FF, FF, v) X(XcdSync *, sync, sync, v) X(const uint8_t *, wdn, wdn, v) X(float *, x_out, x_out, v) X(float *, slabs, slabs, v) X(uint32_t *, xq, xq, v) X(float *, act, act, v) X(StepCtl *, ctl, ctl, v) X(float, eps, eps, v) X(int, spin_limit, spin_limit, v) X(int, delay_w, delay_w, v) X(unsigned long long *, stamps, stamps, v)
#define LG_XFFN_STAMPS 16
#define LG_XFFN_THREADS 768        // 8 compute wavefronts, 4 for the row work (the first of them serves the hand-overs)

#define LG_XFFN_ERR_PLACE 0x100    // StepCtl.err: the workgroups of a group did not all run on one XCD
#define LG_XFFN_ERR_WAIT  0x200    // StepCtl.err: a hand-over was given up

// one 8-byte / 2-byte piece of a weight stream, non-temporal (streams pass through the caches once)
__device__ __forceinline__ lg_v2u lg_ldw8(const void *p) { return __builtin_nontemporal_load((const lg_v2u *)p); }
// loads that are served by the XCD's L2 (not by this CU's L1): what another workgroup of the XCD stored
__device__ __forceinline__ unsigned long long lg_ld_l2_u64(const void *p) {
    return __hip_atomic_load((const unsigned long long *)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The hand-over wavefront's side of a flag barrier: publish this rank's arrival (its stores have been waited for),
// then poll the flags of ranks 0..n-1 (lane i polls flag i) until all have reached `epoch`.  Returns 0, or the error
// bits: a flag written from another XCD, or the bounded wait given up.
__device__ __forceinline__ int lg_xcd_arrive_wait(uint32_t *flags, int rank, bool arrive, int n, uint32_t epoch, int xcc, int spin_limit) {
    const int lane = threadIdx.x & 63;
    if (arrive && lane == 0) lg_st_sc<0>(flags + rank, (epoch << 4) | (uint32_t)xcc);
    for (int spins = 0; spins < spin_limit; ++spins) {
        const uint32_t f = lane < n ? lg_ld_sc<2>(flags + lane) : ((epoch << 4) | (uint32_t)xcc);
        const bool there = (int)(((f >> 4) - epoch) << 4) >= 0;              // epochs are 28-bit counters that wrap
        if (__all(there)) return __any((int)(f & 15) != xcc) ? LG_XFFN_ERR_PLACE : 0;
    }
    return LG_XFFN_ERR_WAIT;
}

// one operand step: 32 weight rows x one q4_0 block against the block's activations (8 row slots), the scaled
// block dots of the lane's four draft rows added to p in place: p = fma(xd * dw, (float)dot, p)
__device__ __forceinline__ void lg_xffn_step(const lg_v4i av, const float (&xd)[4], const float (&cf)[4], lg_v2u q, float dw,
                                             const lg_v16i &magic, float (&p)[4]) {
    lg_v4i b;
    b.x = q.x & 0x0F0F0F0F; b.y = q.y & 0x0F0F0F0F; b.z = (q.x >> 4) & 0x0F0F0F0F; b.w = (q.y >> 4) & 0x0F0F0F0F;
    const lg_v16i d = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, b, magic, 0, 0, 0);
    #pragma unroll
    for (int i = 0; i < 4; ++i) p[i] = lg_fmaf(xd[i] * dw, __int_as_float(d[i]) - cf[i], p[i]);
}
// the activation operand and the four rows' {scale, 12582912 + 8*sum} of one 80-dword block in LDS
struct XffnAct { lg_v4i av; float xd[4], cf[4]; };
__device__ __forceinline__ XffnAct lg_xffn_act(const unsigned char *lb, int arow, int h) {
    XffnAct r;
    r.av = *(const lg_v4i *)(lb + arow * 32 + h * 16);
    const int4 sc0 = *(const int4 *)(lb + 256 + h * 32), sc1 = *(const int4 *)(lb + 256 + h * 32 + 16);
    r.xd[0] = __int_as_float(sc0.x); r.xd[1] = __int_as_float(sc0.z); r.xd[2] = __int_as_float(sc1.x); r.xd[3] = __int_as_float(sc1.z);
    r.cf[0] = __int_as_float(sc0.y); r.cf[1] = __int_as_float(sc0.w); r.cf[2] = __int_as_float(sc1.y); r.cf[3] = __int_as_float(sc1.w);
    return r;
}

// Synchronisation among the LG_XFFN_ROWW row-work wavefronts only (a counter in LDS that starts at 0; the k-th use
// waits for k * LG_XFFN_ROWW arrivals).  LDS executes a wavefront's accesses in order, so what a wavefront wrote to LDS
// before its arrival is visible to whoever has seen the arrival.
#define LG_XFFN_ROWW 4
__device__ __forceinline__ void lg_rowsync(uint32_t *cnt, uint32_t &uses) {
    uses += LG_XFFN_ROWW;
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if ((threadIdx.x & 63) == 0) __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    while (__hip_atomic_load(cnt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < uses) __builtin_amdgcn_s_sleep(1);
    asm volatile("" ::: "memory");
}

// M: rows of the block (4..8).  OPS: gate/up operands per workgroup; NC: capacity in blocks of a gate/up K segment;
// UW: ffn_down chains per wavefront; NDC: capacity in blocks of an ffn_down segment; CBC: capacity in q8 blocks of a
// group's activations.
template <int M, int OPS, int NC, int UW, int NDC, int CBC>
__global__ __launch_bounds__(LG_XFFN_THREADS) void lg_k_ffn_xcd(LG_XFFN_FIELDS(LG_XP, _) int p_end_) {
    XffnArgs a; LG_XFFN_FIELDS(LG_XI, a)
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float rsum[2][4];
    __shared__ uint32_t rcnt;
    const XffnGeo g = lg_xffn_geo(a.E, a.FF);
    const int wg = blockIdx.x, x = wg & (LG_XCDS - 1), r = wg >> 3;
    const int t = threadIdx.x, lane = t & 63, n = lane & 31, h = lane >> 5;
    const int s = __builtin_amdgcn_readfirstlane(t >> 6);             // 0..7: K segment of a compute wavefront; 8..11: row work and hand-overs
    const bool compute = s < 8, service = s == 8;
    const int E = g.E, nit = g.nit, W = OPS * 32;
    unsigned char *la = smem;                                                 // [nb][320]: A operand blocks of gate/up; before that the row on its way out
    float *red = (float *)(smem + (size_t)g.nb * 320);                        // [8 segments][M][W]
    unsigned char *lad = (unsigned char *)(red + 8 * M * W);                  // [SX*nitd][320]: A operand blocks of ffn_down
    float *actbuf = (float *)(lad + (size_t)g.SX * g.nitd * 320);             // [M][CW]: this workgroup's gelu(gate)*up on its way out
    float *red2 = actbuf + (size_t)M * g.CW;                                  // [units][M][32]: the chain sums of ffn_down
    uint32_t *rowbuf = (uint32_t *)la;                                        // [nb][10]
    uint32_t *flags1 = a.sync->flags[x][0], *flags2 = a.sync->flags[x][1];
    uint32_t *xq = a.xq + (size_t)x * g.nb * LG_MU_DWORDS;
    float *act = a.act + (size_t)x * M * g.C;
    const bool row_wg = r < M;
    auto stamp = [&](int i) { if (a.stamps && (t & 511) == 0) a.stamps[((size_t)wg * 2 + (t >> 9)) * LG_XFFN_STAMPS + i] = wall_clock64(); };
    stamp(0);
    if (t == 512) rcnt = 0;
    __syncthreads();                                                  // (#0: the row-work wavefronts' counter is set)
    lg_v16i magic;                                                    // (float)(dot - 8*sum) in one subtraction: see lg_k_geglu_m
    #pragma unroll
    for (int i = 0; i < 16; ++i) magic[i] = 0x4B400000;
    asm volatile("" : "+v"(magic));                                   // (kept in registers: rebuilt per use it costs 24 instructions)
    const int arow = n < 8 ? n : 7;

    if (compute) {
        // ================= the compute wavefronts: weights and dots =================
        const uint8_t *gs = a.wgu + (size_t)wg * g.gu_bytes + (size_t)s * g.gu_seg;
        struct GuPair { lg_x4u q[OPS]; uint32_t sw[OPS]; };
        auto fetch_gu = [&](int jp) {                                 // blocks 2jp and 2jp+1 of the segment, every operand
            GuPair w;
            const int jc = 2 * jp < g.nitp ? jp : g.nitp / 2 - 1;    // past the segment: its last pair again, never used
            #pragma unroll
            for (int o = 0; o < OPS; ++o) {
                const int vr = g.R2 - 32 * o < 32 ? g.R2 - 32 * o : 32, nn = n < vr ? n : vr - 1;
                const uint8_t *ob = gs + (size_t)32 * o * g.rb;
                w.q[o] = __builtin_nontemporal_load((const lg_x4u *)(ob + (size_t)((jc * 2 + h) * vr + nn) * 16));
                w.sw[o] = __builtin_nontemporal_load((const uint32_t *)(ob + (size_t)g.nitp * vr * 16 + (size_t)(jc * vr + nn) * 4));
            }
            return w;
        };
        GuPair w[3];                                                  // (a ring by position: no register is copied, a copy would wait for its load)
        w[0] = fetch_gu(0); w[1] = fetch_gu(1);                       // in flight while the row work is done
        __builtin_amdgcn_sched_barrier(0);
        stamp(1);
        __syncthreads();                                              // (#1: the group's q8 rows are in LDS)
        stamp(3);
        float p[OPS][4];
        #pragma unroll
        for (int o = 0; o < OPS; ++o)
            #pragma unroll
            for (int i = 0; i < 4; ++i) p[o][i] = 0.0f;
        #pragma unroll
        for (int jp = 0; jp < (NC + 1) / 2; ++jp) {
            if (2 * jp < nit) {                                       // (a guard, not a break: the arrays stay in registers)
                if (2 * jp + 4 < nit) w[(jp + 2) % 3] = fetch_gu(jp + 2);   // two pairs ahead of the one that is multiplied
                __builtin_amdgcn_sched_barrier(0);
                const GuPair &cur = w[jp % 3];
                #pragma unroll
                for (int e = 0; e < 2; ++e) {
                    if (2 * jp + e < nit) {
                        const XffnAct ac = lg_xffn_act(la + (size_t)(s * nit + 2 * jp + e) * (LG_MU_DWORDS * 4), arow, h);
                        #pragma unroll
                        for (int o = 0; o < OPS; ++o) {
                            lg_v2u q; q.x = e ? cur.q[o].z : cur.q[o].x; q.y = e ? cur.q[o].w : cur.q[o].y;
                            lg_xffn_step(ac.av, ac.xd, ac.cf, q, lg_h2f((uint16_t)(e ? cur.sw[o] >> 16 : cur.sw[o])), magic, p[o]);
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                if (jp < 5) stamp(11 + jp);
            }
        }
        stamp(4);
        #pragma unroll
        for (int o = 0; o < OPS; ++o)
            #pragma unroll
            for (int i = 0; i < 4; ++i) if (4 * h + i < M) red[(s * M + 4 * h + i) * W + 32 * o + n] = p[o][i];
        // the wavefront's chains of ffn_down: chain uu is (operand of 32 rows, K segment) number s + 8*uu of the workgroup's;
        // 8 is a multiple of the segments per XCD, so a wavefront's chains share their segment and with it every
        // activation operand.  Their first pair of blocks is requested now and arrives under the GeGLU and the hand-over.
        const int sx = s % g.SX;
        struct DnPair { lg_x4u q[UW]; uint32_t sw[UW]; };
        int uvr[UW]; bool uon[UW]; const uint8_t *ubase[UW];
        #pragma unroll
        for (int uu = 0; uu < UW; ++uu) {
            const int u = s + 8 * uu;
            uon[uu] = u < g.units;
            const int gr = (uon[uu] ? u : s) / g.SX;                 // past the end: the wavefront's first chain again, never stored
            uvr[uu] = g.RW - 32 * gr < 32 ? g.RW - 32 * gr : 32;
            ubase[uu] = a.wdn + (size_t)wg * g.dn_bytes + (size_t)(gr * g.SX * 32 + sx * uvr[uu]) * g.rbd;
        }
        auto fetch_dn = [&](int jp) {
            DnPair w;
            const int jc = 2 * jp < g.nitdp ? jp : g.nitdp / 2 - 1;
            #pragma unroll
            for (int uu = 0; uu < UW; ++uu) {
                const int vr = uvr[uu], nn = n < vr ? n : vr - 1;
                w.q[uu] = __builtin_nontemporal_load((const lg_x4u *)(ubase[uu] + (size_t)((jc * 2 + h) * vr + nn) * 16));
                w.sw[uu] = __builtin_nontemporal_load((const uint32_t *)(ubase[uu] + (size_t)g.nitdp * vr * 16 + (size_t)(jc * vr + nn) * 4));
            }
            return w;
        };
        const bool any = s < g.units;
        DnPair dw[(NDC + 1) / 2];                                     // the whole chains: nothing else streams while they arrive
        #pragma unroll
        for (int jp = 0; jp < (NDC + 1) / 2; ++jp) dw[jp] = fetch_dn(jp);
        __builtin_amdgcn_sched_barrier(0);
        if (a.delay_w & 0x200) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        stamp(5);
        __syncthreads();                                              // (#2: the segment sums of gate/up are in LDS)
        __syncthreads();                                              // (#3: the group's activations are in LDS, quantized)
        stamp(8);
        float pd[UW][4];
        #pragma unroll
        for (int uu = 0; uu < UW; ++uu)
            #pragma unroll
            for (int i = 0; i < 4; ++i) pd[uu][i] = 0.0f;
        if (any) {
            #pragma unroll
            for (int jp = 0; jp < (NDC + 1) / 2; ++jp) {
                if (2 * jp < g.nitd) {
                    const DnPair dcur = dw[jp];
                    #pragma unroll
                    for (int e = 0; e < 2; ++e) {
                        if (2 * jp + e < g.nitd) {
                            const XffnAct ac = lg_xffn_act(lad + (size_t)(sx * g.nitd + 2 * jp + e) * (LG_MU_DWORDS * 4), arow, h);
                            #pragma unroll
                            for (int uu = 0; uu < UW; ++uu) {
                                lg_v2u q; q.x = e ? dcur.q[uu].z : dcur.q[uu].x; q.y = e ? dcur.q[uu].w : dcur.q[uu].y;
                                lg_xffn_step(ac.av, ac.xd, ac.cf, q, lg_h2f((uint16_t)(e ? dcur.sw[uu] >> 16 : dcur.sw[uu])), magic, pd[uu]);
                            }
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            #pragma unroll
            for (int uu = 0; uu < UW; ++uu)
                if (uon[uu]) {
                    #pragma unroll
                    for (int i = 0; i < 4; ++i) if (4 * h + i < M) red2[((s + 8 * uu) * M + 4 * h + i) * 32 + n] = pd[uu][i];
                }
        }
        stamp(9);
    } else {
        // ================= the row-work wavefronts: everything that is handed over through memory =================
        if (a.delay_w & 0x100) __builtin_amdgcn_s_setprio(3);        // (their few instructions ahead of the others')
        const int tt = t - 512;                                       // 0..255: the thread index of lg_k_rows
        uint32_t uses = 0, gen = 0;
        int xcc = 0, err = 0;
        const uint32_t *genp = a.sync->gen + x;
        if (row_wg) {
            // ---- A: this workgroup's row (the arithmetic and the lane assignment of lg_k_rows); its q8 goes to LDS in
            //      the 80-dword block order, from where the first of these wavefronts publishes it
            const int nq = E >> 2;
            float4 xv[LG_ROWV], dv[LG_ROWV], wpost[LG_ROWV], wpre[LG_ROWV];
            {
                const float4 *xr = (const float4 *)(a.x + (size_t)r * E), *dr = (const float4 *)(a.dout + (size_t)r * E);
                const float4 *wo = (const float4 *)a.w_post, *wp = (const float4 *)a.w_pre;
                #pragma unroll
                for (int v = 0; v < LG_ROWV; ++v) if (tt + 256 * v < nq) { xv[v] = xr[tt + 256 * v]; dv[v] = dr[tt + 256 * v]; wpost[v] = wo[tt + 256 * v]; wpre[v] = wp[tt + 256 * v]; }
            }
            if (service) gen = __hip_atomic_load(genp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // (behind the row's loads: it is needed after them)
            stamp(11);
            float ss = 0.0f;
            #pragma unroll
            for (int v = 0; v < LG_ROWV; ++v) if (tt + 256 * v < nq) ss = lg_sumsq4(dv[v], ss);
            ss = lg_wave_sum64(ss);
            if (lane == 0) rsum[0][s - 8] = ss;
            lg_rowsync(&rcnt, uses);
            stamp(12);
            const float scd = 1.0f / sqrtf(((rsum[0][0] + rsum[0][1]) + (rsum[0][2] + rsum[0][3])) / (float)E + a.eps);
            ss = 0.0f;
            #pragma unroll
            for (int v = 0; v < LG_ROWV; ++v) if (tt + 256 * v < nq) {
                const float4 w = wpost[v];
                float4 q;
                q.x = xv[v].x + dv[v].x * scd * w.x;  q.y = xv[v].y + dv[v].y * scd * w.y;
                q.z = xv[v].z + dv[v].z * scd * w.z;  q.w = xv[v].w + dv[v].w * scd * w.w;
                xv[v] = q;
                if (x == 0) ((float4 *)(a.x_out + (size_t)r * E))[tt + 256 * v] = q;
                ss = lg_sumsq4(q, ss);
            }
            ss = lg_wave_sum64(ss);
            if (lane == 0) rsum[1][s - 8] = ss;
            lg_rowsync(&rcnt, uses);
            stamp(13);
            const float scx = 1.0f / sqrtf(((rsum[1][0] + rsum[1][1]) + (rsum[1][2] + rsum[1][3])) / (float)E + a.eps);
            #pragma unroll
            for (int v = 0; v < LG_ROWV; ++v) {
                if (tt + 256 * v >= nq) break;                        // nq is a multiple of 64: whole wavefronts
                const float4 w = wpre[v];
                const float4 hq = make_float4(xv[v].x * scx * w.x, xv[v].y * scx * w.y, xv[v].z * scx * w.z, xv[v].w * scx * w.w);
                float d; int sum;
                const uint32_t packed = lg_quant4_8lanes(hq, &d, &sum);
                const int quad = tt + 256 * v, dw = quad & 7;
                uint32_t *blk = rowbuf + (size_t)(quad >> 3) * 10;
                blk[(dw & 1) | ((dw & 2) << 1) | ((dw & 4) >> 1)] = packed;
                if ((tt & 7) == 0) *(float2 *)(blk + 8) = make_float2(d, 12582912.0f + (float)(8 * sum));
            }
            lg_rowsync(&rcnt, uses);
            stamp(14);
            if (service) {                                            // the row into the group's L2: slot r of every block
                for (int b = lane; b < g.nb; b += 64) {
                    const uint32_t *src = rowbuf + (size_t)b * 10;
                    uint32_t *dst = xq + (size_t)b * LG_MU_DWORDS;
                    const uint2 v0 = *(const uint2 *)src, v1 = *(const uint2 *)(src + 2), v2 = *(const uint2 *)(src + 4), v3 = *(const uint2 *)(src + 6), v4 = *(const uint2 *)(src + 8);
                    *(uint4 *)(dst + r * 8) = make_uint4(v0.x, v0.y, v1.x, v1.y);
                    *(uint4 *)(dst + r * 8 + 4) = make_uint4(v2.x, v2.y, v3.x, v3.y);
                    *(uint2 *)(dst + 64 + 2 * r) = v4;
                }
                lg_wait_vm();                                         // the row is in the group's L2
            }
            stamp(15);
        } else if (service) gen = lg_ld_sc<2>(genp);
        // ---- A -> B: the first wavefront publishes and polls, the others wait for it; then all four copy the group's
        //      q8 rows into LDS for the compute wavefronts
        if (service) {
            xcc = lg_xcc_id();
            err |= lg_xcd_arrive_wait(flags1, r, row_wg, M, 2 * gen + 1, xcc, a.spin_limit);
        }
        stamp(2);
        lg_rowsync(&rcnt, uses);
        {
            const int n16 = g.nb * (LG_MU_DWORDS / 4);                // 16-byte units of the group's rows
            for (int i0 = tt; i0 < n16; i0 += 4 * 256) {
                const int i1 = min(i0 + 256, n16 - 1), i2 = min(i0 + 512, n16 - 1), i3 = min(i0 + 768, n16 - 1);
                lg_x4u v0 = lg_ld4_sc_issue<2>((const uint4 *)xq + i0), v1 = lg_ld4_sc_issue<2>((const uint4 *)xq + i1);
                lg_x4u v2 = lg_ld4_sc_issue<2>((const uint4 *)xq + i2), v3 = lg_ld4_sc_issue<2>((const uint4 *)xq + i3);
                lg_ld4_wait(v0, v1, v2, v3);
                ((lg_x4u *)la)[i0] = v0; ((lg_x4u *)la)[i1] = v1; ((lg_x4u *)la)[i2] = v2; ((lg_x4u *)la)[i3] = v3;
            }
        }
        stamp(4);
        __syncthreads();                                              // (#1)
        __syncthreads();                                              // (#2)
        // ---- segment tree and GeGLU of this workgroup's columns, one (row, column) per thread
        for (int i = tt; i < M * g.CW; i += 256) {
            const int j = i / g.CW, c = i - j * g.CW;
            float gg[8], uu[8];
            #pragma unroll
            for (int k = 0; k < 8; ++k) { gg[k] = red[(k * M + j) * W + c]; uu[k] = red[(k * M + j) * W + g.CW + c]; }
            const float gate = ((gg[0] + gg[1]) + (gg[2] + gg[3])) + ((gg[4] + gg[5]) + (gg[6] + gg[7]));
            const float up = ((uu[0] + uu[1]) + (uu[2] + uu[3])) + ((uu[4] + uu[5]) + (uu[6] + uu[7]));
            actbuf[i] = lg_gelu(gate) * up;
        }
        lg_rowsync(&rcnt, uses);
        // ---- B -> C
        if (service) {
            for (int i = lane; i < M * g.CW; i += 64) { const int j = i / g.CW; act[(size_t)j * g.C + r * g.CW + (i - j * g.CW)] = actbuf[i]; }
            lg_wait_vm();
            stamp(6);
            err |= lg_xcd_arrive_wait(flags2, r, true, LG_XCD_WGS, 2 * gen + 2, xcc, a.spin_limit);
        }
        lg_rowsync(&rcnt, uses);
        stamp(7);
        // ---- the group's activations, q8 (the quantization of lg_k_geglu_m's epilogue) into LDS
        {
            constexpr int TK = (M * CBC * 8 + 255) / 256;             // (row, block, lane of 8) tasks per thread
            const int ntask = M * g.CB * 8;
            #pragma unroll
            for (int u0 = 0; u0 < TK; u0 += 4) {
                lg_x4u v[4];
                #pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int q = min(tt + 256 * (u0 + u), ntask - 1), blk = q >> 3, j = blk % M, kbx = blk / M;
                    v[u] = lg_ld4_sc_issue<2>(act + (size_t)j * g.C + kbx * 32 + (q & 7) * 4);
                }
                lg_ld4_wait(v[0], v[1], v[2], v[3]);
                #pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int q = tt + 256 * (u0 + u), blk = q >> 3, j = blk % M, kbx = blk / M, dw = q & 7;
                    const float4 f = make_float4(__uint_as_float(v[u].x), __uint_as_float(v[u].y), __uint_as_float(v[u].z), __uint_as_float(v[u].w));
                    float d; int sum;
                    const uint32_t packed = lg_quant4_8lanes(f, &d, &sum);
                    if (u0 + u < TK && q < ntask) {
                        uint32_t *bp = (uint32_t *)(lad + (size_t)kbx * (LG_MU_DWORDS * 4));
                        bp[j * 8 + ((dw & 1) | ((dw & 2) << 1) | ((dw & 4) >> 1))] = packed;
                        if (dw == 0) *(float2 *)(bp + 64 + 2 * j) = make_float2(d, 12582912.0f + (float)(8 * sum));
                    }
                }
            }
        }
        stamp(8);
        __syncthreads();                                              // (#3)
        if (service && lane == 0) {
            if (r == 0) lg_st_sc<0>(a.sync->gen + x, gen + 1);        // every rank of the group has read gen long ago (it passed B -> C)
            if (err) atomicOr(&a.ctl->err, err);
        }
    }
    __syncthreads();                                                  // (#4: the chain sums of ffn_down are in LDS)
    for (int idx = t; idx < M * g.RW; idx += LG_XFFN_THREADS) {       // the group's levels of the segment tree, slab x
        const int j = idx / g.RW, rr = idx - j * g.RW, gr = rr >> 5, nn = rr & 31;
        float v;
        if (g.SX == 4) {
            const float *b = red2 + ((size_t)gr * 4 * M + j) * 32 + nn;
            v = (b[0] + b[(size_t)M * 32]) + (b[(size_t)2 * M * 32] + b[(size_t)3 * M * 32]);
        } else v = red2[((size_t)gr * M + j) * 32 + nn];
        a.slabs[((size_t)x * M + j) * E + r * g.RW + rr] = v;
    }
    stamp(10);
}

// ---------------------------------------------------------------------------------------------------------
// ffn_down of verify blocks (4..8 rows) on the matrix cores, as a kernel of its own: exactly 256 workgroups whatever the
// shape.  Workgroup (row group r of 64, K quarter q of 4): its E/64 output rows (one or two operands of up to 32 rows)
// against the 8 K segments 8q .. 8q+7 of the 32, one segment per wavefront: the serial chain of the segment's blocks,
// p = fma(xd * dw, (float)dot, p), one v_mfma_i32_32x32x32_i8 per block and operand (A = the block's activations in 8 row
// slots, B = the rows' nibbles); the 8 chain sums of a row meet in LDS in the adjacent-pair tree (the bottom three
// levels of the 32-segment tree) and go to slab q of four; the consumer adds (p0 + p1) + (p2 + p3), the top two.
// Every CU streams the same E * FF * 18 / 32 / 256 bytes of weights (the v_dot4 kernel's cut, 10 rows x all of K per CU,
// has the same balance but stages all FF activations per workgroup, 64 KB at 5 x 10240, and spends a third of its time
// on vector instructions); a wavefront reads only its own segment's activation blocks.
// Weights: per workgroup, segment and operand the stream layout of the kernels above (pairs of blocks: [pair][half h][row n]
// 8 + 8 nibble bytes, then [pair][row n] the two f16 scales; rows past the operand's count are not stored: their lanes
// read the last row again).  Activations: the 80-dword blocks that lg_k_geglu_m writes when asked to (gq_units = 2).
struct DownMGeo {
    int E, FF, RW, ops, nitd, nitdp, npairs;
    size_t seg_bytes, wg_bytes;        // stream bytes of a (workgroup, segment): all operands; of a workgroup
    bool ok;
};
__host__ __device__ static inline DownMGeo lg_down_m_geo(int E, int FF) {
    DownMGeo g{};
    g.E = E; g.FF = FF;
    g.ok = E >= 64 && E % 64 == 0 && E <= 4096 && FF % 1024 == 0 && lg_segments(FF) == 32;
    if (!g.ok) return g;
    g.RW = E >> 6; g.ops = (g.RW + 31) >> 5;
    g.nitd = (FF >> 5) >> 5; g.nitdp = (g.nitd + 1) & ~1; g.npairs = g.nitdp >> 1;
    g.seg_bytes = (size_t)g.RW * g.nitdp * 18;
    g.wg_bytes = 8 * g.seg_bytes;
    g.ok = g.ops <= 2;
    return g;
}
// The four workgroups of a row group can also add their slabs themselves: workgroup id = 64 q + r puts them on one XCD
// (ids that differ by a multiple of 8), quarters 1..3 store their slab, wait for the stores and raise a flag, quarter 0
// polls the three flags, reads the three slabs from the XCD's L2 and stores (p0 + p1) + (p2 + p3) over its own: slab 0
// then holds the whole sums and the consumer reads a quarter of the bytes.  Only quarter 0 waits, for workgroups that
// wait for nobody, so no residency is assumed; the wait is bounded and a flag from another XCD is reported (StepCtl.err).
struct DownMSync {
    uint32_t gen[64];            // per row group: launches so far (advanced by its quarter 0 once it has seen the flags)
    uint32_t flags[64][4];       // (epoch << 4 | XCD id) of the quarter's last arrival, epoch = gen + 1
};
struct DownMArgs {
    const uint8_t *w;        // [256][wg_bytes]
    const uint32_t *act;     // [FF / 32][80]
    float *slabs;            // [4][M][E]
    int E, FF;
    DownMSync *sync;         // nullptr: leave four slabs to the consumer
    StepCtl *ctl;
    int spin_limit;
};
#define LG_DOWNM_FIELDS(X, v) X(const uint8_t *, w, w, v) X(const uint32_t *, act, act, v) X(int, E, E, v) X(int, FF, FF, v) X(float *, slabs, slabs, v) \
    X(DownMSync *, sync, sync, v) X(StepCtl *, ctl, ctl, v) X(int, spin_limit, spin_limit, v)
// M: rows of the block; OPS: operands of 32 rows per workgroup; NDP: capacity in pairs of blocks of a segment.
template <int M, int OPS, int NDP>
__global__ __launch_bounds__(512) void lg_k_down_m(LG_DOWNM_FIELDS(LG_XP, _) int p_end_) {
    DownMArgs a; LG_DOWNM_FIELDS(LG_XI, a)
    extern __shared__ __align__(16) unsigned char smem[];
    const DownMGeo g = lg_down_m_geo(a.E, a.FF);
    const int wg = blockIdx.x, r = wg & 63, q = wg >> 6;
    const int t = threadIdx.x, lane = t & 63, n = lane & 31, h = lane >> 5;
    const int s = __builtin_amdgcn_readfirstlane(t >> 6);             // segment 8q + s
    const uint32_t gen = a.sync ? a.sync->gen[r] : 0u;
    unsigned char *la = smem + (size_t)s * g.nitd * (LG_MU_DWORDS * 4);                          // this wavefront's blocks
    float *red = (float *)(smem + (size_t)8 * g.nitd * (LG_MU_DWORDS * 4));                      // [8 segments][OPS][8 row slots][32]
    // the activation blocks of the segment first (they come from nearer), then the whole chain's weights
    const uint4 *src = (const uint4 *)(a.act + (size_t)(8 * q + s) * g.nitd * LG_MU_DWORDS);
    const int nu = g.nitd * (LG_MU_DWORDS / 4);
    const int i0 = min(lane, nu - 1), i1 = min(lane + 64, nu - 1), i2 = min(lane + 128, nu - 1), i3 = min(lane + 192, nu - 1), i4 = min(lane + 256, nu - 1);
    const uint4 t0 = src[i0], t1 = src[i1], t2 = src[i2], t3 = src[i3], t4 = src[i4];                // (up to 16 blocks per segment)
    __builtin_amdgcn_sched_barrier(0);
    struct Pair { lg_x4u q; uint32_t sw; };
    Pair w[OPS][NDP];
    const uint8_t *sb = a.w + (size_t)(4 * r + q) * g.wg_bytes + (size_t)s * g.seg_bytes;
    #pragma unroll
    for (int o = 0; o < OPS; ++o) {
        const int vr = g.RW - 32 * o < 32 ? g.RW - 32 * o : 32, vc = vr > 0 ? vr : 1, nn = n < vc ? n : vc - 1;
        const uint8_t *ob = sb + (size_t)32 * o * g.nitdp * 18;
        #pragma unroll
        for (int jp = 0; jp < NDP; ++jp) {
            const int jc = jp < g.npairs ? jp : g.npairs - 1;
            w[o][jp].q = __builtin_nontemporal_load((const lg_x4u *)(ob + (size_t)((jc * 2 + h) * vc + nn) * 16));
            w[o][jp].sw = __builtin_nontemporal_load((const uint32_t *)(ob + (size_t)g.nitdp * vc * 16 + (size_t)(jc * vc + nn) * 4));
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    ((uint4 *)la)[i0] = t0; ((uint4 *)la)[i1] = t1; ((uint4 *)la)[i2] = t2; ((uint4 *)la)[i3] = t3; ((uint4 *)la)[i4] = t4;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    lg_v16i magic;
    #pragma unroll
    for (int i = 0; i < 16; ++i) magic[i] = 0x4B400000;
    asm volatile("" : "+v"(magic));
    const int arow = n < 8 ? n : 7;
    float p[OPS][4];
    #pragma unroll
    for (int o = 0; o < OPS; ++o)
        #pragma unroll
        for (int i = 0; i < 4; ++i) p[o][i] = 0.0f;
    #pragma unroll
    for (int jp = 0; jp < NDP; ++jp) {
        #pragma unroll
        for (int e = 0; e < 2; ++e) {
            if (2 * jp + e < g.nitd) {
                const XffnAct ac = lg_xffn_act(la + (size_t)(2 * jp + e) * (LG_MU_DWORDS * 4), arow, h);
                #pragma unroll
                for (int o = 0; o < OPS; ++o) {
                    lg_v2u qq; qq.x = e ? w[o][jp].q.z : w[o][jp].q.x; qq.y = e ? w[o][jp].q.w : w[o][jp].q.y;
                    lg_xffn_step(ac.av, ac.xd, ac.cf, qq, lg_h2f((uint16_t)(e ? w[o][jp].sw >> 16 : w[o][jp].sw)), magic, p[o]);
                }
            }
        }
    }
    #pragma unroll
    for (int o = 0; o < OPS; ++o)
        #pragma unroll
        for (int i = 0; i < 4; ++i) red[((size_t)(s * OPS + o) * 8 + 4 * h + i) * 32 + n] = p[o][i];
    __syncthreads();
    // the quarter's three levels of the segment tree: one output per thread (M * RW <= 8 * 64)
    const bool on = t < M * g.RW;
    const int j = on ? t / g.RW : 0, rr = on ? t - j * g.RW : 0;
    float *p0 = a.slabs + (size_t)j * a.E + (size_t)r * g.RW + rr;    // this output in slab 0
    const size_t slab = (size_t)M * a.E;
    float mine = 0.0f;
    if (on) {
        const float *b = red + ((size_t)(rr >> 5) * 8 + j) * 32 + (rr & 31);
        const size_t sg = (size_t)OPS * 8 * 32;
        mine = ((b[0] + b[sg]) + (b[2 * sg] + b[3 * sg])) + ((b[4 * sg] + b[5 * sg]) + (b[6 * sg] + b[7 * sg]));
        p0[q * slab] = mine;
    }
    if (!a.sync) return;
    // ---- the row group's four slabs added here ----
    const int xcc = lg_xcc_id();
    const uint32_t epoch = gen + 1;
    if (q != 0) {
        lg_wait_vm();
        __syncthreads();
        if (t == 0) lg_st_sc<0>(&a.sync->flags[r][q], (epoch << 4) | (uint32_t)xcc);
        return;
    }
    if (s == 0) {
        int err = LG_XFFN_ERR_WAIT;
        for (int spins = 0; spins < a.spin_limit; ++spins) {
            const uint32_t f = (lane >= 1 && lane < 4) ? lg_ld_sc<2>(&a.sync->flags[r][lane]) : ((epoch << 4) | (uint32_t)xcc);
            const bool there = (int)(((f >> 4) - epoch) << 4) >= 0;
            if (__all(there)) { err = __any((int)(f & 15) != xcc) ? LG_XFFN_ERR_PLACE : 0; break; }
        }
        if (err && lane == 0) atomicOr(&a.ctl->err, err);
        if (lane == 0) a.sync->gen[r] = epoch;
    }
    __syncthreads();
    if (on) {
        uint32_t v1, v2, v3;                                          // one round trip for the three
        asm volatile("global_load_dword %0, %1, off sc1" : "=v"(v1) : "v"(p0 + slab) : "memory");
        asm volatile("global_load_dword %0, %1, off sc1" : "=v"(v2) : "v"(p0 + 2 * slab) : "memory");
        asm volatile("global_load_dword %0, %1, off sc1" : "=v"(v3) : "v"(p0 + 3 * slab) : "memory");
        asm volatile("s_waitcnt vmcnt(0)" : "+v"(v1), "+v"(v2), "+v"(v3) :: "memory");
        *p0 = (mine + __uint_as_float(v1)) + (__uint_as_float(v2) + __uint_as_float(v3));
    }
}

// q8 of rows x k floats into the 80-dword blocks (8 lanes per block of 32, one float4 each): what lg_k_geglu_m writes
// in its epilogue, as a kernel of its own for the isolated entry point of lg_k_down_m.
__global__ __launch_bounds__(LG_WG) void lg_k_quant_mu(const float *x, int rows, int k, uint32_t *q) {
    const int g = (blockIdx.x * LG_WG + threadIdx.x) >> 3, l = threadIdx.x & 7, nb = k >> 5;
    const bool live = g < rows * nb;
    const float4 h = live ? ((const float4 *)x)[(size_t)g * 8 + l] : make_float4(0, 0, 0, 0);
    float d; int sum;
    const uint32_t packed = lg_quant4_8lanes(h, &d, &sum);
    if (!live) return;
    const int j = g / nb, b = g - j * nb;
    uint32_t *blk = q + (size_t)b * LG_MU_DWORDS;
    blk[j * 8 + ((l & 1) | ((l & 2) << 1) | ((l & 4) >> 1))] = packed;
    if (l == 0) *(float2 *)(blk + 64 + 2 * j) = make_float2(d, 12582912.0f + (float)(8 * sum));
}
