// lg_xcd.h — cooperation between the workgroups of one XCD (gfx950: 8 XCDs of 32 CUs, one L2 per XCD).
//
// A kernel boundary is the cheapest synchronisation of the WHOLE chip, but it is paid by every hand-over of a
// layer, also by those that only a few dozen workgroups take part in.  The workgroups of one XCD share an L2:
// what one of them has stored (vector stores write through the CU's L1 into that L2) another can load without
// any cache maintenance, provided its load does not hit its own CU's L1.  So a hand-over inside an XCD is
//   producer:  stores ... ; s_waitcnt vmcnt(0) ; barrier ; one lane stores the workgroup's flag
//   consumer:  lanes poll the flags of the group with L1-bypassing loads ; barrier ; L1-bypassing loads of the data
// with no fence, no write-back and no invalidate.  The dispatcher deals the workgroups of a launch to the XCDs in
// turn, going on where the previous launch stopped: the workgroups i with the same i % 8 run on one XCD (which
// lg_hip_xcd_map measures), but which XCD that is differs from launch to launch.  A kernel that relies on it puts
// its XCD id register into every flag it raises, and a reader that sees another id than its own reports it
// instead of computing with stale data.
//
// Scope of an access (gfx942/gfx950 sc bits): 0 = plain, 1 = sc0 (workgroup), 2 = sc1 (agent), 3 = sc0 sc1 (system).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define LG_XCDS 8                 // XCDs of the chip
#define LG_XCD_WGS 32             // workgroups of one launch per XCD when the launch has one per CU

__device__ __forceinline__ int lg_xcc_id() {
    int x;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(x));
    return x & 15;
}
__device__ __forceinline__ uint32_t lg_hw_id() {
    uint32_t h;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(h));
    return h;
}
__device__ __forceinline__ void lg_wait_vm() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

template <int SC>
__device__ __forceinline__ uint32_t lg_ld_sc(const uint32_t *p) {
    uint32_t v;
    if (SC == 0)      asm volatile("global_load_dword %0, %1, off\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
    else if (SC == 1) asm volatile("global_load_dword %0, %1, off sc0\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
    else if (SC == 2) asm volatile("global_load_dword %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
    else              asm volatile("global_load_dword %0, %1, off sc0 sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
    return v;
}
template <int SC>
__device__ __forceinline__ void lg_st_sc(uint32_t *p, uint32_t v) {
    if (SC == 0)      asm volatile("global_store_dword %0, %1, off" :: "v"(p), "v"(v) : "memory");
    else if (SC == 1) asm volatile("global_store_dword %0, %1, off sc0" :: "v"(p), "v"(v) : "memory");
    else if (SC == 2) asm volatile("global_store_dword %0, %1, off sc1" :: "v"(p), "v"(v) : "memory");
    else              asm volatile("global_store_dword %0, %1, off sc0 sc1" :: "v"(p), "v"(v) : "memory");
}

// 16-byte loads of a scope that are requested without waiting; lg_ld4_wait makes the values usable (the registers
// pass through the wait, so no use of them can be scheduled ahead of it).
typedef unsigned lg_x4u __attribute__((ext_vector_type(4)));     // a native 128-bit register operand
template <int SC>
__device__ __forceinline__ lg_x4u lg_ld4_sc_issue(const void *p) {
    lg_x4u v;
    if (SC == 0)      asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(v) : "v"(p) : "memory");
    else if (SC == 1) asm volatile("global_load_dwordx4 %0, %1, off sc0" : "=v"(v) : "v"(p) : "memory");
    else if (SC == 2) asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v) : "v"(p) : "memory");
    else              asm volatile("global_load_dwordx4 %0, %1, off sc0 sc1" : "=v"(v) : "v"(p) : "memory");
    return v;
}
__device__ __forceinline__ void lg_ld4_wait(lg_x4u &a, lg_x4u &b, lg_x4u &c, lg_x4u &d) {
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) :: "memory");
}
template <int SC>
__device__ __forceinline__ void lg_st4_sc(void *p, lg_x4u v) {
    if (SC == 0)      asm volatile("global_store_dwordx4 %0, %1, off" :: "v"(p), "v"(v) : "memory");
    else if (SC == 1) asm volatile("global_store_dwordx4 %0, %1, off sc0" :: "v"(p), "v"(v) : "memory");
    else if (SC == 2) asm volatile("global_store_dwordx4 %0, %1, off sc1" :: "v"(p), "v"(v) : "memory");
    else              asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" :: "v"(p), "v"(v) : "memory");
}

// ---- probes -------------------------------------------------------------------------------------------------
// A hand-over among the n workgroups of a group, `rounds` times: every member stores `words` dwords (its rank and the
// round), waits for its stores, raises its flag; every member then polls the n flags (lane i of its first wavefront
// polls flag i, a bounded number of times) and reads its neighbour's words back, counting the ones that are not
// what the neighbour wrote in this round.  set_mode 0: the group is the workgroups i with i % 8 == sel (one XCD
// when workgroups are dealt to the XCDs in turn), rank i / 8; set_mode 1: the workgroups sel*n .. sel*n + n - 1
// (n consecutive ones: spread over all XCDs).  Every other workgroup of the launch leaves at once.
// Buffers are used in turn (round & 1): a member cannot be two rounds ahead of one that still reads.
// res[rank] = { ticks of s_memrealtime over the rounds, mismatching words, polls given up, XCD id }.
struct XcdProbeArgs {
    uint32_t *flags;        // [n], zero on entry
    uint32_t *data;         // [2][n][words]
    int32_t  *res;          // [n][4]
    int n, words, rounds, set_mode, sel, spin_limit;
};
template <int ST, int LD>
__global__ __launch_bounds__(256) void lg_k_xcd_handover(XcdProbeArgs a) {
    const int wg = blockIdx.x;
    int rank;
    if (a.set_mode == 0) { if (wg % LG_XCDS != a.sel || wg / LG_XCDS >= a.n) return; rank = wg / LG_XCDS; }
    else { if (wg < a.sel * a.n || wg >= (a.sel + 1) * a.n) return; rank = wg - a.sel * a.n; }
    __shared__ int s_bad, s_lost;
    if (threadIdx.x == 0) { s_bad = 0; s_lost = 0; }
    __syncthreads();
    const int nb = (rank + 1) % a.n;
    long long t0 = 0;
    int bad = 0, lost = 0;
    for (int r = 1; r <= a.rounds + 1; ++r) {               // round 1 warms up and is not timed
        if (r == 2 && threadIdx.x == 0) t0 = wall_clock64();
        uint32_t *mine = a.data + ((size_t)(r & 1) * a.n + rank) * a.words;
        for (int i = threadIdx.x; i < (a.words >> 2); i += blockDim.x) {
            const uint32_t w = ((uint32_t)r << 16) | ((uint32_t)rank << 8) | (uint32_t)(i & 255);
            lg_st4_sc<ST>(mine + 4 * i, lg_x4u{ w, w + 0x1000000u, w + 0x2000000u, w + 0x3000000u });
        }
        lg_wait_vm();
        __syncthreads();
        if (threadIdx.x == 0) lg_st_sc<ST>(a.flags + rank, (uint32_t)r);
        if (threadIdx.x < 64) {
            const int lane = threadIdx.x;
            int spins = 0;
            for (;;) {
                const uint32_t f = lane < a.n ? lg_ld_sc<LD>(a.flags + lane) : (uint32_t)r;
                const bool ok = (int)(f - (uint32_t)r) >= 0;
                if (__all(ok)) break;
                if (++spins >= a.spin_limit) { if (!ok) lost++; break; }
            }
        }
        __syncthreads();
        const uint32_t *theirs = a.data + ((size_t)(r & 1) * a.n + nb) * a.words;
        const int nq = a.words >> 2;                          // 16-byte units, four per thread in flight
        for (int i0 = threadIdx.x; i0 < nq; i0 += 4 * blockDim.x) {
            const int i1 = min(i0 + (int)blockDim.x, nq - 1), i2 = min(i0 + 2 * (int)blockDim.x, nq - 1), i3 = min(i0 + 3 * (int)blockDim.x, nq - 1);
            lg_x4u v0 = lg_ld4_sc_issue<LD>(theirs + 4 * i0), v1 = lg_ld4_sc_issue<LD>(theirs + 4 * i1);
            lg_x4u v2 = lg_ld4_sc_issue<LD>(theirs + 4 * i2), v3 = lg_ld4_sc_issue<LD>(theirs + 4 * i3);
            lg_ld4_wait(v0, v1, v2, v3);
            const uint32_t tag = ((uint32_t)r << 16) | ((uint32_t)nb << 8);
            auto wrong = [&](lg_x4u v, int i) {
                const uint32_t w = tag | (uint32_t)(i & 255);
                return (int)(v.x != w) + (int)(v.y != w + 0x1000000u) + (int)(v.z != w + 0x2000000u) + (int)(v.w != w + 0x3000000u);
            };
            bad += wrong(v0, i0) + wrong(v1, i1) + wrong(v2, i2) + wrong(v3, i3);
        }
    }
    const long long t1 = wall_clock64();
    if (bad) atomicAdd(&s_bad, bad);
    if (lost) atomicAdd(&s_lost, lost);
    __syncthreads();
    if (threadIdx.x == 0) {
        a.res[rank * 4 + 0] = (int32_t)(t1 - t0);
        a.res[rank * 4 + 1] = s_bad;
        a.res[rank * 4 + 2] = s_lost;
        a.res[rank * 4 + 3] = lg_xcc_id();
    }
}
