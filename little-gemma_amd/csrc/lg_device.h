// lg_device.h — device-side building blocks of the verify step (gfx950, wave64).
//
// Numeric contract shared with the CPU oracle: every float reduction below has ONE defined
// order, chosen to be natural for a 64-lane wavefront, and every elementary function comes
// from include/lg_math.h.  Integer work (q8 quantization, q4_0 x q8 block dots) is exact.
//   * row sum of squares: 256 lane partials, element i belongs to lane (i/4)%256, fma in
//     ascending i, then an adjacent-pair binary tree over the lanes;
//   * q4_0 x q8 matmul: S contiguous K segments per output (S = 8, or 32 for rows of more than
//     128 blocks), one lane each, serial fma over the segment's blocks, adjacent-pair tree over
//     the S lanes;
//   * attention: 32-key tiles aligned to absolute positions (see lg_kernels.h).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "../../include/lg_math.h"

#define LG_WG        256      // threads per workgroup: 4 wavefronts
#define LG_TILE      1152     // bytes of one weight tile: 64 lanes x 16 B of nibbles + 64 x 2 B of scales
#define LG_TK        32       // keys per attention tile
#define LG_MAXV      16       // float4 per lane of a residual row: n_embd <= 4096
#define LG_HIP_MAX_ROWS_DEV 8   // widest draft block (same value as LG_HIP_MAX_ROWS in lg_hip.h)

// Loads of weight tiles.  The weights of a step (gigabytes) pass through the memory-side cache once per step;
// loaded plainly they push out of it what the step re-reads every time and what fits there: the K/V windows, the
// norm vectors, the PLE gate tiles, the per-layer inputs.  With the non-temporal hint they do not, and the kernels
// that read those (attention tiles, row kernels, PLE gate) run 0.2-0.4 us faster each while the weight kernels
// themselves run no faster: E4B shape, 5 rows, 2.65 -> 2.53 ms per step.  Loading any one large matrix class plainly
// again (ffn_down, or the attention output projection) gives most of that back; the scope bits (sc0 / sc1) on the same
// loads change nothing, and non-temporal stores of kernel outputs gain nothing either.
typedef unsigned lg_ntv4u __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 lg_ldw16(const void *p) {
    const lg_ntv4u v = __builtin_nontemporal_load((const lg_ntv4u *)p);
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint16_t lg_ldw2(const void *p) { return __builtin_nontemporal_load((const uint16_t *)p); }
// Buffer descriptor over memory that starts at a wavefront-uniform address (raw buffer, byte offsets, no bounds
// to speak of): loads through it take the lane's offset in one vector register and a per-load offset in a scalar one.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t lg_buffer_rsrc(const void *base) {
    const uint64_t b = (uint64_t)base;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)b), hi = __builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
    return __builtin_amdgcn_make_buffer_rsrc((void *)(((uint64_t)hi << 32) | lo), 0, 0x7FFFFFFF, 0x00020000);
}
// Tile `it` of a wavefront's run of weight tiles: 16 bytes of nibbles per lane, and the lane's row scale.
__device__ __forceinline__ uint4 lg_ldt16(const uint8_t *base, int it, int lane) { return lg_ldw16(base + (size_t)it * LG_TILE + lane * 16); }
__device__ __forceinline__ uint16_t lg_ldt2(const uint8_t *base, int it, int lane) { return lg_ldw2(base + (size_t)it * LG_TILE + 1024 + lane * 2); }
// The same through a buffer descriptor over the run (lg_buffer_rsrc of its first tile), `it` wavefront-uniform: the
// lane's offset stays in one register for the whole run and the tile's offset travels in a scalar one, where the
// flat form pays 64-bit vector address arithmetic per load.  (The 2 in the last argument is the non-temporal bit.)
// Measured kernel by kernel: the matrix-core gate/up kernel runs 0.15 us faster with these, the small v_dot4
// kernels (qkv, attention output) 0.3 us slower, so only the former uses them.
__device__ __forceinline__ uint4 lg_ldt16b(__amdgpu_buffer_rsrc_t r, int it, int lane) {
    const auto v = __builtin_amdgcn_raw_buffer_load_b128(r, lane * 16, __builtin_amdgcn_readfirstlane(it) * LG_TILE, 2);
    return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ uint16_t lg_ldt2b(__amdgpu_buffer_rsrc_t r, int it, int lane) {
    return (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(r, 1024 + lane * 2, __builtin_amdgcn_readfirstlane(it) * LG_TILE, 2);
}

// Weight tile order (built on the host by lg_hip_repack_q4_0): a row of k/32 q4_0 blocks is cut
// into S contiguous segments of nit blocks (S = lg_segments(k): 8, or 32 for rows of more than 128
// blocks); the m x k matrix is cut into groups of 64/S rows; tile (group, it) holds, for
// lane = r*S + c, the 16 nibble bytes and the f16 scale of block c*nit + it of row r of the group.
// A wavefront reads one tile with one 16-byte load and one 2-byte load per lane.
// (a long row whose block count is no multiple of 32, like the 2 x 3840 inputs of a draft head's pre-projection on a 3840-wide
// backbone, keeps 8 segments)
__host__ __device__ static inline int lg_segments(int k) { return ((k >> 5) > 128 && ((k >> 5) & 31) == 0) ? 32 : 8; }

// Order of a q8 activation row in memory.  A matmul lane (row r, segment c) needs, at step `it`,
// block c*nit + it of the row; lanes c = 0..S-1 therefore want blocks that lie nit apart.  Rows are
// stored so that these are neighbours: the 16-byte unit w of the natural order (block b = w/2, half
// = w%2) lives at unit it*2S + half*S + c, and the block's {scale,sum} pair at it*S + c, with
// c = b / nit, it = b % nit.  A wavefront's LDS reads are then consecutive 16-byte units (no bank
// conflicts), and producers write this order directly.
// b / nit is taken as (b * inv) >> 16 with inv = 65536 / nit + 1: exact for b < 65536 / nit (a row has at most
// a few hundred blocks), and two instructions per lane where a division by a run-time value costs about
// fifteen; the layout itself is wavefront-uniform, so its own division runs on the scalar unit.
struct ActLayout { int S, nit; unsigned inv; };
__host__ __device__ static inline ActLayout lg_act_layout(int k) {
    const int S = lg_segments(k), nit = (k >> 5) / S;
    return { S, nit, 65536u / (unsigned)nit + 1u };
}
__host__ __device__ static inline int lg_act_seg(ActLayout a, int b) { return (int)(((unsigned)b * a.inv) >> 16); }
__host__ __device__ static inline int lg_act_unit(ActLayout a, int w) {
    const int b = w >> 1, c = lg_act_seg(a, b), it = b - c * a.nit;
    return it * 2 * a.S + (w & 1) * a.S + c;
}
__host__ __device__ static inline int lg_act_block(ActLayout a, int b) {
    const int c = lg_act_seg(a, b), it = b - c * a.nit;
    return it * a.S + c;
}

// Cross-lane exchange for the reductions.  Within a row of 16 lanes DPP moves data in one VALU
// instruction; the partner patterns (swap inside pairs, swap pairs inside quads, mirror 8, mirror
// 16) differ from xor-butterflies only in which lane of the already-uniform sub-group supplies the
// value, so sums come out in the same adjacent-pair tree order (addition is commutative) and
// max / integer sums are order-free anyway.
template <int CTRL>
__device__ __forceinline__ float lg_dpp_f(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, false));
}
template <int CTRL>
__device__ __forceinline__ int lg_dpp_i(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, false);
}
#define LG_DPP_SWAP1   0xB1     // quad_perm [1,0,3,2]
#define LG_DPP_SWAP2   0x4E     // quad_perm [2,3,0,1]
#define LG_DPP_MIRROR8 0x141    // row_half_mirror
#define LG_DPP_MIRROR16 0x140   // row_mirror

__device__ __forceinline__ float lg_sum8(float v) {
    v = v + lg_dpp_f<LG_DPP_SWAP1>(v);
    v = v + lg_dpp_f<LG_DPP_SWAP2>(v);
    v = v + lg_dpp_f<LG_DPP_MIRROR8>(v);
    return v;
}
__device__ __forceinline__ float lg_sum16(float v) {
    v = lg_sum8(v);
    v = v + lg_dpp_f<LG_DPP_MIRROR16>(v);
    return v;
}
// Lane l and lane l^16 (l^32): v_permlane16_swap (v_permlane32_swap) with the value as both operands leaves
// the even rows (the lower half) in one result and the odd rows (the upper half) in the other, each in every
// lane of the pair; combining the two results gives v[l] (+) v[l^16] in one VALU step, where a shuffle through
// the LDS crossbar costs an LDS round trip.  The combination is commutative, so the order of the pair is free.
typedef unsigned lg_u2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ lg_u2 lg_pair16(uint32_t v) { return __builtin_amdgcn_permlane16_swap(v, v, false, false); }
__device__ __forceinline__ lg_u2 lg_pair32(uint32_t v) { return __builtin_amdgcn_permlane32_swap(v, v, false, false); }
__device__ __forceinline__ float lg_add_x16(float v) { const lg_u2 r = lg_pair16(__float_as_uint(v)); return __uint_as_float(r.x) + __uint_as_float(r.y); }
__device__ __forceinline__ float lg_add_x32(float v) { const lg_u2 r = lg_pair32(__float_as_uint(v)); return __uint_as_float(r.x) + __uint_as_float(r.y); }
__device__ __forceinline__ float lg_sum32(float v) {
    v = lg_sum16(v);
    return lg_add_x16(v);
}
__device__ __forceinline__ float lg_wave_sum64(float v) {
    v = lg_sum32(v);
    return lg_add_x32(v);
}
template <int S>
__device__ __forceinline__ float lg_sum_seg(float v) {       // S = 8 or 32 adjacent lanes
    if (S == 8) return lg_sum8(v);
    return lg_sum32(v);
}
__device__ __forceinline__ float lg_max8(float v) {
    v = fmaxf(v, lg_dpp_f<LG_DPP_SWAP1>(v));
    v = fmaxf(v, lg_dpp_f<LG_DPP_SWAP2>(v));
    v = fmaxf(v, lg_dpp_f<LG_DPP_MIRROR8>(v));
    return v;
}
__device__ __forceinline__ float lg_max_n(float v, int n) {       // n = 8, 32 or 64 lanes
    v = lg_max8(v);
    if (n >= 16) v = fmaxf(v, lg_dpp_f<LG_DPP_MIRROR16>(v));
    if (n >= 32) { const lg_u2 r = lg_pair16(__float_as_uint(v)); v = fmaxf(__uint_as_float(r.x), __uint_as_float(r.y)); }
    if (n >= 64) { const lg_u2 r = lg_pair32(__float_as_uint(v)); v = fmaxf(__uint_as_float(r.x), __uint_as_float(r.y)); }
    return v;
}
__device__ __forceinline__ int lg_isum_n(int v, int n) {          // n = 8 or 32 lanes
    v += lg_dpp_i<LG_DPP_SWAP1>(v);
    v += lg_dpp_i<LG_DPP_SWAP2>(v);
    v += lg_dpp_i<LG_DPP_MIRROR8>(v);
    if (n >= 16) v += lg_dpp_i<LG_DPP_MIRROR16>(v);
    if (n >= 32) { const lg_u2 r = lg_pair16((uint32_t)v); v = (int)r.x + (int)r.y; }
    return v;
}

__device__ __forceinline__ float lg_sumsq4(float4 v, float acc) {
    acc = lg_fmaf(v.x, v.x, acc);
    acc = lg_fmaf(v.y, v.y, acc);
    acc = lg_fmaf(v.z, v.z, acc);
    acc = lg_fmaf(v.w, v.w, acc);
    return acc;
}

// amax / 127.0f for amax >= 0, in three instructions: with r = the float nearest to 1/127, q0 = amax * r,
// the residual amax - 127*q0 is exact in one fma and the corrected quotient fma(residual, r, q0) equals the
// correctly rounded IEEE quotient for every non-negative finite float (checked exhaustively on a CPU, all
// 2,139,095,040 of them, subnormals included); the generic division sequence costs about ten instructions.
__device__ __forceinline__ float lg_div127(float amax) {
    const float r = 1.0f / 127.0f;
    const float q0 = amax * r;
    return lg_fmaf(lg_fmaf(-127.0f, q0, amax), r, q0);
}

// q8 quantization of 32 consecutive values held as one float4 in each of 8 adjacent lanes:
// amax, d = amax/127, id = 1/d (0 when d == 0), q = rint_even(x*id), sum of q.
// Returns the 4 packed int8; *d_out / *sum_out are the same in all 8 lanes.
__device__ __forceinline__ uint32_t lg_quant4_8lanes(float4 h, float *d_out, int *sum_out) {
    float amax = fmaxf(fmaxf(fabsf(h.x), fabsf(h.y)), fmaxf(fabsf(h.z), fabsf(h.w)));
    amax = lg_max_n(amax, 8);
    const float d = lg_div127(amax);
    const float id = d > 0.0f ? 1.0f / d : 0.0f;
    const int q0 = (int)lg_rintf(h.x * id), q1 = (int)lg_rintf(h.y * id);
    const int q2 = (int)lg_rintf(h.z * id), q3 = (int)lg_rintf(h.w * id);
    *d_out = d;
    *sum_out = lg_isum_n(q0 + q1 + q2 + q3, 8);
    return (uint32_t)(q0 & 255) | ((uint32_t)(q1 & 255) << 8) | ((uint32_t)(q2 & 255) << 16) | ((uint32_t)(q3 & 255) << 24);
}

// Same for 32 values held one per lane in 32 adjacent lanes (half a wavefront).
__device__ __forceinline__ int lg_quant1_32lanes(float h, float *d_out, int *sum_out) {
    const float amax = lg_max_n(fabsf(h), 32);
    const float d = lg_div127(amax);
    const float id = d > 0.0f ? 1.0f / d : 0.0f;
    const int q = (int)lg_rintf(h * id);
    *d_out = d;
    *sum_out = lg_isum_n(q, 32);
    return q;
}

__device__ __forceinline__ float lg_h2f(uint16_t h) {
    return __half2float(__ushort_as_half(h));
}
__device__ __forceinline__ uint16_t lg_f2h(float f) {
    // The value converted is the binary32 one.  Without the barrier the compiler folds a multiply that produced f
    // into one multiply-and-convert instruction (v_fma_mixlo_f16), which rounds once instead of twice and differs
    // from the stored-then-converted value in rare tie cases.
    asm("" : "+v"(f));
    return __half_as_ushort(__float2half_rn(f));
}

// Four consecutive elements (e0 % 4 == 0) of row `row` of a tiled q4_0 matrix, dequantized.
__device__ __forceinline__ float4 lg_tiled_deq4(const uint8_t *w, int nit, int S, int row, int e0) {
    const int b = e0 >> 5, o = e0 & 31, rw = 64 / S;
    const int c = b / nit, it = b - c * nit;
    const uint8_t *tile = w + ((size_t)(row / rw) * nit + it) * LG_TILE;
    const int slot = (row % rw) * S + c;
    const uint32_t qs = *(const uint32_t *)(tile + slot * 16 + (o & 15));
    const float d = lg_h2f(*(const uint16_t *)(tile + 1024 + slot * 2));
    const uint32_t nib = (o & 16) ? (qs >> 4) : qs;
    float4 r;
    r.x = d * (float)((int)(nib & 15) - 8);
    r.y = d * (float)((int)((nib >> 8) & 15) - 8);
    r.z = d * (float)((int)((nib >> 16) & 15) - 8);
    r.w = d * (float)((int)((nib >> 24) & 15) - 8);
    return r;
}

// One element of a q4_0 row in plain GGUF order (18-byte blocks).
__device__ __forceinline__ float lg_q4_0_elem(const uint8_t *row, int e) {
    const uint8_t *blk = row + (size_t)(e >> 5) * 18;
    const float d = lg_h2f((uint16_t)(blk[0] | (blk[1] << 8)));
    const int o = e & 31;
    const int nib = (o & 16) ? (blk[2 + (o & 15)] >> 4) : (blk[2 + o] & 15);
    return d * (float)(nib - 8);
}

// Inner product of one weight tile lane (16 nibble bytes = one q4_0 block) with the 32 int8 of
// an activation block: sum(c*q) - 8*sum(q) == sum((c-8)*q), exact in int32.
__device__ __forceinline__ int lg_block_dot(uint4 wq, int4 a0, int4 a1, int act_sum) {
    int dot = -8 * act_sum;                                   // starts the accumulator: one multiply instead of a move and a subtract
    dot = __builtin_amdgcn_sdot4((int)(wq.x & 0x0F0F0F0Fu), a0.x, dot, false);
    dot = __builtin_amdgcn_sdot4((int)(wq.y & 0x0F0F0F0Fu), a0.y, dot, false);
    dot = __builtin_amdgcn_sdot4((int)(wq.z & 0x0F0F0F0Fu), a0.z, dot, false);
    dot = __builtin_amdgcn_sdot4((int)(wq.w & 0x0F0F0F0Fu), a0.w, dot, false);
    dot = __builtin_amdgcn_sdot4((int)((wq.x >> 4) & 0x0F0F0F0Fu), a1.x, dot, false);
    dot = __builtin_amdgcn_sdot4((int)((wq.y >> 4) & 0x0F0F0F0Fu), a1.y, dot, false);
    dot = __builtin_amdgcn_sdot4((int)((wq.z >> 4) & 0x0F0F0F0Fu), a1.z, dot, false);
    dot = __builtin_amdgcn_sdot4((int)((wq.w >> 4) & 0x0F0F0F0Fu), a1.w, dot, false);
    return dot;
}
