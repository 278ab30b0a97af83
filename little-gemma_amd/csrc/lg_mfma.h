// lg_mfma.h — the q4_0 x q8 matmul for wide row blocks (prefill), on the matrix cores.
//
// Same arithmetic and the same float order as the wavefront-dot kernels of lg_kernels.h (so a
// prompt processed 32 positions at a time leaves bit-identical cache rows): per 32-weight block an
// exact int32 dot, then p = fma(xd*dw, (float)dot, p) along each of the S contiguous K segments,
// then the adjacent-pair tree over the segments.  What changes is who computes the dots:
// one v_mfma_i32_32x32x32_i8 gives the 32 x 32 block dots of 32 weight rows against 32 activation
// rows for one q4_0 block (K = 32).
//
// Operand roles: A = weights (row m = lane % 32 of the 32-row block, k-half h = lane / 32),
// B = activations (row n = lane % 32 of the row tile, same k-half).  The result register i of lane
// (n, h) is the dot of activation row n with weight row 8*(i/4) + 4*h + i%4.  A lane's 16 k-values
// are, for the weights, the two nibbles of the 8 bytes h*8..h*8+7 of the block (elements
// 8h..8h+7 and 16+8h..16+8h+7), and the same elements of the activation block: any common order
// of the contraction index gives the same integer.
//
// Weights keep the tile layout of lg_device.h.  A workgroup (8 wavefronts, two per SIMD so that the
// float epilogue of one overlaps the loads of the other) owns one 32-row block and 8 K segments:
// per step `it` four of its wavefronts load the block's 256 (row, segment) slots (one 16-byte load
// per lane), park them in LDS in operand order (double buffered, one barrier per step), and every
// wavefront then runs the one segment it owns.  Activations and their {scale, sum} pairs are read
// straight from the q8 activation buffer, which producers of wide blocks write in operand order
// (lg_q8_off: a wavefront's operand load is 512 consecutive bytes).
#pragma once
#include "lg_kernels.h"

typedef int lg_v4i __attribute__((ext_vector_type(4)));
typedef int lg_v16i __attribute__((ext_vector_type(16)));

#define LG_WIDE 32                         // activation rows per row tile (one MFMA operand)
#define LG_WIDE_ROWS 512                   // rows of the widest block: its 16 row tiles share every launch (and every weight tile's trip through L2)
#define LG_WIDE_MID 128                    // the block between that and a single row tile, for prompts and remainders below 512

#define LG_WIDE_WG 512                     // 8 wavefronts: two per SIMD, one K segment each

#ifndef LG_WIDE_U
#define LG_WIDE_U 1
#endif
struct MfmaGeo {
    static constexpr int AW_STRIDE = 33;   // uint2 per (segment, half) row of the operand store (32 + 1 pad)
    static constexpr size_t aw_bytes = (size_t)8 * 2 * AW_STRIDE * 8;
    static constexpr size_t dw_bytes = (size_t)8 * 32 * 4;
    static constexpr int U = LG_WIDE_U;    // steps per chunk: tiles and activation operands are requested a chunk ahead
    static constexpr size_t step_bytes = aw_bytes + dw_bytes;
    static constexpr size_t chunk_bytes = 2 * U * step_bytes;     // double-buffered chunks
    static constexpr size_t lds_bytes = chunk_bytes > 32768 ? chunk_bytes : 32768;   // the final exchange (32 KiB) reuses it
};
static_assert(8 * 16 * 64 * 4 <= MfmaGeo::lds_bytes, "the final exchange must fit");

// One 32-row weight block `rb` against row tile `tile` of the R-row q8 activation buffer, for the 8
// K segments 8*part .. 8*part+7 (S = 8: part = 0 and that is the whole row; S = 32: one quarter, the
// caller adds the four partial results in tree order).  Wavefront w owns segment 8*part + w.
// On return wavefront w, lane (n, h) holds in res[0..1] the finished sums of activation row
// tile*32 + n and weight rows 32*rb + lg_wide_col(w, h) + {0, 1}.  All 512 threads must call it;
// `smem` needs MfmaGeo::lds_bytes and is free again on return.
__device__ __forceinline__ int lg_wide_col(int wave, int h) { return 8 * (wave >> 1) + 4 * h + 2 * (wave & 1); }

// RB: the weights are in row-block tiles (lg_k_geglu_t: tile (64-row block, kb), lane = row) instead of
// the segment tiles of lg_device.h; S must then be 8.
template <int R, int S, bool DUMP, bool RB = false>
__device__ __forceinline__ void lg_mfma_block(const uint8_t *w, int k, int rb, int part, const int8_t *q_in, int tile, int rows,
                                              unsigned char *smem, float (&res)[2], int32_t *dots, int m_total) {
    using G = MfmaGeo;
    constexpr int RW = 64 / S, TPB = 32 / RW;                 // weight rows per tile group; tiles per 32-row block and step
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nb = k >> 5, nit = nb / S;
    const int n = lane & 31, h = lane >> 5, c = 8 * part + wave;
    // operands of row tile `tile` in the wide q8 layout (lg_q8_off): per 16-byte unit the two halves of the
    // 32 rows side by side, so lane (n, h) reads 8 of 512 consecutive bytes; rows past `rows` hold
    // whatever the buffer holds and their results are dropped by the caller.
    // Every load of the loop is a buffer load: a wavefront-uniform base (the row tile, the row block) in scalar
    // registers, a 32-bit lane offset computed once, and the step's offset in a scalar register, so a step spends no
    // vector instructions on addresses.
    const auto rsrc = [](const void *base) { return lg_buffer_rsrc(base); };
    const __amdgpu_buffer_rsrc_t r_act = rsrc(q_in + (size_t)tile * 32 * k);
    const __amdgpu_buffer_rsrc_t r_ds = rsrc(lg_q8_ds<R>(q_in, k) + (size_t)tile * 32 * nb);
    const int vo_a0 = (h * 32 + n) * 8 + c * 512, vo_a1 = vo_a0 + S * 512, vo_d = (c * 32 + n) * 8;

    // wavefronts 0..3 fetch the step's 256 (row, segment) slots: slot -> tile, lane inside the tile, row of the block
    const int slot = (wave & 3) * 64 + lane;
    int st_tile, st_lane, st_m, st_c, vo_w;
    const uint8_t *wbase;
    if (RB) {       // slot = (segment, row): the 32 rows of block rb are lanes 32*(rb&1) .. +31 of tile (rb/2, segment*nit + it)
        st_c = slot >> 5; st_m = slot & 31; st_lane = 32 * (rb & 1) + st_m; st_tile = 0;
        wbase = w + (size_t)(rb >> 1) * nb * LG_TILE;
        vo_w = st_c * nit * LG_TILE;
    } else {
        if (S == 8) { st_tile = slot >> 6; st_lane = slot & 63; st_m = st_tile * 8 + (st_lane >> 3); st_c = st_lane & 7; }
        else        { st_tile = slot >> 4; st_c = slot & 7; const int r = (slot >> 3) & 1; st_lane = r * 32 + 8 * part + st_c; st_m = st_tile * 2 + r; }
        wbase = w + (size_t)rb * TPB * nit * LG_TILE;
        vo_w = st_tile * nit * LG_TILE;
    }
    const __amdgpu_buffer_rsrc_t r_w = rsrc(wbase);
    const int vo_wq = vo_w + st_lane * 16, vo_ws = vo_w + 1024 + st_lane * 2;
    // What a step needs from memory: the lane's slot of the weight tiles (wavefronts 0..3), its 16 operand bytes of
    // the activation block and the block's {scale, sum}.  Two sets, used in turn: step it+1 is requested before the
    // barrier of step it and first waited for after the barrier of step it+1.
    struct Ops { lg_v4i tq; uint32_t ts; uint2 b0, b1; float2 xs; };
    auto fetch = [&](Ops &o, int it_) {
        const int it = __builtin_amdgcn_readfirstlane(it_);   // (uniform: keeps the step offsets in scalar registers)
        if (wave < 4) {
            o.tq = __builtin_amdgcn_raw_buffer_load_b128(r_w, vo_wq, it * LG_TILE, 0);
            o.ts = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(r_w, vo_ws, it * LG_TILE, 0);
        }
        const auto a0 = __builtin_amdgcn_raw_buffer_load_b64(r_act, vo_a0, it * (2 * S * 512), 0);
        const auto a1 = __builtin_amdgcn_raw_buffer_load_b64(r_act, vo_a1, it * (2 * S * 512), 0);
        const auto ds = __builtin_amdgcn_raw_buffer_load_b64(r_ds, vo_d, it * (S * 32 * 8), 0);
        o.b0 = make_uint2((unsigned)a0[0], (unsigned)a0[1]); o.b1 = make_uint2((unsigned)a1[0], (unsigned)a1[1]);
        o.xs = make_float2(__int_as_float(ds[0]), __int_as_float(ds[1]));
    };
    auto park = [&](const Ops &o, unsigned char *cbase) {     // the tile slots into LDS, in operand order
        uint2 *aw = (uint2 *)cbase;
        float *dwf = (float *)(cbase + G::aw_bytes);
        aw[(st_c * 2 + 0) * G::AW_STRIDE + st_m] = make_uint2((unsigned)o.tq[0], (unsigned)o.tq[1]);
        aw[(st_c * 2 + 1) * G::AW_STRIDE + st_m] = make_uint2((unsigned)o.tq[2], (unsigned)o.tq[3]);
        dwf[st_c * 32 + st_m] = lg_h2f((uint16_t)o.ts);
    };
    float p[16];
    #pragma unroll
    for (int i = 0; i < 16; ++i) p[i] = 0.0f;
    lg_v16i magic;
    #pragma unroll
    for (int i = 0; i < 16; ++i) magic[i] = 0x4B400000;      // 12582912.0f
    // kept in 16 registers of its own: left as a known constant the compiler rebuilds it in the accumulator
    // registers before every MFMA (23 moves per step)
    asm volatile("" : "+v"(magic));
    auto compute = [&](const Ops &o, const unsigned char *cbase, int it) {
        const uint2 *aw = (const uint2 *)cbase;
        const float *dwf = (const float *)(cbase + G::aw_bytes);
        // operand and the 16 weight scales of this lane's outputs: all five LDS reads go out together, ahead of the
        // MFMA (interleaved with the epilogue, as the compiler would have them, each costs an LDS round trip)
        const uint2 a = aw[(wave * 2 + h) * G::AW_STRIDE + n];
        float4 d4[4];
        #pragma unroll
        for (int g = 0; g < 4; ++g) d4[g] = *(const float4 *)(dwf + wave * 32 + 8 * g + 4 * h);
        __builtin_amdgcn_sched_barrier(0);
        lg_v4i av, bv;
        av[0] = (int)(a.x & 0x0F0F0F0Fu); av[1] = (int)(a.y & 0x0F0F0F0Fu);
        av[2] = (int)((a.x >> 4) & 0x0F0F0F0Fu); av[3] = (int)((a.y >> 4) & 0x0F0F0F0Fu);
        bv[0] = (int)o.b0.x; bv[1] = (int)o.b0.y; bv[2] = (int)o.b1.x; bv[3] = (int)o.b1.y;
        // The accumulator starts at the bit pattern of 1.5 * 2^23: the integer dot (|dot| < 2^22) lands in the
        // mantissa, so the result read as a float is 12582912 + dot exactly, and one float subtraction of
        // 12582912 + 8*sum gives (float)(dot - 8*sum) exactly: one instruction per output instead of an
        // integer subtract and a conversion.
        const lg_v16i acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, bv, magic, 0, 0, 0);
        const int corr = 8 * __float_as_int(o.xs.y);
        const float cf = 12582912.0f + (float)corr;
        #pragma unroll
        for (int g = 0; g < 4; ++g) {
            const float dv[4] = { d4[g].x, d4[g].y, d4[g].z, d4[g].w };
            #pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float fdot = __int_as_float(acc[4 * g + j]) - cf;
                if (DUMP) {
                    const int row = 32 * rb + 8 * g + 4 * h + j;
                    if (tile * LG_WIDE + n < rows) dots[((size_t)(tile * LG_WIDE + n) * m_total + row) * nb + (c * nit + it)] = (int)fdot;
                }
                p[4 * g + j] = lg_fmaf(o.xs.x * dv[j], fdot, p[4 * g + j]);
            }
        }
    };
    Ops oa, ob;
    unsigned char *const c0 = smem, *const c1 = smem + G::step_bytes;
    fetch(oa, 0);
    int it = 0;
    // (no condition around a fetch inside the loop: with one, the wait for the older set has to assume that the newer
    // one was never requested, and becomes a wait for everything)
    for (; it + 2 < nit; it += 2) {
        if (wave < 4) park(oa, c0);
        fetch(ob, it + 1);
        __syncthreads();
        compute(oa, c0, it);
        if (wave < 4) park(ob, c1);
        fetch(oa, it + 2);
        __syncthreads();
        compute(ob, c1, it + 1);
    }
    if (wave < 4) park(oa, c0);                              // the last one or two steps
    if (it + 1 < nit) fetch(ob, it + 1);
    __syncthreads();
    compute(oa, c0, it);
    if (it + 1 < nit) {
        if (wave < 4) park(ob, c1);
        __syncthreads();
        compute(ob, c1, it + 1);
    }
    // adjacent-pair tree over the eight segments (one per wavefront)
    __syncthreads();
    float *red = (float *)smem;                              // [8 wavefronts][16][64]
    #pragma unroll
    for (int i = 0; i < 16; ++i) red[(wave * 16 + i) * 64 + lane] = p[i];
    __syncthreads();
    #pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int i = 2 * wave + j;
        float v[8];
        #pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = red[(u * 16 + i) * 64 + lane];
        res[j] = ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
    }
    __syncthreads();
}

// Plain matmul for wide blocks: out[row][i] f32.  grid = (m / 32, row tiles, parts): S = 8 has one
// part; S = 32 has four, each writing its own [R][m] slab of `out` (the consumer adds them as
// (p0 + p1) + (p2 + p3), the top of the segment tree).
template <int R, int S, bool DUMP>
__global__ __launch_bounds__(LG_WIDE_WG) void lg_k_mm_wide(MmArgs a, int rows) {
    extern __shared__ __align__(16) unsigned char smem[];
    float res[2];
    lg_mfma_block<R, S, DUMP>(a.w, a.k, blockIdx.x, blockIdx.z, a.q_in, blockIdx.y, rows, smem, res, a.dots, a.m);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, an = blockIdx.y * LG_WIDE + (lane & 31);
    if (an < rows)
        *(float2 *)(a.out + (size_t)blockIdx.z * R * a.m + (size_t)an * a.m + 32 * blockIdx.x + lg_wide_col(wave, lane >> 5)) = make_float2(res[0], res[1]);
}

// 32 x 32 finished values (activation row, column of this workgroup's block) -> one q8 block per
// row, written in the activation order of a consumer of width kq.  vbuf: [32][33] floats in LDS.
template <int R>
__device__ __forceinline__ void lg_wide_quant32(float *vbuf, int8_t *q, int kq, int block, int tile, int rows) {
    const int t = threadIdx.x, n = t >> 3, qd = t & 7, an = tile * LG_WIDE + n;
    if (t >= 256) return;                                    // whole wavefronts leave; the other four stay whole
    const float4 v = make_float4(vbuf[n * 33 + 4 * qd], vbuf[n * 33 + 4 * qd + 1], vbuf[n * 33 + 4 * qd + 2], vbuf[n * 33 + 4 * qd + 3]);
    float d; int sum;
    const uint32_t packed = lg_quant4_8lanes(v, &d, &sum);
    if (an >= rows) return;
    const int quad = block * 8 + qd;
    *(uint32_t *)(q + lg_q8_off<R>(kq, an, quad >> 2, (quad & 3) * 4)) = packed;
    if (qd == 0) lg_q8_ds<R>(q, kq)[lg_q8_ds_idx<R>(kq, an, block)] = make_float2(d, __int_as_float(sum));
}

// Gate/up with the GeGLU and the q8 of its result (see lg_k_geglu_t): row-block tiles, per 32 FFN
// columns a block of 32 gate rows followed by the block of the 32 up rows.  grid = (n_ff/32, row tiles).
template <int R>
__global__ __launch_bounds__(LG_WIDE_WG, 2) void lg_k_mm_geglu_wide(GegluArgs a, int rows) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float vbuf[32 * 33];
    float g[2], u[2];
    lg_mfma_block<R, 8, false, true>(a.w, a.k, 2 * blockIdx.x, 0, a.q_in, blockIdx.y, rows, smem, g, nullptr, 0);
    lg_mfma_block<R, 8, false, true>(a.w, a.k, 2 * blockIdx.x + 1, 0, a.q_in, blockIdx.y, rows, smem, u, nullptr, 0);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n = lane & 31, col = lg_wide_col(wave, lane >> 5);
    #pragma unroll
    for (int j = 0; j < 2; ++j) vbuf[n * 33 + col + j] = lg_gelu(g[j]) * u[j];
    __syncthreads();
    lg_wide_quant32<R>(vbuf, a.gq, a.n_ff, blockIdx.x, blockIdx.y, rows);
}

// PLE gate for wide blocks (see lg_k_mm_plegate): gelu(inp_gate . x) * ipl[layer], q8 of the result.
// grid = (ple/32, row tiles).
template <int R>
__global__ __launch_bounds__(LG_WIDE_WG) void lg_k_mm_plegate_wide(PleGateArgs a, int rows) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float vbuf[32 * 33];
    __shared__ float ipl[32][32];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, ple = a.ple;
    #pragma unroll
    for (int jj = 0; jj < LG_WIDE / (LG_WIDE_WG / 64); ++jj) {
        const int j = wave + jj * (LG_WIDE_WG / 64);
        int an = blockIdx.y * LG_WIDE + j;
        if (an >= rows) an = rows - 1;
        if (lane < 32) ipl[j][lane] = a.ipl[(size_t)an * a.n_layer * ple + (size_t)a.layer * ple + blockIdx.x * 32 + lane];
    }
    float r[2];
    lg_mfma_block<R, 8, false>(a.w, a.k, blockIdx.x, 0, a.q_in, blockIdx.y, rows, smem, r, nullptr, 0);
    const int n = lane & 31, col = lg_wide_col(wave, lane >> 5);
    #pragma unroll
    for (int j = 0; j < 2; ++j) vbuf[n * 33 + col + j] = lg_gelu(r[j]) * ipl[n][col + j];
    __syncthreads();
    lg_wide_quant32<R>(vbuf, a.pq, ple, blockIdx.x, blockIdx.y, rows);
}
