// lg_kernels.h — the kernels of one verify step (rows = M draft-block rows, M <= 8).
//
// One step is a graph of small kernels; a dependent kernel boundary costs ~1.5 us on MI355X, an
// all-CU software barrier ten times that, so the step is NOT a persistent megakernel.  Per layer:
//   rows(norm+q8) -> qkv -> qkv_post(norm,rope,KV write) -> attn tiles -> attn merge(+q8) -> o
//   -> rows -> gate/up+GeGLU(+q8) -> down -> rows+ple gate(+q8) -> ple proj
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
// Kernel arguments are passed one by one, not as a struct: the first dozen dwords of a kernel's arguments can be
// handed to its wavefronts in scalar registers at launch (-amdgpu-kernarg-preload-count), which a struct passed by
// value is not, and a kernel whose first loads need only those starts them without waiting for a load of its
// arguments.  Each argument struct lists its fields once, most urgent first (LG_*_FIELDS: type, parameter name,
// member); the lists expand to the kernel's parameters (LG_XP), to the arguments of a launch (LG_XA) and to the
// struct's reassembly inside the kernel (LG_XI), so the kernel bodies and the host code keep using the structs.
#define LG_XP(T, id, mem, v) T p_##id,
#define LG_XA(T, id, mem, v) (v).mem,
#define LG_XI(T, id, mem, v) (v).mem = p_##id;

struct RowArgs {
    const float   *x;        // [M][E] residual stream; nullptr when the rows are embeddings
    const float   *dout;     // [M][E] previous sub-layer output to be rmsnormed and added, or nullptr
    int            dparts;   // 4: dout is four [M][E] slabs of partial sums, added here as (p0+p1)+(p2+p3); else 1
    const float   *w_post;   // [E] norm weight for dout
    const float   *os;       // scalar layer_output_scale applied after the add, or nullptr
    float         *x_out;    // [M][E] updated residual, or nullptr
    const float   *w_pre;    // [E] norm weight applied before quantization, or nullptr (quantize x itself)
    float         *h_out;    // [M][E] normed rows before quantization, or nullptr
    const uint8_t *emb;      // tiled token_embd: rows are token lookups scaled by emb_scale
    const int32_t *toks;     // token schedule base ([n_steps][M])
    int8_t        *q;        // q8 activation buffer: [M][E] values, then [M][E/32] {scale, sum}
    int            q_units;  // write q in a block-major order instead (M <= 8 only): 1 = units of lg_k_geglu_t, 2 = blocks of lg_k_geglu_m
    int            emb_nit, emb_seg;
    float          emb_scale;
    int            E;
    float          eps;
    int            slices;   // workgroups per row (gridDim.y): as an argument it arrives with the others, the launch dimensions need a load of their own
    uint32_t      *bump;     // nullptr, or a counter that the launch advances by LG_RG_STEP (the step's first kernel: epochs of lg_k_rows_geglu)
};
#define LG_RG_STEP 256       // more than the launches of a step
#define LG_ROW_FIELDS(X, v) X(const float *, x, x, v) X(const float *, dout, dout, v) X(const float *, w_post, w_post, v) X(const float *, w_pre, w_pre, v) X(int, E, E, v) X(int, dparts, dparts, v) X(int, slices, slices, v) X(const float *, os, os, v) X(float *, x_out, x_out, v) X(float *, h_out, h_out, v) X(int8_t *, q, q, v) X(int, q_units, q_units, v) X(float, eps, eps, v) X(const uint8_t *, emb, emb, v) X(const int32_t *, toks, toks, v) X(int, emb_nit, emb_nit, v) X(int, emb_seg, emb_seg, v) X(float, emb_scale, emb_scale, v) X(uint32_t *, bump, bump, v)

// Sum over the 256 lanes of a workgroup in adjacent-pair tree order; every thread gets the result.
// `scratch4` must not be in use by an earlier call that other wavefronts may still be reading: each call
// site has its own four floats, so one barrier is enough.
__device__ __forceinline__ float lg_block_sum256(float v, float *scratch4) {
    v = lg_wave_sum64(v);
    if ((threadIdx.x & 63) == 0) scratch4[threadIdx.x >> 6] = v;
    __syncthreads();
    return (scratch4[0] + scratch4[1]) + (scratch4[2] + scratch4[3]);
}

// A q8 activation buffer holds the M rows of int8 values ([M][k], order of lg_act_layout(k))
// immediately followed by their per-32 {scale, sum} pairs ([M][k/32] float2): one contiguous
// region of M*k*5/4 bytes, copied to LDS in one go.
template <int M>
__device__ __forceinline__ const float2 *lg_q8_ds(const int8_t *q, int k) { return (const float2 *)(q + (size_t)M * k); }
template <int M>
__device__ __forceinline__ float2 *lg_q8_ds(int8_t *q, int k) { return (float2 *)(q + (size_t)M * k); }
// Where row j keeps byte `byte` of its natural 16-byte unit w, and the {scale, sum} pair of block b.
// Blocks of up to LG_HIP_MAX_ROWS_DEV rows: row-major rows in the order of lg_act_layout (what the
// wavefront-dot kernels stage in LDS).  Wider blocks (the matrix-core kernels): tiles of 32 rows, and
// inside a tile the 8-byte halves of a unit of all 32 rows side by side, so that the 64 lanes of an
// operand load (row n = lane % 32, half = lane / 32) read 512 consecutive bytes.
template <int M>
__device__ __forceinline__ size_t lg_q8_off(int k, int j, int w, int byte) {
    const int u = lg_act_unit(lg_act_layout(k), w);
    if (M <= LG_HIP_MAX_ROWS_DEV) return (size_t)j * k + (size_t)u * 16 + byte;
    return (size_t)(j >> 5) * 32 * k + ((size_t)(u * 2 + (byte >> 3)) * 32 + (j & 31)) * 8 + (byte & 7);
}
template <int M>
__device__ __forceinline__ size_t lg_q8_ds_idx(int k, int j, int b) {
    const int u = lg_act_block(lg_act_layout(k), b);
    if (M <= LG_HIP_MAX_ROWS_DEV) return (size_t)j * (k >> 5) + u;
    return (size_t)(j >> 5) * 32 * (k >> 5) + (size_t)u * 32 + (j & 31);
}
#define LG_MU_DWORDS 80                     // dwords per block of the lg_k_geglu_m activation order
#define LG_ROWV ((LG_MAXV + 3) / 4)        // float4 per thread of a residual row, 256 threads per row
template <int M>
__global__ __launch_bounds__(LG_WG) void lg_k_rows(const StepCtl *ctl, LG_ROW_FIELDS(LG_XP, _) int p_end_) {
    RowArgs s; LG_ROW_FIELDS(LG_XI, s)
    __shared__ float red[2][4];
    const int t = threadIdx.x, j = blockIdx.x;
    // gridDim.y > 1: every workgroup of a row forms the row's sums, workgroup y stores and quantizes only the
    // float4 t + 256*y of each lane (the tail of the kernel is the longest part of it and splits freely)
    const int vs = s.slices > 1 ? (int)blockIdx.y : -1;
    const int E = s.E, nq = E >> 2;                          // float4 quads in a row; thread t owns quads t + 256*v
    if (s.bump && blockIdx.x == 0 && blockIdx.y == 0 && t == 0) *s.bump += LG_RG_STEP;
    float4 xv[LG_ROWV], dv[LG_ROWV], wpost[LG_ROWV], wpre[LG_ROWV];
    // issue every load up front: one memory round trip for the whole row
    if (!s.x) {                                              // (rows that are token lookups have no residual yet)
        const int tok = s.toks[ctl->step * M + j];
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) {
            const float4 e = lg_tiled_deq4(s.emb, s.emb_nit, s.emb_seg, tok, 4 * (t + 256 * v));
            xv[v] = make_float4(e.x * s.emb_scale, e.y * s.emb_scale, e.z * s.emb_scale, e.w * s.emb_scale);
        }
    } else {
        const float4 *xr = (const float4 *)(s.x + (size_t)j * E);
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) xv[v] = xr[t + 256 * v];
    }
    const bool has_os = s.dout != nullptr && s.os != nullptr;
    const float osv = has_os ? s.os[0] : 1.0f;               // (requested with the rows, not after the first sum)
    if (s.dout) {
        const float4 *dr = (const float4 *)(s.dout + (size_t)j * E), *wr = (const float4 *)s.w_post;
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) { dv[v] = dr[t + 256 * v]; wpost[v] = wr[t + 256 * v]; }
        if (s.dparts == 8) {                                 // ... over the 8 XCDs: the top three levels of the tree
            const size_t slab = (size_t)M * nq;
            #pragma unroll
            for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) {
                const float4 *b = dr + t + 256 * v;
                const float4 p1 = b[slab], p2 = b[2 * slab], p3 = b[3 * slab], p4 = b[4 * slab], p5 = b[5 * slab], p6 = b[6 * slab], p7 = b[7 * slab], p0 = dv[v];
                dv[v] = make_float4(((p0.x + p1.x) + (p2.x + p3.x)) + ((p4.x + p5.x) + (p6.x + p7.x)), ((p0.y + p1.y) + (p2.y + p3.y)) + ((p4.y + p5.y) + (p6.y + p7.y)),
                                    ((p0.z + p1.z) + (p2.z + p3.z)) + ((p4.z + p5.z) + (p6.z + p7.z)), ((p0.w + p1.w) + (p2.w + p3.w)) + ((p4.w + p5.w) + (p6.w + p7.w)));
            }
        }
        if (s.dparts == 4) {                                 // top of the K-segment tree of a matmul that was split over four workgroups
            const size_t slab = (size_t)M * nq;
            #pragma unroll
            for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) {
                const float4 p1 = dr[slab + t + 256 * v], p2 = dr[2 * slab + t + 256 * v], p3 = dr[3 * slab + t + 256 * v], p0 = dv[v];
                dv[v] = make_float4((p0.x + p1.x) + (p2.x + p3.x), (p0.y + p1.y) + (p2.y + p3.y),
                                    (p0.z + p1.z) + (p2.z + p3.z), (p0.w + p1.w) + (p2.w + p3.w));
            }
        }
    }
    if (s.w_pre) {
        const float4 *wr = (const float4 *)s.w_pre;
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) wpre[v] = wr[t + 256 * v];
    }
    if (s.dout) {
        float ss = 0.0f;
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) ss = lg_sumsq4(dv[v], ss);
        ss = lg_block_sum256(ss, red[0]);
        const float sc = 1.0f / sqrtf(ss / (float)E + s.eps);
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) {
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
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq && (vs < 0 || v == vs)) xo[t + 256 * v] = xv[v];
    }
    if (s.w_pre) {
        float ss = 0.0f;
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) ss = lg_sumsq4(xv[v], ss);
        ss = lg_block_sum256(ss, red[1]);
        const float sc = 1.0f / sqrtf(ss / (float)E + s.eps);
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) {
            const float4 w = wpre[v];
            xv[v] = make_float4(xv[v].x * sc * w.x, xv[v].y * sc * w.y, xv[v].z * sc * w.z, xv[v].w * sc * w.w);
        }
    }
    if (s.h_out) {
        float4 *ho = (float4 *)(s.h_out + (size_t)j * E);
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq && (vs < 0 || v == vs)) ho[t + 256 * v] = xv[v];
    }
    float2 *dsb = lg_q8_ds<M>(s.q, E);
    #pragma unroll
    for (int v = 0; v < LG_ROWV; ++v) {
        // nq is a multiple of 64, so a whole wavefront is either inside the row or outside it
        if (t + 256 * v >= nq) break;
        if (vs >= 0 && v != vs) continue;
        float d; int sum;
        const uint32_t packed = lg_quant4_8lanes(xv[v], &d, &sum);
        const int quad = t + 256 * v;                        // 4 values = a quarter of a 16-byte unit
        if (M <= LG_HIP_MAX_ROWS_DEV && s.q_units == 1) {     // units of 32 dwords per (block, 3 rows): see lg_k_geglu_t
            uint32_t *unit = (uint32_t *)s.q + ((size_t)(quad >> 3) * ((M + 2) / 3) + j / 3) * 32;
            unit[(j % 3) * 8 + (quad & 7)] = packed;
            if ((t & 7) == 0) *(float2 *)(unit + 24 + 2 * (j % 3)) = make_float2(d, __int_as_float(sum));
            continue;
        }
        if (M <= LG_HIP_MAX_ROWS_DEV && s.q_units == 2) {     // 80 dwords per block, 8 row slots: see lg_k_geglu_m
            uint32_t *blk = (uint32_t *)s.q + (size_t)(quad >> 3) * LG_MU_DWORDS;
            const int dw = quad & 7;
            blk[j * 8 + ((dw & 1) | ((dw & 2) << 1) | ((dw & 4) >> 1))] = packed;
            if ((t & 7) == 0) *(float2 *)(blk + 64 + 2 * j) = make_float2(d, 12582912.0f + (float)(8 * sum));
            continue;
        }
        *(uint32_t *)(s.q + lg_q8_off<M>(E, j, quad >> 2, (quad & 3) * 4)) = packed;
        if ((t & 7) == 0) dsb[lg_q8_ds_idx<M>(E, j, quad >> 3)] = make_float2(d, __int_as_float(sum));
    }
}

// Plain q8 quantization of rows x k floats (no norm): 8 lanes per group of 32, output in the
// activation row order of lg_act_layout(k).
__global__ __launch_bounds__(LG_WG) void lg_k_quant_flat(const float *x, int rows, int k, int8_t *q) {
    float2 *ds = (float2 *)(q + (size_t)rows * k);
    const int g = (blockIdx.x * LG_WG + threadIdx.x) >> 3, l = threadIdx.x & 7, nb = k >> 5;
    const bool live = g < rows * nb;
    const float4 h = live ? ((const float4 *)x)[(size_t)g * 8 + l] : make_float4(0, 0, 0, 0);
    float d; int sum;
    const uint32_t packed = lg_quant4_8lanes(h, &d, &sum);
    if (!live) return;
    const int j = g / nb, b = g - j * nb;
    if (rows > LG_HIP_MAX_ROWS_DEV) {                        // a wide block: the matrix-core kernels' layout
        *(uint32_t *)(q + lg_q8_off<LG_HIP_MAX_ROWS_DEV + 1>(k, j, b * 2 + (l >> 2), (l & 3) * 4)) = packed;
        if (l == 0) ds[lg_q8_ds_idx<LG_HIP_MAX_ROWS_DEV + 1>(k, j, b)] = make_float2(d, __int_as_float(sum));
        return;
    }
    const ActLayout lay = lg_act_layout(k);
    ((uint32_t *)(q + (size_t)j * k))[lg_act_unit(lay, b * 2 + (l >> 2)) * 4 + (l & 3)] = packed;
    if (l == 0) ds[(size_t)j * nb + lg_act_block(lay, b)] = make_float2(d, __int_as_float(sum));
}

// Copy M already-quantized rows (int8 + {scale,sum}) from global memory into LDS.
// Eight loads are issued before the first store (named temporaries, not an array, and a scheduling
// barrier between the two halves), so a workgroup pays about one memory round trip per 8 elements
// per thread instead of one per element.  Indices past the end are clamped to the last element,
// which is then copied more than once with the same value: no branches.
template <typename T>
__device__ __forceinline__ void lg_copy_batched(const T *src, T *dst, int n, int nt_known = 0) {
    const int nt = nt_known ? nt_known : (int)blockDim.x;
    for (int i0 = threadIdx.x; i0 < n; i0 += 8 * nt) {
        const int last = n - 1;
        const int a0 = min(i0, last), a1 = min(i0 + nt, last), a2 = min(i0 + 2 * nt, last), a3 = min(i0 + 3 * nt, last);
        const int a4 = min(i0 + 4 * nt, last), a5 = min(i0 + 5 * nt, last), a6 = min(i0 + 6 * nt, last), a7 = min(i0 + 7 * nt, last);
        const T t0 = src[a0], t1 = src[a1], t2 = src[a2], t3 = src[a3], t4 = src[a4], t5 = src[a5], t6 = src[a6], t7 = src[a7];
        __builtin_amdgcn_sched_barrier(0);
        dst[a0] = t0; dst[a1] = t1; dst[a2] = t2; dst[a3] = t3; dst[a4] = t4; dst[a5] = t5; dst[a6] = t6; dst[a7] = t7;
    }
}
template <int M>
__device__ __forceinline__ void lg_load_q8(const int8_t *q, int k, int8_t *lq) {
    lg_copy_batched<uint4>((const uint4 *)q, (uint4 *)lq, M * k * 5 / 64);
}
// The same copy in two halves, for kernels that also have weight tiles to request: the rows' first batch is
// requested first (lg_load_q8_issue), then the tiles, then the batch is stored and the rest copied
// (lg_load_q8_commit).  Loads return in the order they were requested, so the rows (written a moment ago, on their
// way from the memory-side cache) are in LDS while the tiles (from HBM) are still arriving; requested after the
// tiles, the rows' stores wait for every tile.
struct CopyBatch { uint4 t0, t1, t2, t3, t4, t5, t6, t7; };
template <int M>
__device__ __forceinline__ CopyBatch lg_load_q8_issue(const int8_t *q, int k, int nt) {
    const uint4 *src = (const uint4 *)q;
    const int last = M * k * 5 / 64 - 1, i0 = threadIdx.x;
    CopyBatch b;
    b.t0 = src[min(i0, last)]; b.t1 = src[min(i0 + nt, last)];
    if (last >= 2 * nt) {                                     // (short rows, k = 256: two units per thread hold them all)
        b.t2 = src[min(i0 + 2 * nt, last)]; b.t3 = src[min(i0 + 3 * nt, last)];
        b.t4 = src[min(i0 + 4 * nt, last)]; b.t5 = src[min(i0 + 5 * nt, last)]; b.t6 = src[min(i0 + 6 * nt, last)]; b.t7 = src[min(i0 + 7 * nt, last)];
    }
    __builtin_amdgcn_sched_barrier(0);
    return b;
}
template <int M>
__device__ __forceinline__ void lg_load_q8_commit(const CopyBatch &b, const int8_t *q, int k, int8_t *lq, int nt) {
    uint4 *dst = (uint4 *)lq;
    const int n = M * k * 5 / 64, last = n - 1, i0 = threadIdx.x;
    dst[min(i0, last)] = b.t0; dst[min(i0 + nt, last)] = b.t1;
    if (last >= 2 * nt) {
        dst[min(i0 + 2 * nt, last)] = b.t2; dst[min(i0 + 3 * nt, last)] = b.t3;
        dst[min(i0 + 4 * nt, last)] = b.t4; dst[min(i0 + 5 * nt, last)] = b.t5; dst[min(i0 + 6 * nt, last)] = b.t6; dst[min(i0 + 7 * nt, last)] = b.t7;
    }
    if (n > 8 * nt) lg_copy_batched<uint4>((const uint4 *)q + 8 * nt, dst + 8 * nt, n - 8 * nt, nt);
}

// Input of a draft head (src/mtp.c:268-276): cat = [dequant(token_embd[token]) * sqrt(nb), h_prev],
// quantized to q8 as one row of width 2*nb in the activation order of lg_act_layout(2*nb).
// One thread per 4 values, 8 lanes per group of 32.
struct DraftInArgs {
    const uint8_t *emb; int emb_nit, emb_seg; float emb_scale;   // the target's tiled token_embd
    const int32_t *toks;        // token slot (index ctl->step)
    const float   *h_prev;      // [nb]
    int            nb;
    int8_t        *q;           // q8 activation buffer, one row of 2*nb
};
__global__ __launch_bounds__(LG_WG) void lg_k_draft_input(DraftInArgs a, const StepCtl *ctl) {
    const int quad = blockIdx.x * LG_WG + threadIdx.x, k = 2 * a.nb;
    if (quad >= (k >> 2)) return;                            // k is a multiple of 256: whole wavefronts leave
    const int e = quad << 2;
    float4 v;
    if (e < a.nb) {
        const float4 w = lg_tiled_deq4(a.emb, a.emb_nit, a.emb_seg, a.toks[ctl->step], e);
        v = make_float4(w.x * a.emb_scale, w.y * a.emb_scale, w.z * a.emb_scale, w.w * a.emb_scale);
    } else v = *(const float4 *)(a.h_prev + (e - a.nb));
    float d; int sum;
    const uint32_t packed = lg_quant4_8lanes(v, &d, &sum);
    const ActLayout lay = lg_act_layout(k);
    ((uint32_t *)a.q)[lg_act_unit(lay, quad >> 2) * 4 + (quad & 3)] = packed;
    if ((threadIdx.x & 7) == 0) lg_q8_ds<1>(a.q, k)[lg_act_block(lay, quad >> 3)] = make_float2(d, __int_as_float(sum));
}

// ---------------------------------------------------------------------------------------------
// G row groups against M q8 activation rows held in LDS.  A row is cut into S contiguous K
// segments (S = 8, or 32 for rows longer than 128 blocks); lane = r*S + c owns row r of the group
// (64/S rows per group) and segment c, and walks the segment's nit blocks with a serial fma chain.
// The G groups share every activation load (gate with up, or two neighbouring groups).
// Weights are fetched in chunks of LG_U tiles per group; the first chunk is requested before the
// activations are staged (weights depend on nothing), each later chunk while the previous one is
// being consumed.
#define LG_U 2
template <int G, int U = LG_U>
struct WChunk { uint4 q[G][U]; uint32_t s[G][U]; };

template <int G, int U = LG_U>
__device__ __forceinline__ void lg_mm_fetch(WChunk<G, U> &w, const uint8_t *const (&wg)[G], int it0, int nit, int lane) {
    #pragma unroll
    for (int u = 0; u < U; ++u)
        #pragma unroll
        for (int g = 0; g < G; ++g) {
            const int it = it0 + u < nit ? it0 + u : nit - 1;                 // clamp: never read past the group
            w.q[g][u] = lg_ldt16(wg[g], it, lane);
            w.s[g][u] = lg_ldt2(wg[g], it, lane);
        }
}

// On return every lane of a row holds that row's M results (adjacent-pair tree over the S lanes done).
// `first` must hold the chunk of tiles 0..LG_U-1.
template <int M, int S, int G, bool DUMP, int U = LG_U>
__device__ __forceinline__ void lg_mm_groups(const uint8_t *const (&wg)[G], WChunk<G, U> &first, int nit, const int8_t *act,
                                             const float2 *actds, int k, float (&acc)[G][M], int lane,
                                             int32_t *dots, int m, const int (&row)[G]) {
    const int c = lane & (S - 1), nb = k >> 5;
    #pragma unroll
    for (int g = 0; g < G; ++g)
        #pragma unroll
        for (int j = 0; j < M; ++j) acc[g][j] = 0.0f;
    WChunk<G, U> cur = first;
    for (int it0 = 0; it0 < nit; it0 += U) {
        WChunk<G, U> nxt;
        if (it0 + U < nit) lg_mm_fetch<G, U>(nxt, wg, it0 + U, nit, lane);
        #pragma unroll
        for (int u = 0; u < U; ++u) {
            if (it0 + u >= nit) break;
            const int it = it0 + u, b = c * nit + it;        // b: block of the natural order (for DUMP)
            // the LDS reads of all M rows go out together, ahead of the first dot: left to itself the compiler
            // interleaves them row by row and the wavefront waits out an LDS round trip per row
            float2 ds[M]; int4 a0[M], a1[M];
            #pragma unroll
            for (int j = 0; j < M; ++j) {
                ds[j] = actds[j * nb + it * S + c];
                const int8_t *au = act + (size_t)j * k + (size_t)(it * 2 * S + c) * 16;
                a0[j] = *(const int4 *)au; a1[j] = *(const int4 *)(au + S * 16);
            }
            __builtin_amdgcn_sched_barrier(0);
            #pragma unroll
            for (int j = 0; j < M; ++j) {
                #pragma unroll
                for (int g = 0; g < G; ++g) {
                    const int dot = lg_block_dot(cur.q[g][u], a0[j], a1[j], __float_as_int(ds[j].y));
                    if (DUMP) dots[((size_t)j * m + row[g]) * nb + b] = dot;
                    acc[g][j] = lg_fmaf(ds[j].x * lg_h2f((uint16_t)cur.s[g][u]), (float)dot, acc[g][j]);
                }
            }
        }
        if (it0 + U < nit) cur = nxt;
    }
    #pragma unroll
    for (int g = 0; g < G; ++g)
        #pragma unroll
        for (int j = 0; j < M; ++j) acc[g][j] = lg_sum_seg<S>(acc[g][j]);
}

// acc[j] for a lane-dependent j without indexing the register array (an indexed access would
// move the accumulators to scratch memory): bitwise select over the M candidates.
template <int M>
__device__ __forceinline__ float lg_pick(const float (&acc)[M], int j) {
    uint32_t v = 0;
    #pragma unroll
    for (int t = 0; t < M; ++t) v |= __float_as_uint(acc[t]) & (uint32_t)-(int)(j == t);
    return __uint_as_float(v);
}

struct MmArgs {
    const uint8_t *w;        // tiled weights
    int            k, m;     // row length, rows
    float         *out;      // [M][m]
    const int8_t  *q_in;     // q8 activation buffer of the M input rows
    int32_t       *dots;     // DUMP only: [M][m][k/32]
    int            nthreads; // threads per workgroup (blockDim.x): as an argument it arrives with the others
};
#define LG_MM_FIELDS(X, v) X(const uint8_t *, w, w, v) X(const int8_t *, q_in, q_in, v) X(int, k, k, v) X(int, m, m, v) X(int, nthreads, nthreads, v) X(float *, out, out, v) X(int32_t *, dots, dots, v)

// Plain matmul: out[j][i] f32.  blockDim = 64*W wavefronts, each wavefront takes G neighbouring
// row groups (G*64/S rows); grid covers ceil(groups / (W*G)) workgroups.
// U: weight tiles per chunk (requested together, the next chunk while the current one is consumed)
template <int M, int S, int G, bool DUMP, int U = LG_U>
__global__ __launch_bounds__(S == 32 ? 320 : LG_WG, 2) void lg_k_mm(LG_MM_FIELDS(LG_XP, _) int p_end_) {
    MmArgs a; LG_MM_FIELDS(LG_XI, a)
    extern __shared__ __align__(16) unsigned char smem[];
    int8_t *lq = (int8_t *)smem;
    float2 *lds = (float2 *)(smem + (size_t)M * a.k);
    constexpr int RW = 64 / S;                                // rows per group
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = a.nthreads >> 6;
    const int nit = (a.k >> 5) / S, ngroups = a.m / RW;
    const int g0 = (blockIdx.x * nw + wave) * G;
    const uint8_t *wg[G];
    int row[G];
    #pragma unroll
    for (int g = 0; g < G; ++g) {
        const int gi = g0 + g < ngroups ? g0 + g : ngroups - 1;   // ragged tail: recompute the last group
        wg[g] = a.w + (size_t)gi * nit * LG_TILE;
        row[g] = gi * RW + lane / S;
    }
    const CopyBatch rows = lg_load_q8_issue<M>(a.q_in, a.k, a.nthreads); // the rows first, then the tiles
    WChunk<G, U> first;
    lg_mm_fetch<G, U>(first, wg, 0, nit, lane);
    __builtin_amdgcn_sched_barrier(0);
    lg_load_q8_commit<M>(rows, a.q_in, a.k, lq, a.nthreads);
    __syncthreads();
    if (g0 >= ngroups) return;
    float acc[G][M];
    lg_mm_groups<M, S, G, DUMP, U>(wg, first, nit, lq, lds, a.k, acc, lane, a.dots, a.m, row);
    const int c = lane & (S - 1);
    if (c < M) {
        #pragma unroll
        for (int g = 0; g < G; ++g) a.out[(size_t)c * a.m + row[g]] = lg_pick<M>(acc[g], c);
    }
}

// Gate/up matmul with the GeGLU and the q8 quantization of its result as epilogue.
struct GegluArgs {
    const uint8_t *w;        // row-block tiles of [2*n_ff][k], virtual row order: 32 gate, 32 up, 32 gate, ...
    int            k, n_ff;
    const int8_t  *q_in;     // verify blocks: unit order (below); wide blocks: lg_q8_off
    int8_t        *gq;       // q8 activation buffer of the result, width n_ff
    int            gq_units; // lg_k_geglu_m only: 2 = write the 80-dword blocks of the matrix-core kernels (what lg_k_down_m reads) instead of rows
};
#define LG_GEGLU_FIELDS(X, v) X(const uint8_t *, w, w, v) X(const int8_t *, q_in, q_in, v) X(int, k, k, v) X(int, n_ff, n_ff, v) X(int8_t *, gq, gq, v) X(int, gq_units, gq_units, v)
// Gate/up + GeGLU for verify blocks (M <= 8): a wavefront is 64 weight rows x one of
// the 8 K segments, so every lane of it multiplies its own weight block with the SAME activation
// block.  The activations then travel through the scalar cache into SGPRs (loads from the constant
// address space with a wavefront-uniform address) and feed v_dot4 as scalar operands: no LDS fill,
// no barrier before the first dot, no per-lane activation traffic.  Weights: tile (row block of 64 =
// the 32 gate rows and 32 up rows of 32 FFN columns, block kb) = lane r's 16 nibble bytes at r*16 and
// scale at 1024 + r*2, tiles ordered [row block][kb] ("row-block tiles", lg_hip_repack_q4_0_rowblocks).
// Activations: per block kb and group of 3 rows one unit of 32 dwords: 3 x 8 dwords of int8, then
// 3 x {scale, sum}, 2 unused; a unit is requested while the previous one is consumed.
typedef const __attribute__((address_space(4))) int *lg_cint;
template <int M>
__global__ __launch_bounds__(512, 2) void lg_k_geglu_t(LG_GEGLU_FIELDS(LG_XP, _) int p_end_) {
    GegluArgs a; LG_GEGLU_FIELDS(LG_XI, a)
    __shared__ float red[8][M][64];
    constexpr int NU = (M + 2) / 3, CH = 2;
    const int lane = threadIdx.x & 63;
    const int s = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));      // K segment of this wavefront
    const int t = blockIdx.x, nb = a.k >> 5, nit = nb >> 3, nunits = nit * NU;
    const uint8_t *wt = a.w + ((size_t)t * nb + (size_t)s * nit) * LG_TILE;
    lg_cint au = (lg_cint)(uintptr_t)a.q_in + (size_t)s * nunits * 32;
    float p[M];
    #pragma unroll
    for (int j = 0; j < M; ++j) p[j] = 0.0f;
    uint4 wq[CH], nwq[CH]; uint32_t wd[CH], nwd[CH];
    auto fetch = [&](int it0) {
        #pragma unroll
        for (int u = 0; u < CH; ++u) {
            const int it = it0 + u < nit ? it0 + u : nit - 1;
            nwq[u] = lg_ldt16(wt, it, lane);
            nwd[u] = lg_ldt2(wt, it, lane);
        }
    };
    // The units were written by the previous kernel on other XCDs, so the first read of each 128-byte
    // unit from this XCD misses its L2; walked one unit ahead, those misses would queue up behind each
    // other.  One vector load per unit, issued now, brings the segment's lines in side by side.  They go out ahead
    // of the first weight tiles and nothing waits for them before the end (a wait here would also be one for the tiles).
    // (nunits <= 16: k <= 4096 and at most three rows.)  The load is written as an instruction of its own: a volatile
    // load is followed by a wait for every load in flight, a plain one with no use before the end is moved there.  Its
    // register stays reserved until the wait at the end of the loop, which names it as an operand.
    int touch;
    {
        const int *tp = (const int *)a.q_in + ((size_t)s * nunits + (lane < nunits ? lane : nunits - 1)) * 32;
        asm volatile("global_load_dword %0, %1, off" : "=v"(touch) : "v"(tp) : "memory");
    }
    fetch(0);
    int cur[32], nxt[32];
    #pragma unroll
    for (int i = 0; i < 32; ++i) cur[i] = au[i];
    for (int it0 = 0; it0 < nit; it0 += CH) {
        #pragma unroll
        for (int u = 0; u < CH; ++u) { wq[u] = nwq[u]; wd[u] = nwd[u]; }
        if (it0 + CH < nit) fetch(it0 + CH);
        #pragma unroll
        for (int c = 0; c < CH; ++c) {
            if (it0 + c >= nit) break;
            const uint4 q = wq[c];
            const int lo0 = q.x & 0x0F0F0F0F, lo1 = q.y & 0x0F0F0F0F, lo2 = q.z & 0x0F0F0F0F, lo3 = q.w & 0x0F0F0F0F;
            const int hi0 = (q.x >> 4) & 0x0F0F0F0F, hi1 = (q.y >> 4) & 0x0F0F0F0F, hi2 = (q.z >> 4) & 0x0F0F0F0F, hi3 = (q.w >> 4) & 0x0F0F0F0F;
            const float dw = lg_h2f((uint16_t)wd[c]);
            #pragma unroll
            for (int u = 0; u < NU; ++u) {
                const int tu = (it0 + c) * NU + u, tn = tu + 1 < nunits ? tu + 1 : tu;
                // the unit in `cur` must have arrived before the next one is requested: scalar loads
                // return out of order, so the only wait there is waits for everything in flight
                asm volatile("" :: "s"(cur[0]), "s"(cur[8]), "s"(cur[16]), "s"(cur[24]), "s"(cur[31]));
                __builtin_amdgcn_sched_barrier(0);
                #pragma unroll
                for (int i = 0; i < 32; ++i) nxt[i] = au[(size_t)tn * 32 + i];
                __builtin_amdgcn_sched_barrier(0);
                #pragma unroll
                for (int r = 0; r < 3; ++r) {
                    const int j = u * 3 + r;
                    if (j < M) {
                        int dot = -8 * cur[25 + 2 * r];       // the -8*sum term of the block dot, formed on the scalar unit
                        dot = __builtin_amdgcn_sdot4(lo0, cur[r * 8 + 0], dot, false);
                        dot = __builtin_amdgcn_sdot4(lo1, cur[r * 8 + 1], dot, false);
                        dot = __builtin_amdgcn_sdot4(lo2, cur[r * 8 + 2], dot, false);
                        dot = __builtin_amdgcn_sdot4(lo3, cur[r * 8 + 3], dot, false);
                        dot = __builtin_amdgcn_sdot4(hi0, cur[r * 8 + 4], dot, false);
                        dot = __builtin_amdgcn_sdot4(hi1, cur[r * 8 + 5], dot, false);
                        dot = __builtin_amdgcn_sdot4(hi2, cur[r * 8 + 6], dot, false);
                        dot = __builtin_amdgcn_sdot4(hi3, cur[r * 8 + 7], dot, false);
                        p[j] = lg_fmaf(__int_as_float(cur[24 + 2 * r]) * dw, (float)dot, p[j]);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                #pragma unroll
                for (int i = 0; i < 32; ++i) cur[i] = nxt[i];
            }
        }
    }
    // the explicit wait for that load (after the loop every load of this wavefront has long returned: it costs nothing)
    asm volatile("s_waitcnt vmcnt(0)" :: "v"(touch) : "memory");
    #pragma unroll
    for (int j = 0; j < M; ++j) red[s][j][lane] = p[j];
    __syncthreads();
    for (int j = threadIdx.x >> 5; j < M; j += 16) {         // half-wavefront per row, one FFN column per lane
        const int i = threadIdx.x & 31;
        float g[8], u[8];
        #pragma unroll
        for (int c = 0; c < 8; ++c) { g[c] = red[c][j][i]; u[c] = red[c][j][32 + i]; }
        const float gate = ((g[0] + g[1]) + (g[2] + g[3])) + ((g[4] + g[5]) + (g[6] + g[7]));
        const float up = ((u[0] + u[1]) + (u[2] + u[3])) + ((u[4] + u[5]) + (u[6] + u[7]));
        float d; int sum;
        const int q = lg_quant1_32lanes(lg_gelu(gate) * up, &d, &sum);
        const ActLayout lay = lg_act_layout(a.n_ff);          // order the ffn_down matmul reads
        a.gq[(size_t)j * a.n_ff + lg_act_unit(lay, t * 2 + (i >> 4)) * 16 + (i & 15)] = (int8_t)q;
        if (i == 0) lg_q8_ds<M>(a.gq, a.n_ff)[(size_t)j * (a.n_ff >> 5) + lg_act_block(lay, t)] = make_float2(d, __int_as_float(sum));
    }
}

// Gate/up + GeGLU for verify blocks of 4..8 rows on the matrix cores.  Same weight tiles and the same
// wavefront = 64 weight rows x one K segment split as lg_k_geglu_t, but the 8 v_dot4 per (tile, row) become
// two v_mfma_i32_32x32x32_i8 per tile whatever M is: A = the block's activations (row m = draft row, 8 row
// slots, the other 24 rows of the operand are don't-cares whose results are never read), B = the tile's 32
// gate rows, then its 32 up rows, as columns.  A lane's operand is the K half l/32 of column l%32, while a
// tile keeps weight row l whole in lane l, so the two halves of the wavefront first trade 8 bytes each
// (v_permlane32_swap): lane (n, h) then holds nibble bytes 8h..8h+7 of gate row n and of up row n, i.e.
// K = 8h..8h+7 and 16+8h..16+8h+7.  The activation bytes are stored in that order (dwords 0 1 4 5 | 2 3 6 7
// of a row's 32), 80 dwords per block: 8 row slots x 8 dwords, then 8 x {scale, 12582912 + 8*sum as a float}.  Result register
// i of lane (n, h) is draft row 4h+i of column n, so a lane applies 4 scale pairs per column, and the
// per-block float work is 8 x (add, cvt, mul, fma) however many draft rows there are.
// Each wavefront copies its own K segment of the activations into LDS once (wave-private, no barrier).
typedef int lg_v4i __attribute__((ext_vector_type(4)));
typedef int lg_v16i __attribute__((ext_vector_type(16)));
typedef unsigned lg_v2u __attribute__((ext_vector_type(2)));
template <int M>
__global__ __launch_bounds__(512, 2) void lg_k_geglu_m(LG_GEGLU_FIELDS(LG_XP, _) int p_end_) {
    GegluArgs a; LG_GEGLU_FIELDS(LG_XI, a)
    extern __shared__ __align__(16) unsigned char smem[];     // [8 segments][nit][80 dwords]
    __shared__ float red[8][LG_HIP_MAX_ROWS_DEV][64];
    constexpr int CH = 2;
    const int lane = threadIdx.x & 63, n = lane & 31, h = lane >> 5;
    const int s = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));      // K segment of this wavefront
    const int t = blockIdx.x, nb = a.k >> 5, nit = nb >> 3;
    const uint8_t *wt = a.w + ((size_t)t * nb + (size_t)s * nit) * LG_TILE;
    uint4 wq[CH], nwq[CH]; uint32_t wd[CH], nwd[CH];
    const __amdgpu_buffer_rsrc_t rw = lg_buffer_rsrc(wt);
    auto fetch = [&](int it0) {
        #pragma unroll
        for (int u = 0; u < CH; ++u) {
            const int it = it0 + u < nit ? it0 + u : nit - 1;
            nwq[u] = lg_ldt16b(rw, it, lane);
            nwd[u] = lg_ldt2b(rw, it, lane);
        }
    };
    unsigned char *la = smem + (size_t)s * nit * (LG_MU_DWORDS * 4);
    {
        // four loads in flight per lane before the first store (left as a plain loop the copy is one round trip per 16
        // bytes); the first four are requested ahead of the first weight tiles and stored after them: loads return in
        // the order they were requested, and the rows come from nearer than the tiles
        const uint4 *src = (const uint4 *)(a.q_in + (size_t)s * nit * (LG_MU_DWORDS * 4));
        const int nu = nit * (LG_MU_DWORDS / 4);
        {
            const int i0 = min(lane, nu - 1), i1 = min(lane + 64, nu - 1), i2 = min(lane + 128, nu - 1), i3 = min(lane + 192, nu - 1);
            const uint4 t0 = src[i0], t1 = src[i1], t2 = src[i2], t3 = src[i3];
            __builtin_amdgcn_sched_barrier(0);
            fetch(0);
            __builtin_amdgcn_sched_barrier(0);
            ((uint4 *)la)[i0] = t0; ((uint4 *)la)[i1] = t1; ((uint4 *)la)[i2] = t2; ((uint4 *)la)[i3] = t3;
        }
        for (int i0 = lane + 256; i0 < nu; i0 += 256) {
            const int i1 = min(i0 + 64, nu - 1), i2 = min(i0 + 128, nu - 1), i3 = min(i0 + 192, nu - 1);
            const uint4 t0 = src[i0], t1 = src[i1], t2 = src[i2], t3 = src[i3];
            __builtin_amdgcn_sched_barrier(0);
            ((uint4 *)la)[i0] = t0; ((uint4 *)la)[i1] = t1; ((uint4 *)la)[i2] = t2; ((uint4 *)la)[i3] = t3;
        }
        // read back below by other lanes of this wavefront only: LDS serves a wavefront's accesses in order,
        // the fences keep the compiler from moving the reads above the writes
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    float pg[4] = { 0.0f, 0.0f, 0.0f, 0.0f }, pu[4] = { 0.0f, 0.0f, 0.0f, 0.0f };
    // The accumulators start at the bit pattern of 1.5 * 2^23 = 12582912.0f: the integer dot (|dot| < 2^22) lands
    // in the mantissa, the result read as a float is 12582912 + dot exactly, and subtracting the stored
    // 12582912 + 8*sum gives (float)(dot - 8*sum) exactly, in one instruction per output.
    lg_v16i magic;
    #pragma unroll
    for (int i = 0; i < 16; ++i) magic[i] = 0x4B400000;
    const int arow = n < 8 ? n : 7;                           // operand rows past the 8 slots: any readable bytes
    for (int it0 = 0; it0 < nit; it0 += CH) {
        #pragma unroll
        for (int u = 0; u < CH; ++u) { wq[u] = nwq[u]; wd[u] = nwd[u]; }
        if (it0 + CH < nit) fetch(it0 + CH);
        #pragma unroll
        for (int c = 0; c < CH; ++c) {
            if (it0 + c >= nit) break;
            const unsigned char *lb = la + (size_t)(it0 + c) * (LG_MU_DWORDS * 4);
            const lg_v4i av = *(const lg_v4i *)(lb + arow * 32 + h * 16);
            const int4 sc0 = *(const int4 *)(lb + 256 + h * 32), sc1 = *(const int4 *)(lb + 256 + h * 32 + 16);
            const uint4 q = wq[c];
            const lg_v2u s0 = __builtin_amdgcn_permlane32_swap(q.x, q.z, false, false);
            const lg_v2u s1 = __builtin_amdgcn_permlane32_swap(q.y, q.w, false, false);
            const lg_v2u sd = __builtin_amdgcn_permlane32_swap(wd[c], wd[c], false, false);
            lg_v4i bg, bu;
            bg.x = s0.x & 0x0F0F0F0F; bg.y = s1.x & 0x0F0F0F0F; bg.z = (s0.x >> 4) & 0x0F0F0F0F; bg.w = (s1.x >> 4) & 0x0F0F0F0F;
            bu.x = s0.y & 0x0F0F0F0F; bu.y = s1.y & 0x0F0F0F0F; bu.z = (s0.y >> 4) & 0x0F0F0F0F; bu.w = (s1.y >> 4) & 0x0F0F0F0F;
            const float dg = lg_h2f((uint16_t)sd.x), du = lg_h2f((uint16_t)sd.y);
            const lg_v16i d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, bg, magic, 0, 0, 0);
            const lg_v16i d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, bu, magic, 0, 0, 0);
            const float xd[4] = { __int_as_float(sc0.x), __int_as_float(sc0.z), __int_as_float(sc1.x), __int_as_float(sc1.z) };
            const float cf[4] = { __int_as_float(sc0.y), __int_as_float(sc0.w), __int_as_float(sc1.y), __int_as_float(sc1.w) };
            #pragma unroll
            for (int i = 0; i < 4; ++i) {
                pg[i] = lg_fmaf(xd[i] * dg, __int_as_float(d0[i]) - cf[i], pg[i]);
                pu[i] = lg_fmaf(xd[i] * du, __int_as_float(d1[i]) - cf[i], pu[i]);
            }
        }
    }
    #pragma unroll
    for (int i = 0; i < 4; ++i) { red[s][4 * h + i][n] = pg[i]; red[s][4 * h + i][32 + n] = pu[i]; }
    __syncthreads();
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
}

// Per-layer inputs of a block, finished once per step from the raw per_layer_model_proj output and the
// tokens' per-layer embedding rows (the reference builds them once per step in build_per_layer_n,
// src/cuda/model-cuda.cuh:1121-1147): ipl = (rmsnorm(proj/sqrt(E)) * w + tok*sqrt(ple)) / sqrt(2),
// in place over the raw projection.  One wavefront per (layer, row); ple <= 256.
struct IplArgs {
    float         *pmp;      // [rows][n_layer*ple]: raw projection in, ipl out
    int            ple, n_layer, rows_per_step;
    const float   *proj_norm;     // [ple]
    const uint8_t *pte;      // per_layer_token_embd, plain q4_0 rows of n_layer*ple
    const int32_t *toks;
    float          pscale, tscale, rsqrt2, eps;
};
__global__ __launch_bounds__(64) void lg_k_ipl(IplArgs a, const StepCtl *ctl) {
    const int lane = threadIdx.x, L = blockIdx.x, j = blockIdx.y, ple = a.ple, e0 = 4 * lane;
    float *pr = a.pmp + (size_t)j * a.n_layer * ple + (size_t)L * ple;
    const bool on = e0 < ple;
    const float4 p4 = on ? *(const float4 *)(pr + e0) : make_float4(0, 0, 0, 0);
    const float4 wn = on ? *(const float4 *)(a.proj_norm + e0) : make_float4(0, 0, 0, 0);
    const int tok = a.toks[ctl->step * a.rows_per_step + j];
    const uint8_t *trow = a.pte + (size_t)tok * ((size_t)a.n_layer * ple / 32 * 18);
    float tk[4];
    #pragma unroll
    for (int i = 0; i < 4; ++i) tk[i] = on ? lg_q4_0_elem(trow, L * ple + e0 + i) * a.tscale : 0.0f;
    const float4 p = make_float4(p4.x * a.pscale, p4.y * a.pscale, p4.z * a.pscale, p4.w * a.pscale);
    const float ss = lg_wave_sum64(lg_sumsq4(p, 0.0f));                 // one quad per lane
    const float sc = 1.0f / sqrtf(ss / (float)ple + a.eps);
    if (on) *(float4 *)(pr + e0) = make_float4((p.x * sc * wn.x + tk[0]) * a.rsqrt2, (p.y * sc * wn.y + tk[1]) * a.rsqrt2,
                                               (p.z * sc * wn.z + tk[2]) * a.rsqrt2, (p.w * sc * wn.w + tk[3]) * a.rsqrt2);
}

// PLE gate: inp_gate matmul on the q8 of the updated residual, then gelu(.) * ipl and q8.
struct PleGateArgs {
    const uint8_t *w;        // tiled inp_gate [ple][E]
    int            k, ple;
    const int8_t  *q_in;
    const float   *ipl;      // [M][n_layer*ple] per-layer inputs (lg_k_ipl)
    int            layer, n_layer;
    int8_t        *pq;       // q8 activation buffer of the result, width ple
};
// Verify blocks (wide blocks: lg_k_mm_plegate_wide): the row work that precedes the matmul is folded in,
// i.e. the residual update x += rmsnorm(dout) * w_post and the q8 of the new x (what lg_k_rows does
// between two other matmuls).  One workgroup per (block of 32 gate rows, draft row): it updates and quantizes
// its one row (lane assignment and summation order of lg_k_rows; the quantized row goes straight to LDS, the
// workgroups of gate block 0 also write the new residual), then its four wavefronts take 8 gate rows each
// against that row.  The ple/32 workgroups of a draft row repeat its row work, which costs less than a kernel
// boundary; splitting the draft rows over workgroups keeps what one CU has to pull in (row, previous output,
// norm weights, 32 gate rows) near 76 KB at the E4B shape.
struct RowsPleGateArgs {
    PleGateArgs    g;
    const float   *x, *dout, *w_post;   // [M][E] residual, [M][E] ffn_down output, [E]
    float         *x_out;               // [M][E]
    float          eps;
    int            dparts;              // 8: dout is eight [M][E] slabs of partial sums (one per XCD), added here in tree order; else 1
};
#define LG_RPG_FIELDS(X, v) X(const float *, x, x, v) X(const float *, dout, dout, v) X(const float *, w_post, w_post, v) X(const uint8_t *, gw, g.w, v) X(int, gk, g.k, v) X(int, gple, g.ple, v) X(int, dparts, dparts, v) X(const float *, gipl, g.ipl, v) X(int, glayer, g.layer, v) X(int, gnl, g.n_layer, v) X(int8_t *, gpq, g.pq, v) X(const int8_t *, gq_in, g.q_in, v) X(float *, x_out, x_out, v) X(float, eps, eps, v)
// The body for gate block gb and draft row j (a device function: the kernel below runs it per workgroup of its grid,
// lg_k_ple_tail as the first phase of a longer kernel).  xnew receives the lane's float4s of the updated residual;
// after_requests runs once every load of the body has been requested (a caller's own loads go there: loads return
// in the order they were requested, and the row's must not wait behind them).
template <int M, typename Hook>
__device__ __forceinline__ void lg_rows_plegate_body(const RowsPleGateArgs &a, int gb, int j, unsigned char *smem, float *gbuf, float *red,
                                                     float4 (&xnew)[LG_ROWV], bool write_x, Hook &&after_requests) {
    int8_t *lq = (int8_t *)smem;                              // one row: [E] int8, then [E/32] {scale, sum}
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, E = a.g.k, nit = E >> 8, ple = a.g.ple;
    float2 *lds = (float2 *)(smem + (size_t)E);
    const uint8_t *wg[1] = { a.g.w + (size_t)(gb * 4 + wave) * nit * LG_TILE };
    // Every load of the kernel is requested up front, the row's first (loads return in order: the row work then starts
    // while the tiles are still arriving), then the whole row group (nit <= 16 tiles: with this few workgroups the
    // kernel is a chain of memory round trips, and fetching the tiles two at a time adds one per pair), then the
    // per-layer input of the lane's gate column (kept in a register until the end: parked in LDS on arrival, it made
    // the kernel wait for everything requested before it, ahead of the row's own loads).
    const int t = threadIdx.x, nq = E >> 2;
    float4 xv[LG_ROWV], dv[LG_ROWV], wp[LG_ROWV];
    {
        const float4 *wr = (const float4 *)a.w_post, *xr = (const float4 *)(a.x + (size_t)j * E), *dr = (const float4 *)(a.dout + (size_t)j * E);
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) { xv[v] = xr[t + 256 * v]; dv[v] = dr[t + 256 * v]; wp[v] = wr[t + 256 * v]; }
        if (a.dparts == 4) {                                  // the top two levels of the tree of an ffn_down cut by K quarter
            const size_t slab = (size_t)M * nq;
            #pragma unroll
            for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) {
                const float4 p1 = dr[slab + t + 256 * v], p2 = dr[2 * slab + t + 256 * v], p3 = dr[3 * slab + t + 256 * v], p0 = dv[v];
                dv[v] = make_float4((p0.x + p1.x) + (p2.x + p3.x), (p0.y + p1.y) + (p2.y + p3.y),
                                    (p0.z + p1.z) + (p2.z + p3.z), (p0.w + p1.w) + (p2.w + p3.w));
            }
        }
        if (a.dparts == 8) {                                  // the top three levels of the K-segment tree of an ffn_down cut over the 8 XCDs
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
    #pragma unroll
    for (int u = 0; u < LG_MAXV; ++u) {
        const int it = u < nit ? u : nit - 1;
        // (plain loads: the M workgroups of a gate block read the same tiles)
        wq[u] = *(const uint4 *)(wg[0] + (size_t)it * LG_TILE + lane * 16);
        wsc[u] = *(const uint16_t *)(wg[0] + (size_t)it * LG_TILE + 1024 + lane * 2);
    }
    const float iplv = a.g.ipl[(size_t)j * a.g.n_layer * ple + (size_t)a.g.layer * ple + gb * 32 + wave * 8 + (lane >> 3)];   // of this lane's gate column
    after_requests();
    {
        float ss = 0.0f;
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) if (t + 256 * v < nq) ss = lg_sumsq4(dv[v], ss);
        ss = lg_block_sum256(ss, red);
        const float sc = 1.0f / sqrtf(ss / (float)E + a.eps);
        #pragma unroll
        for (int v = 0; v < LG_ROWV; ++v) {
            if (t + 256 * v < nq) {                           // nq is a multiple of 64: whole wavefronts
                const float4 w = wp[v], d = dv[v];
                float4 x = xv[v];
                x.x = x.x + d.x * sc * w.x;  x.y = x.y + d.y * sc * w.y;
                x.z = x.z + d.z * sc * w.z;  x.w = x.w + d.w * sc * w.w;
                if (write_x) ((float4 *)(a.x_out + (size_t)j * E))[t + 256 * v] = x;
                xnew[v] = x;
                float dq; int sum;
                const uint32_t packed = lg_quant4_8lanes(x, &dq, &sum);
                const int quad = t + 256 * v;
                *(uint32_t *)(lq + lg_q8_off<1>(E, 0, quad >> 2, (quad & 3) * 4)) = packed;
                if ((t & 7) == 0) lds[lg_q8_ds_idx<1>(E, 0, quad >> 3)] = make_float2(dq, __int_as_float(sum));
            }
        }
    }
    __syncthreads();
    {
        const int c = lane & 7;
        float p = 0.0f;
        #pragma unroll
        for (int u = 0; u < LG_MAXV; ++u) {
            if (u < nit) {                                    // (a guard, not a break: the arrays stay in registers)
                const float2 ds = lds[u * 8 + c];
                const int8_t *au = lq + (size_t)(u * 16 + c) * 16;
                const int dot = lg_block_dot(wq[u], *(const int4 *)au, *(const int4 *)(au + 8 * 16), __float_as_int(ds.y));
                p = lg_fmaf(ds.x * lg_h2f((uint16_t)wsc[u]), (float)dot, p);
            }
        }
        p = lg_sum_seg<8>(p);
        if (c == 0) gbuf[wave * 8 + (lane >> 3)] = lg_gelu(p) * iplv;
    }
    __syncthreads();
    if (threadIdx.x < 32) {
        const int i = threadIdx.x;
        float d; int sum;
        const int q = lg_quant1_32lanes(gbuf[i], &d, &sum);
        const ActLayout lay = lg_act_layout(ple);
        a.g.pq[(size_t)j * ple + lg_act_unit(lay, gb * 2 + (i >> 4)) * 16 + (i & 15)] = (int8_t)q;
        if (i == 0) lg_q8_ds<M>(a.g.pq, ple)[(size_t)j * (ple >> 5) + lg_act_block(lay, gb)] = make_float2(d, __int_as_float(sum));
    }
}
template <int M>
__global__ __launch_bounds__(LG_WG) void lg_k_rows_plegate(LG_RPG_FIELDS(LG_XP, _) int p_end_) {
    RowsPleGateArgs a; LG_RPG_FIELDS(LG_XI, a)
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float gbuf[32], red[4];
    float4 xnew[LG_ROWV];
    lg_rows_plegate_body<M>(a, (int)blockIdx.x, (int)blockIdx.y, smem, gbuf, red, xnew, blockIdx.x == 0, [] {});
}

// lm_head: each workgroup walks `passes` blocks of 64 vocabulary rows (4 wavefronts x 2 groups
// sharing activation loads), applies the soft cap and keeps a running argmax per draft row
// (first maximum: lower index wins ties, src/cuda/model-cuda.cuh:703-720); one partial per
// workgroup and row goes to global memory.
struct HeadArgs {
    const uint8_t *w; int k, n_vocab, passes;
    const int8_t *q_in;
    float softcap;
    float *logits;          // [M][n_vocab] or nullptr
    float *pval; int *pidx; // [gridDim.x][M]
};
#define LG_HEAD_FIELDS(X, v) X(const uint8_t *, w, w, v) X(const int8_t *, q_in, q_in, v) X(int, k, k, v) X(int, n_vocab, n_vocab, v) X(int, passes, passes, v) X(float, softcap, softcap, v) X(float *, logits, logits, v) X(float *, pval, pval, v) X(int *, pidx, pidx, v)
template <int M>
__global__ __launch_bounds__(LG_WG, 2) void lg_k_mm_head(LG_HEAD_FIELDS(LG_XP, _) int p_end_) {
    HeadArgs a; LG_HEAD_FIELDS(LG_XI, a)
    extern __shared__ __align__(16) unsigned char smem[];
    int8_t *lq = (int8_t *)smem;
    float2 *lds = (float2 *)(smem + (size_t)M * a.k);
    __shared__ float sv[4][LG_HIP_MAX_ROWS_DEV];
    __shared__ int si[4][LG_HIP_MAX_ROWS_DEV];
    lg_load_q8<M>(a.q_in, a.k, lq);
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
        WChunk<2> first;
        lg_mm_fetch<2>(first, wg, 0, nit, lane);
        lg_mm_groups<M, 8, 2, false>(wg, first, nit, lq, lds, a.k, acc, lane, nullptr, 0, row);
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
#define LG_ACCEPT_FIELDS(X, v) X(const float *, pval, pval, v) X(const int *, pidx, pidx, v) X(int, n_part, n_part, v) X(int, E, E, v) X(const int32_t *, toks, toks, v) X(const float *, hidden_rows, hidden_rows, v) X(int32_t *, out, out, v) X(int32_t *, adv, adv, v) X(float *, g_hidden, g_hidden, v)
template <int M>
__global__ __launch_bounds__(LG_WG) void lg_k_accept(StepCtl *ctl, LG_ACCEPT_FIELDS(LG_XP, _) int p_end_) {
    AcceptArgs a; LG_ACCEPT_FIELDS(LG_XI, a)
    __shared__ float sv[LG_HIP_MAX_ROWS_DEV][LG_WG / 64];
    __shared__ int si[LG_HIP_MAX_ROWS_DEV][LG_WG / 64];
    __shared__ int s_adv;
    const int step = ctl->step, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // the block's tokens and this thread's slice of every row's hidden state are requested with the partials: read
    // when they are needed (the tokens one after the other in the accept loop, the accepted row after it) each costs
    // a memory round trip of its own at the end of the step
    int tk[M];
    #pragma unroll
    for (int j = 0; j < M; ++j) tk[j] = a.toks[(size_t)step * M + j];
    constexpr int HS = 4;                                     // float4 per thread and row: E <= 4096
    float4 hrow[M][HS];
    const bool hregs = a.E <= HS * 4 * LG_WG && (a.E & 3) == 0;
    if (hregs) {
        #pragma unroll
        for (int j = 0; j < M; ++j)
            #pragma unroll
            for (int u = 0; u < HS; ++u) {
                const int q4 = (int)threadIdx.x + u * LG_WG;
                hrow[j][u] = ((const float4 *)(a.hidden_rows + (size_t)j * a.E))[q4 < (a.E >> 2) ? q4 : 0];
            }
    }
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
        int adv = 1;
        #pragma unroll
        for (int j = 1; j < M; ++j) if (adv == j && best[j - 1] == tk[j]) adv = j + 1;
        for (int j = 0; j < M; ++j) a.out[(size_t)step * M + j] = best[j];
        a.adv[step] = adv;
        s_adv = adv;
    }
    __syncthreads();
    const int adv = s_adv;
    if (hregs) {
        #pragma unroll
        for (int u = 0; u < HS; ++u) {
            const int q4 = (int)threadIdx.x + u * LG_WG;
            float4 h = hrow[0][u];
            #pragma unroll
            for (int j = 1; j < M; ++j) if (adv - 1 == j) h = hrow[j][u];
            if (q4 < (a.E >> 2)) ((float4 *)a.g_hidden)[q4] = h;
        }
    } else {
        for (int i = threadIdx.x; i < a.E; i += LG_WG) a.g_hidden[i] = a.hidden_rows[(size_t)(adv - 1) * a.E + i];
    }
    __syncthreads();
    if (threadIdx.x == 0) { ctl->pos += adv; ctl->step = step + 1; }
}

// Prefill blocks skip the head: only the position advances.
__global__ void lg_k_advance(StepCtl *ctl, int rows) { ctl->pos += rows; ctl->step += 1; }

// Glue of a speculative round that stays on the device (the host loop it replaces: src/run.c:54-71): one thread
// moves tokens between the draft head's and the target's step state, so that K chained drafts and the verify
// step that checks them run back to back with no copy to the host.
//   phase 1..K   (before draft `phase`): the head's input token = the block's chosen token (phase 1) or the head's
//                previous draft, which also becomes row phase-1 of the target's block; the head drafts for
//                position pos + phase - 1 (src/run.c:60-66).
//   phase K+1    (before the verify step): the last draft becomes row K of the block.
//   phase 0      (after the verify step, whose accept kernel has advanced pos and step): the greedy successor of
//                the last accepted row is the next block's chosen token (src/run.c:569-574).
struct LinkArgs {
    StepCtl *hctl; const StepCtl *tctl;
    int32_t *hsched; const int32_t *hout;        // head: token slot 0, drafted token 0
    int32_t *tsched; const int32_t *tout, *tadv; // target: [steps][M] blocks, [steps][M] successors, [steps]
    int M, phase;
};
__global__ void lg_k_link(LinkArgs a) {
    const int s = a.tctl->step;
    if (a.phase == 0) {
        a.tsched[(size_t)s * a.M] = a.tout[(size_t)(s - 1) * a.M + a.tadv[s - 1] - 1];
        return;
    }
    const int tok = a.phase == 1 ? a.tsched[(size_t)s * a.M] : a.hout[0];
    if (a.phase > 1) a.tsched[(size_t)s * a.M + a.phase - 1] = tok;
    if (a.phase < a.M) {
        a.hsched[0] = tok;
        a.hctl->pos = a.tctl->pos + a.phase - 1;
        a.hctl->step = 0;
    }
}

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
// One head vector (hd <= 512 floats) per wavefront, in two steps so that a wavefront with several vectors to do
// has all their loads in flight first.  lg_head_load: 4 consecutive elements per lane (and 4 more at +256).
// lg_head_finish: rmsnorm (weighted by `w`, or plain when w == nullptr) in the 256-lane sum order, then NeoX
// rotary at position `pos` when `rope`; the result lands in vec[0..hd), LDS private to the wavefront.
// NV = 1 serves hd <= 256 with half the registers.
template <int NV> struct HeadVec { float4 x[NV]; };
template <int NV>
__device__ __forceinline__ HeadVec<NV> lg_head_load(const float *src, int hd) {
    const int lane = threadIdx.x & 63;
    HeadVec<NV> h;
    #pragma unroll
    for (int v = 0; v < NV; ++v) {
        // lanes past the vector load its first elements and never use them (every sum and store below is guarded by
        // the lane's range): an unconditional load, where a choice between the loaded value and zeros made the
        // compiler wait for the first vector before it requested the next
        const int e0 = 256 * v + 4 * lane;
        h.x[v] = *(const float4 *)(src + (e0 < hd ? e0 : 0));
    }
    return h;
}
// The rotary table entries of the pairs this lane rotates (p = lane + 64 i), loaded ahead of their use.
template <int NV> struct RopeVals { float tab[2 * NV], ff[2 * NV]; };
template <int NV>
__device__ __forceinline__ RopeVals<NV> lg_rope_load(const float *rope_tab, const float *rope_ff, int hd) {
    const int lane = threadIdx.x & 63, half = hd >> 1;
    RopeVals<NV> r;
    #pragma unroll
    for (int i = 0; i < 2 * NV; ++i) {
        const int p = lane + 64 * i;
        r.tab[i] = p < half ? rope_tab[p] : 0.0f;
        r.ff[i] = (p < half && rope_ff) ? rope_ff[p] : 1.0f;
    }
    return r;
}
__device__ __forceinline__ void lg_wave_lds_sync() {
    // LDS serves one wavefront's accesses in order; the fences keep the compiler from reordering around it
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
// rmsnorm of a head vector (weighted by `w`, or plain) in the 256-lane sum order; the result stays in registers.
template <int NV>
__device__ __forceinline__ HeadVec<NV> lg_head_norm(HeadVec<NV> h, HeadVec<NV> w, bool weighted, int hd, float eps) {
    const int lane = threadIdx.x & 63;
    float ss0 = 0.0f, ss1 = 0.0f;                            // lanes l and l+64 of the 256-lane sum order
    if (4 * lane < hd) ss0 = lg_sumsq4(h.x[0], 0.0f);
    if (NV > 1 && 256 + 4 * lane < hd) ss1 = lg_sumsq4(h.x[NV - 1], 0.0f);
    const float ss = NV > 1 ? lg_wave_sum64(ss0) + lg_wave_sum64(ss1) : lg_wave_sum64(ss0);    // ss1 == 0 adds nothing
    const float sc = 1.0f / sqrtf(ss / (float)hd + eps);
    HeadVec<NV> r;
    #pragma unroll
    for (int v = 0; v < NV; ++v) {
        const float4 x = h.x[v], ww = w.x[v];
        if (weighted) r.x[v] = make_float4(x.x * sc * ww.x, x.y * sc * ww.y, x.z * sc * ww.z, x.w * sc * ww.w);
        else r.x[v] = make_float4(x.x * sc, x.y * sc, x.z * sc, x.w * sc);
    }
    return r;
}
template <int NV>
__device__ __forceinline__ void lg_head_store(const HeadVec<NV> &r, int hd, float *vec) {
    const int lane = threadIdx.x & 63;
    #pragma unroll
    for (int v = 0; v < NV; ++v) if (256 * v + 4 * lane < hd) *(float4 *)(vec + 256 * v + 4 * lane) = r.x[v];
    lg_wave_lds_sync();
}
// NeoX rotary at position `pos` of a normed vector: it goes through vec[0..hd) (LDS private to the wavefront,
// the pairs (p, p + hd/2) sit in different lanes), and out(p, lo, hi) receives the rotated pair p = lane + 64 i.
template <int NV, typename Out>
__device__ __forceinline__ void lg_head_rope(const HeadVec<NV> &r, int hd, int pos, const RopeVals<NV> &rv, float *vec, Out out) {
    const int lane = threadIdx.x & 63, half = hd >> 1;
    lg_head_store<NV>(r, hd, vec);
    #pragma unroll
    for (int i = 0; i < 2 * NV; ++i) {
        const int p = lane + 64 * i;
        if (p >= half) continue;
        const float ang = (float)pos * rv.tab[i] / rv.ff[i];
        float sn, cs;
        lg_sincosf(ang, &sn, &cs);
        const float x0 = vec[p], x1 = vec[p + half];
        out(p, x0 * cs - x1 * sn, x0 * sn + x1 * cs);
    }
}
// Both steps with the result left in vec.
template <int NV>
__device__ __forceinline__ void lg_head_finish(HeadVec<NV> h, HeadVec<NV> w, bool weighted, int hd, float eps, bool rope, int pos,
                                               const RopeVals<NV> &rv, float *vec) {
    const HeadVec<NV> r = lg_head_norm<NV>(h, w, weighted, hd, eps);
    if (rope) {
        const int half = hd >> 1;
        lg_head_rope<NV>(r, hd, pos, rv, vec, [&](int p, float lo, float hi) { vec[p] = lo; vec[p + half] = hi; });
        lg_wave_lds_sync();
    } else lg_head_store<NV>(r, hd, vec);
}

__global__ __launch_bounds__(64) void lg_k_qkv_post(QkvPostArgs a, const StepCtl *ctl) {
    __shared__ __align__(16) float vec[512];
    const int lane = threadIdx.x, job = blockIdx.x, j = blockIdx.y, hd = a.hd;
    const int pos = ctl->pos + j;
    const bool isq = job < a.H, isv = job >= a.H + a.nkv;
    const int head = isq ? job : (job - a.H) % a.nkv;
    const float *src = a.qkv + (size_t)j * a.ld + (isq ? (size_t)head * hd : (size_t)(isv ? a.v_off : a.k_off) + (size_t)head * hd);
    const float *w = isq ? a.q_norm : (isv ? nullptr : a.k_norm);
    const HeadVec<2> h = lg_head_load<2>(src, hd);
    const HeadVec<2> wv = w ? lg_head_load<2>(w, hd) : h;
    const RopeVals<2> rv = lg_rope_load<2>(a.rope_tab, a.rope_ff, hd);
    lg_head_finish<2>(h, wv, w != nullptr, hd, a.eps, !isv, pos, rv, vec);
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
// positions 32n..32n+31); for each (head, draft row, tile) a partial softmax (max, sum,
// V-accumulator) is written, merged afterwards in ascending tile order.
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
    int pos_off;             // added to the step position: -1 for a draft head, whose query at pos sees keys < pos
    // lg_k_attn<true> only: the raw q/k/v projections of the block and what lg_k_qkv_post would apply to them
    const float *qkv;        // [M][ld]: q at 0, k at k_off, v at v_off
    int ld, k_off, v_off;
    const float *q_norm, *k_norm, *rope_tab, *rope_ff;
    uint16_t *kcw, *vcw;     // this layer's own cache, to receive the block's rows (nullptr: it reads another layer's)
    float eps;
    int gx, gz;              // lg_k_attn: its launch dimensions x and z (as arguments they arrive with the others)
    __device__ __forceinline__ uint4 kc4(size_t off) const { return *(const uint4 *)(kc + off); }
    __device__ __forceinline__ uint4 vc4(size_t off) const { return *(const uint4 *)(vc + off); }
    // for the kernels that stage a tile once for all the rows of a block: no second reader, so non-temporal
    __device__ __forceinline__ uint4 kc4s(size_t off) const { return lg_ldw16(kc + off); }
    __device__ __forceinline__ uint4 vc4s(size_t off) const { return lg_ldw16(vc + off); }
};
#define LG_ATTN_FIELDS(X, v) X(int, gx, gx, v) X(int, gz, gz, v) X(int, hd, hd, v) X(int, window, window, v) X(int, pos_off, pos_off, v) X(int, seq, seq, v) X(int, kv_dim, kv_dim, v) X(const uint16_t *, kc, kc, v) X(const uint16_t *, vc, vc, v) X(int, H, H, v) X(int, nkv, nkv, v) X(const float *, qkv, qkv, v) X(const float *, q_norm, q_norm, v) X(const float *, k_norm, k_norm, v) X(const float *, rope_tab, rope_tab, v) X(const float *, rope_ff, rope_ff, v) X(int, ld, ld, v) X(int, k_off, k_off, v) X(int, v_off, v_off, v) X(uint16_t *, kcw, kcw, v) X(uint16_t *, vcw, vcw, v) X(const float *, q, q, v) X(float *, pm, pm, v) X(float *, pl, pl, v) X(float *, pacc, pacc, v) X(int, tiles_max, tiles_max, v) X(float, eps, eps, v)

__device__ __forceinline__ int lg_win_start(int pos, int window) {
    return (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
}

// One workgroup per (tile, kv head, draft row): the G = H/nkv query heads of the kv head's group.
// The score of (query g, key slot) is split over two lanes of the same wavefront (lane and lane^32):
// each runs two of the four partial chains, and the halves meet as (a0+a1)+(a2+a3).
//
// FQ: the block's raw projections are normed and rotated here instead of by lg_k_qkv_post (one launch less per
// layer; blocks of up to LG_HIP_MAX_ROWS_DEV rows; pos_off == 0 unless the layer owns no cache).  Every workgroup prepares its own row's G
// queries (wavefront g = head g).  The block's own K/V rows are not in the cache yet: a workgroup whose tile
// holds some of them builds the ones its row may see straight into the LDS tile (K row r by wavefront r % 4,
// V row r by wavefront 3 - r % 4), and the workgroups of the last row, which see all of them, also store them to the cache.
// The ring has at least LG_WIDE_ROWS spare rows, so no row another workgroup still reads is overwritten.
#define LG_ATTN_JOBS (2 * ((LG_HIP_MAX_ROWS_DEV + 3) / 4)) // K and V rows one wavefront may have to build
template <bool FQ, int NV>
__global__ __launch_bounds__(LG_WG, NV > 1 ? 2 : 4) void lg_k_attn(const StepCtl *ctl, LG_ATTN_FIELDS(LG_XP, _) int p_end_) {
    AttnArgs a; LG_ATTN_FIELDS(LG_XI, a)
    extern __shared__ __align__(16) unsigned char smem[];
    const int hd = a.hd, G = a.H / a.nkv;
    const int kst = hd + 8;                                   // padded V tile row (halves): 16-byte rows, read along the row
    // K is read down a column (32 lanes = 32 key slots, the same two dims): an odd row stride in dwords spreads
    // the slots over all 32 banks (a 16-byte-aligned stride leaves them 4 to a bank, and the score loop is
    // bound by exactly these reads); the price is 4-byte stores when the tile is staged
    const int ksk = hd + 2;                                   // K tile row (halves)
    float *qs = (float *)smem;                                // [G][hd]
    uint16_t *kt = (uint16_t *)(qs + (size_t)G * hd);         // [32][ksk]
    uint16_t *vt = kt + 32 * kst;                             // [32][kst]
    float *es = (float *)(vt + 32 * kst);                     // [G][32]
    float *hv = (float *)(smem + (((size_t)((unsigned char *)(es + G * 32 + G) - smem) + 15) & ~(size_t)15));   // FQ: [4 wavefronts][hd] staging
    // dispatched last rows and last tiles first: those hold the block's own K/V rows, the longest workgroups
    const int kvh = blockIdx.y, j = a.gz - 1 - (int)blockIdx.z, bx = a.gx - 1 - (int)blockIdx.x;
    const int pos0 = ctl->pos + a.pos_off, pj = pos0 + j;
    const int startj = lg_win_start(pj, a.window);
    const int n = (lg_win_start(pos0, a.window) >> 5) + bx;
    if (n < (startj >> 5) || n > (pj >> 5)) return;           // tile outside this row's keys
    const int t0 = n << 5;
    // FQ: positions tnew..pj of this tile are rows of the block itself (none when the layer reads another's cache)
    const int tnew = (FQ && a.kcw) ? ctl->pos : 0x7FFFFFFF;
    {   // stage q (G heads of this row) and the tile's K/V rows; loads are issued in groups ahead of
        // the LDS stores (named temporaries + scheduling barrier, see lg_copy_batched)
        const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
        const int per_row = hd >> 3, nk8 = 32 * per_row;     // 16-byte chunks per tile row / per tile
        // (per_row is a power of two and the tile's first ring row is wavefront-uniform: shifts and one scalar
        // remainder, where a division per element cost a hundred vector instructions ahead of the tile's loads)
        const int lgpr = 31 - __builtin_clz(per_row), ring0 = t0 % a.seq;
        // element u of the batch that starts at i0: LDS offset (halves) in `lo`, cache offset in `go`, validity in `ok`
        auto place = [&](int i0, int u, int &lo, int &lk, size_t &go, bool &ok, bool &own) {
            const int idx = min(i0 + u * LG_WG, nk8 - 1);
            const int sl = idx >> lgpr, e0 = (idx & (per_row - 1)) << 3, t = t0 + sl;
            ok = t >= startj && t <= pj;
            own = ok && t >= tnew;                            // a row of the block: built by `prepare`, not read from the cache
            ok = ok && !own;
            lo = sl * kst + e0; lk = sl * ksk + e0;
            // the slot's ring row, whether the row is live or not: what a dead slot holds is read and zeroed below
            int rr = ring0 + sl;
            if (rr >= a.seq) rr -= a.seq;
            if (rr >= a.seq) rr %= a.seq;                     // (rings of fewer than 32 rows)
            go = (size_t)rr * a.kv_dim + (size_t)kvh * hd + e0;
        };
        auto keep = [](uint4 v, bool ok) {                   // zero the rows no query of this block may see
            const uint32_t mk = ok ? 0xFFFFFFFFu : 0u;
            return make_uint4(v.x & mk, v.y & mk, v.z & mk, v.w & mk);
        };
        auto putk = [&](int lk, uint4 v) {                   // four 4-byte stores: K rows are only 4-byte aligned
            uint32_t *d = (uint32_t *)(kt + lk);
            d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
        };
        // The tile's first batch (all of it up to 256-wide heads) is requested before anything else of this block:
        // its addresses need nothing from memory, and placed after the row's vectors its address arithmetic reused
        // their registers and waited for them.
        int l0, l1, l2, l3, m0, m1, m2, m3; size_t g0, g1, g2, g3; bool ok0, ok1, ok2, ok3, ow0, ow1, ow2, ow3;
        place(threadIdx.x, 0, l0, m0, g0, ok0, ow0); place(threadIdx.x, 1, l1, m1, g1, ok1, ow1);
        place(threadIdx.x, 2, l2, m2, g2, ok2, ow2); place(threadIdx.x, 3, l3, m3, g3, ok3, ow3);
        const uint4 fk0 = a.kc4(g0), fk1 = a.kc4(g1), fk2 = a.kc4(g2), fk3 = a.kc4(g3);
        const uint4 fv0 = a.vc4(g0), fv1 = a.vc4(g1), fv2 = a.vc4(g2), fv3 = a.vc4(g3);
        __builtin_amdgcn_sched_barrier(0);
        HeadVec<NV> hq[2], hj[LG_ATTN_JOBS], wq, wk;
        RopeVals<NV> rv;
        int njobs = 0, r0 = 0;
        if (FQ) {                                             // all loads of this wavefront's vectors first
            const float *qrow = a.qkv + (size_t)j * a.ld + (size_t)kvh * G * hd;
            #pragma unroll
            for (int u = 0; u < 2; ++u) if (wv + 4 * u < G) hq[u] = lg_head_load<NV>(qrow + (size_t)(wv + 4 * u) * hd, hd);
            wq = lg_head_load<NV>(a.q_norm, hd);
            rv = lg_rope_load<NV>(a.rope_tab, a.rope_ff, hd);
            const int rlo = t0 > tnew ? t0 - tnew : 0, rhi = (t0 + 31 < pj ? t0 + 31 : pj) - tnew;   // block rows in this tile
            if (pj >= tnew && rhi >= rlo) { njobs = rhi - rlo + 1; r0 = rlo; }
            wk = lg_head_load<NV>(njobs == 0 ? a.q_norm : a.k_norm, hd);   // no K rows to build: k_norm may not exist (a choice of address, not of loaded values: that one waits for the loads)
            #pragma unroll
            for (int u = 0; u < LG_ATTN_JOBS; ++u) {          // slots 0,1: K rows wv, wv+4; slots 2,3: V rows 3-wv, 7-wv
                const bool isv = u >= LG_ATTN_JOBS / 2;
                const int rr = (isv ? 3 - wv : wv) + 4 * (u & 1);
                if (rr < njobs) hj[u] = lg_head_load<NV>(a.qkv + (size_t)(r0 + rr) * a.ld + (isv ? a.v_off : a.k_off) + (size_t)kvh * hd, hd);
            }
        } else {
            const float *qrow = a.q + (size_t)j * a.H * hd + (size_t)kvh * G * hd;
            lg_copy_batched<float4>((const float4 *)qrow, (float4 *)qs, G * (hd >> 2));
        }
        auto prepare = [&]() {                                // queries, then this wavefront's K or V rows of the block
            #pragma unroll
            for (int u = 0; u < 2; ++u)
                if (wv + 4 * u < G)
                    lg_head_finish<NV>(hq[u], wq, true, hd, a.eps, true, ctl->pos + j, rv, qs + (size_t)(wv + 4 * u) * hd);   // in place
            float *vec = hv + (size_t)wv * hd;
            const int half = hd >> 1;
            #pragma unroll
            for (int u = 0; u < LG_ATTN_JOBS; ++u) {
                const bool isv = u >= LG_ATTN_JOBS / 2;
                const int rr = (isv ? 3 - wv : wv) + 4 * (u & 1);
                if (rr >= njobs) continue;
                const int t = tnew + r0 + rr, sl = t - t0;
                const HeadVec<NV> r = lg_head_norm<NV>(hj[u], wk, !isv, hd, a.eps);
                const size_t coff = (size_t)(t % a.seq) * a.kv_dim + (size_t)kvh * hd;
                const bool wr_cache = blockIdx.z == 0;       // the last row's workgroups see every row of the block
                if (isv) {                                    // V: no rotary, straight from the registers
                    #pragma unroll
                    for (int v = 0; v < NV; ++v) {
                        const int e0 = 256 * v + 4 * lane;
                        if (e0 >= hd) continue;
                        const uint2 h4 = make_uint2((uint32_t)lg_f2h(r.x[v].x) | ((uint32_t)lg_f2h(r.x[v].y) << 16),
                                                    (uint32_t)lg_f2h(r.x[v].z) | ((uint32_t)lg_f2h(r.x[v].w) << 16));
                        *(uint2 *)(vt + sl * kst + e0) = h4;
                        if (wr_cache) *(uint2 *)(a.vcw + coff + e0) = h4;
                    }
                } else {
                    uint16_t *row = kt + sl * ksk, *crow = a.kcw + coff;
                    lg_head_rope<NV>(r, hd, t, rv, vec, [&](int p, float lo, float hi) {
                        const uint16_t hl = lg_f2h(lo), hh = lg_f2h(hi);
                        row[p] = hl; row[p + half] = hh;
                        if (wr_cache) { crow[p] = hl; crow[p + half] = hh; }
                    });
                }
            }
        };
        __builtin_amdgcn_sched_barrier(0);
        if (!ow0) { putk(m0, keep(fk0, ok0));  *(uint4 *)(vt + l0) = keep(fv0, ok0); }
        if (!ow1) { putk(m1, keep(fk1, ok1));  *(uint4 *)(vt + l1) = keep(fv1, ok1); }
        if (!ow2) { putk(m2, keep(fk2, ok2));  *(uint4 *)(vt + l2) = keep(fv2, ok2); }
        if (!ow3) { putk(m3, keep(fk3, ok3));  *(uint4 *)(vt + l3) = keep(fv3, ok3); }
        for (int i0 = threadIdx.x + 4 * LG_WG; i0 < nk8; i0 += 4 * LG_WG) {      // (512-wide heads: a second batch)
            place(i0, 0, l0, m0, g0, ok0, ow0); place(i0, 1, l1, m1, g1, ok1, ow1); place(i0, 2, l2, m2, g2, ok2, ow2); place(i0, 3, l3, m3, g3, ok3, ow3);
            const uint4 k0 = a.kc4(g0), k1 = a.kc4(g1), k2 = a.kc4(g2), k3 = a.kc4(g3);
            const uint4 v0 = a.vc4(g0), v1 = a.vc4(g1), v2 = a.vc4(g2), v3 = a.vc4(g3);
            __builtin_amdgcn_sched_barrier(0);
            if (!ow0) { putk(m0, keep(k0, ok0));  *(uint4 *)(vt + l0) = keep(v0, ok0); }
            if (!ow1) { putk(m1, keep(k1, ok1));  *(uint4 *)(vt + l1) = keep(v1, ok1); }
            if (!ow2) { putk(m2, keep(k2, ok2));  *(uint4 *)(vt + l2) = keep(v2, ok2); }
            if (!ow3) { putk(m3, keep(k3, ok3));  *(uint4 *)(vt + l3) = keep(v3, ok3); }
        }
        if (FQ) prepare();                                    // its loads were issued ahead of the tile's
    }
    __syncthreads();
    {   // scores, tile max, exp, tile sum
        const int sl = threadIdx.x & 31, part = threadIdx.x >> 5, t = t0 + sl;
        const bool valid = t >= startj && t <= pj;
        for (int unit = part; unit < 2 * G; unit += LG_WG / 32) {
            const int g = unit >> 1, hf = unit & 1;
            const float *qv = qs + (size_t)g * hd + 2 * hf;
            const uint16_t *kr = kt + sl * ksk + 2 * hf;
            float ax = 0.0f, ay = 0.0f;                       // chains 2hf and 2hf+1
            for (int i = 0; i < hd; i += 8) {
                const float2 q0 = *(const float2 *)(qv + i), q1 = *(const float2 *)(qv + i + 4);
                const uint32_t k0 = *(const uint32_t *)(kr + i), k1 = *(const uint32_t *)(kr + i + 4);
                ax = lg_fmaf(q0.x, lg_h2f((uint16_t)(k0 & 0xFFFF)), ax);
                ay = lg_fmaf(q0.y, lg_h2f((uint16_t)(k0 >> 16)), ay);
                ax = lg_fmaf(q1.x, lg_h2f((uint16_t)(k1 & 0xFFFF)), ax);
                ay = lg_fmaf(q1.y, lg_h2f((uint16_t)(k1 >> 16)), ay);
            }
            float s = lg_add_x32(ax + ay);                     // (a0+a1) + (a2+a3): the two halves sit 32 lanes apart
            if (!valid) s = -INFINITY;
            const float mx = lg_max_n(s, 32);
            const float e = valid ? lg_expf(s - mx) : 0.0f;
            const float l = lg_sum32(e);
            if (hf == 0) {
                es[g * 32 + sl] = e;
                if (sl == 0) {
                    const size_t pi = ((size_t)j * a.H + kvh * G + g) * a.tiles_max + bx;
                    a.pm[pi] = mx; a.pl[pi] = l;
                }
            }
        }
    }
    __syncthreads();
    // acc[d] = sum over valid slots of e * V[slot][d]; thread = (head g, 4 dims)
    // The valid slots of a tile are one run [lo, hi) (positions startj..pj), the same for every head of the
    // row: 8 slots are read at a time, clamped to the tile, and the fma of a slot past the run is skipped
    // by a wavefront-uniform test after all 16 reads are in flight.
    const int lo = startj > t0 ? startj - t0 : 0, hi = pj - t0 + 1 < 32 ? pj - t0 + 1 : 32;
    for (int unit = threadIdx.x; unit < G * (hd >> 2); unit += LG_WG) {
        const int g = unit / (hd >> 2), d0 = (unit - g * (hd >> 2)) << 2;
        float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        for (int sl0 = lo; sl0 < hi; sl0 += 8) {
            float e8[8]; uint2 v8[8];
            #pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int sl = sl0 + u < 32 ? sl0 + u : 31;
                e8[u] = es[g * 32 + sl];
                v8[u] = *(const uint2 *)(vt + sl * kst + d0);
            }
            #pragma unroll
            for (int u = 0; u < 8; ++u) {
                if (sl0 + u < hi) {
                    acc.x = lg_fmaf(e8[u], lg_h2f((uint16_t)(v8[u].x & 0xFFFF)), acc.x);
                    acc.y = lg_fmaf(e8[u], lg_h2f((uint16_t)(v8[u].x >> 16)), acc.y);
                    acc.z = lg_fmaf(e8[u], lg_h2f((uint16_t)(v8[u].y & 0xFFFF)), acc.z);
                    acc.w = lg_fmaf(e8[u], lg_h2f((uint16_t)(v8[u].y >> 16)), acc.w);
                }
            }
        }
        const size_t pi = ((size_t)j * a.H + kvh * G + g) * a.tiles_max + bx;
        *(float4 *)(a.pacc + pi * hd + d0) = acc;
    }
}

// Merge the tile partials of one (row, head) in ascending tile order, divide, quantize to q8.
struct MergeArgs {
    const float *pm, *pl, *pacc; int tiles_max;
    int H, hd, window, pos_off;
    int8_t *xq;                // q8 activation buffer of the attention output, width H*hd (input of attn_output)
    float *xf;                 // optional f32 copy [M][H*hd]
};
#define LG_MERGE_FIELDS(X, v) X(const float *, pm, pm, v) X(const float *, pl, pl, v) X(const float *, pacc, pacc, v) X(int, tiles_max, tiles_max, v) X(int, H, H, v) X(int, hd, hd, v) X(int, window, window, v) X(int, pos_off, pos_off, v) X(int8_t *, xq, xq, v) X(float *, xf, xf, v)
// The body for (head, row j) as a device function run by 256 threads numbered tid (the kernel below runs it per workgroup
// of its grid, lg_k_merge_o and lg_k_attn_tail as their first phase; a workgroup of 512 threads runs two at once, and
// every thread of the workgroup has to be inside one of them: the body synchronises the workgroup).  wts, pls: 512 floats of LDS each (exp(m_tile - M) and the sums of up to 512 tiles at a time), wmx: 4.
// after_first_fetch runs once the first batch of partials has been requested (a caller's own loads go behind it);
// sink(d, r, q, dq, sum) receives dim d's result, its q8 value and its block's scale and sum.  WIDE_OK = false: heads of at most 256 dims.
template <bool WIDE_OK = true, typename Hook, typename Sink>
__device__ __forceinline__ void lg_attn_merge_body(const StepCtl *ctl, const MergeArgs &a, int head, int j, int tid, float *wts, float *pls, float *wmx,
                                                   Hook &&after_first_fetch, Sink &&sink) {
    const int hd = a.hd;
    const int pos = ctl->pos + a.pos_off, pj = pos + j;
    const int first = lg_win_start(pos, a.window) >> 5;
    const int lo = (lg_win_start(pj, a.window) >> 5) - first, hi = (pj >> 5) - first;
    const size_t base = ((size_t)j * a.H + head) * a.tiles_max;
    // rows with at most one tile per thread (every sliding layer, global layers up to 8192 keys) read each tile's
    // maximum and sum once, with the pass that finds the row's maximum
    const bool once = hi - lo < LG_WG;
    const int mine = lo + tid <= hi ? lo + tid : hi;
    const float pm1 = a.pm[base + mine], pl1 = a.pl[base + mine];
    // a batch of partials is one memory round trip (they were written by other CUs a moment ago), so the batch is
    // made large enough to hold all the tiles of a sliding layer.  Buffer loads: the row's partials as the base in
    // scalar registers, the lane's dim as the lane offset, the tile's offset in a scalar register (as flat loads every
    // one of them cost a dozen vector instructions of 64-bit address arithmetic).  The first batch does not depend on
    // the weights and is requested here, with the maxima.
    constexpr int U = 24;
    float pau[U], pbu[U];                                     // dims 0..255, dims 256..511 (hd = 512 only)
    const bool wide = WIDE_OK && hd > LG_WG;                  // (a caller that never sees heads wider than 256 saves the second batch's registers)
    const int tl = tid < hd ? tid : hd - 1;   // (lanes past a short head repeat its last dim; their sums are never used)
    auto fetch = [&](int c0, int cn, int n0) {
        const __amdgpu_buffer_rsrc_t rp = lg_buffer_rsrc(a.pacc + (base + c0) * hd);
        #pragma unroll
        for (int u = 0; u < U; ++u) {
            const int n = __builtin_amdgcn_readfirstlane(n0 + u < cn ? n0 + u : cn - 1);
            pau[u] = __int_as_float(__builtin_amdgcn_raw_buffer_load_b32(rp, tl * 4, n * hd * 4, 0));
        }
        if (wide) {
            #pragma unroll
            for (int u = 0; u < U; ++u) {
                const int n = __builtin_amdgcn_readfirstlane(n0 + u < cn ? n0 + u : cn - 1);
                pbu[u] = __int_as_float(__builtin_amdgcn_raw_buffer_load_b32(rp, (LG_WG + tid) * 4, n * hd * 4, 0));
            }
        }
    };
    fetch(lo, hi - lo + 1 < 512 ? hi - lo + 1 : 512, 0);
    after_first_fetch();
    float mx = pm1;
    for (int n = lo + tid + LG_WG; n <= hi; n += LG_WG) mx = fmaxf(mx, a.pm[base + n]);
    mx = lg_max_n(mx, 64);
    if ((tid & 63) == 0) wmx[tid >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(wmx[0], wmx[1]), fmaxf(wmx[2], wmx[3]));
    float L = 0.0f, o[2] = { 0.0f, 0.0f };
    for (int c0 = lo; c0 <= hi; c0 += 512) {
        const int cn = hi - c0 + 1 < 512 ? hi - c0 + 1 : 512;
        if (once) {
            if (tid < cn) { wts[tid] = lg_expf(pm1 - mx); pls[tid] = pl1; }
        } else {
            __syncthreads();
            for (int n = tid; n < cn; n += LG_WG) { wts[n] = lg_expf(a.pm[base + c0 + n] - mx); pls[n] = a.pl[base + c0 + n]; }
        }
        __syncthreads();
        for (int n0 = 0; n0 < cn; n0 += U) {                  // fma in tile order
            if (c0 != lo || n0 != 0) fetch(c0, cn, n0);
            __builtin_amdgcn_sched_barrier(0);                // every load of the batch issued before the first fma waits
            #pragma unroll
            for (int u = 0; u < U; ++u) {
                if (n0 + u < cn) {                            // (a guard, not a break: the arrays stay in registers)
                    const float wn = wts[n0 + u];
                    L = lg_fmaf(pls[n0 + u], wn, L);
                    o[0] = lg_fmaf(pau[u], wn, o[0]);
                    if (wide) o[1] = lg_fmaf(pbu[u], wn, o[1]);
                }
            }
        }
    }
    #pragma unroll
    for (int h2 = 0; h2 < 2; ++h2) {
        const int d = h2 * LG_WG + tid;
        if (h2 * LG_WG >= hd) break;
        const float r = d < hd ? o[h2] / L : 0.0f;
        float dq; int sum;
        const int q = lg_quant1_32lanes(r, &dq, &sum);
        if (d < hd) sink(d, r, q, dq, sum);
    }
}
template <int M>
__global__ __launch_bounds__(LG_WG) void lg_k_attn_merge(const StepCtl *ctl, LG_MERGE_FIELDS(LG_XP, _) int p_end_) {
    MergeArgs a; LG_MERGE_FIELDS(LG_XI, a)
    __shared__ float wts[512], pls[512], wmx[LG_WG / 64];
    const int head = blockIdx.x, j = blockIdx.y, hd = a.hd, qd = a.H * hd;
    lg_attn_merge_body(ctl, a, head, j, (int)threadIdx.x, wts, pls, wmx, [] {}, [&](int d, float r, int q, float dq, int sum) {
        const int e = head * hd + d;                           // element of the row, natural order
        a.xq[lg_q8_off<M>(qd, j, e >> 4, e & 15)] = (int8_t)q;          // order the attn_output matmul reads
        if ((d & 31) == 0) lg_q8_ds<M>(a.xq, qd)[lg_q8_ds_idx<M>(qd, j, e >> 5)] = make_float2(dq, __int_as_float(sum));
        if (a.xf) a.xf[(size_t)j * qd + e] = r;
    });
}
