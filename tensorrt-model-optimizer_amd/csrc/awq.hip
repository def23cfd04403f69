// Kernels behind AWQ-lite and SmoothQuant for gfx950: per-channel scaling, the fused
// scale -> block amax -> INT-N quantize-dequantize of a weight, column statistics and the
// squared-error loss.  All HBM-bound except the search GEMM, which is not in this file.
#include "common.h"
#include "awq_ops.h"

namespace mo {

template <int DT>
__device__ __forceinline__ float round_to(float v) {
    if constexpr (DT == MO_BF16) return round_to_bf16(v);
    else if constexpr (DT == MO_F16) return f16_bits_to_f32(f32_to_f16_bits(v));
    else return v;
}

// 8 consecutive scale values s[c0 .. c0 + 8) as fp32 (c0 % 8 == 0, s 16-byte aligned)
__device__ __forceinline__ void load_scales8(const void* s, int s_dtype, int64_t c0, float (&f)[8]) {
    if (s_dtype == MO_F32) load_chunk<MO_F32>(s, c0, f);
    else if (s_dtype == MO_F16) load_chunk<MO_F16>(s, c0, f);
    else load_chunk<MO_BF16>(s, c0, f);
}

// y[r, c] = T( f32(x[r, c]) * f32(s[c]) )   (bf16 * bf16 -> bf16 and bf16 * fp32 -> fp32 -> bf16
// both reduce to one fp32 product rounded once to T).
// Vector path (k % 8 == 0, aligned): a workgroup owns kMulRows rows of 256 column chunks; a lane
// loads its chunk of every row and the scales of its 8 columns first, in straight-line code,
// then multiplies and stores -- no load is issued behind a store, which it would have to wait
// for.  (Conditional stores would do for the short last slab, but the compiler then sinks a
// row's load into the block of its store; the short slab has a path of its own instead.)
constexpr int kMulRows = 8;
template <int DT, int SD>
__global__ __launch_bounds__(256) void mul_cols8_kernel(const void* __restrict__ x, int64_t rows,
                                                        int64_t k, int64_t col_groups,
                                                        const void* __restrict__ s,
                                                        void* __restrict__ y) {
    const int64_t slab = (int64_t)blockIdx.x / col_groups;
    const int64_t group = (int64_t)blockIdx.x - slab * col_groups;
    const int64_t col = (group * 256 + threadIdx.x) << 3;
    if (col >= k) return;
    const int64_t r0 = slab * kMulRows;
    RawChunk<SD> sraw;
    load_raw<SD>(s, col, sraw);
    if (r0 + kMulRows <= rows) {
        RawChunk<DT> raw[kMulRows];
#pragma unroll
        for (int u = 0; u < kMulRows; ++u) load_raw<DT>(x, (r0 + u) * k + col, raw[u]);
        float sc[8];
        unpack_raw<SD>(sraw, sc);
#pragma unroll
        for (int u = 0; u < kMulRows; ++u) {
            float v[8];
            unpack_raw<DT>(raw[u], v);
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] *= sc[j];
            store_chunk<DT>(y, (r0 + u) * k + col, v);
        }
    } else {
        // the last, short slab of the tensor: row by row
        float sc[8];
        unpack_raw<SD>(sraw, sc);
        for (int64_t r = r0; r < rows; ++r) {
            float v[8];
            load_chunk<DT>(x, r * k + col, v);
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] *= sc[j];
            store_chunk<DT>(y, r * k + col, v);
        }
    }
}

template <int DT>
__global__ __launch_bounds__(256) void mul_cols_kernel(const void* __restrict__ x, int64_t rows,
                                                       int64_t k, const void* __restrict__ s,
                                                       int s_dtype, void* __restrict__ y) {
    const int64_t kc = (k + 7) >> 3, total = rows * kc;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += stride) {
        const int64_t r = t / kc, c0 = (t - r * kc) << 3;
        float v[8];
        load_chunk_guarded<DT>(x, r * k, c0, k, v);
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if (c0 + j < k) v[j] *= load_scalar(s, s_dtype, c0 + j);
        store_chunk_guarded<DT>(y, r * k, c0, k, v);
    }
}

// Static block INT-N fake quantisation along the last axis with an optional per-column
// pre-scale, fused:  xs = T(x * s[c]);  amax = max |xs| over each block of `bs` columns (zero
// padded);  scale = bound / f32(amax) (amax <= 2^-24 -> output 0);
// y = T( clamp(rne(f32(xs) * scale), lo, bound) / scale ).
// A lane owns a chunk of 8 columns; the G = bs / 8 lanes of a block share the amax by shuffles.
// The division is the exact reciprocal-and-FMA quotient whenever the scale is mid-range.
constexpr int kQdqRounds = 4;          // chunks per lane (2 measures the same, 1 is 10 % slower)
constexpr int kQdqTileChunks = 256 * kQdqRounds;

template <int DT, bool VEC>
__global__ __launch_bounds__(256) void scale_block_int_qdq_kernel(
    const void* __restrict__ x, int64_t rows, int64_t k, const void* __restrict__ s, int s_dtype,
    int lg_g, float bound, float lo, void* __restrict__ y) {
    const int G = 1 << lg_g;
    const int64_t bs = (int64_t)G << 3;
    const int64_t kp = (k + bs - 1) / bs * bs, kc = kp >> 3, total = rows * kc;
    // one workgroup per tile of 256 * kQdqRounds chunks; total and the tile size are multiples
    // of G, so the lanes of a block stay together and are all live or all idle
    const int64_t t0 = (int64_t)blockIdx.x * kQdqTileChunks + threadIdx.x;
    int64_t r[kQdqRounds], c0[kQdqRounds];
    RawChunk<DT> raw[kQdqRounds];
    float v[kQdqRounds][8];
#pragma unroll
    for (int u = 0; u < kQdqRounds; ++u) {
        const int64_t t = t0 + u * 256;
        r[u] = c0[u] = 0;
        zero_raw<DT>(raw[u]);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[u][j] = 0.0f;
        if (t < total) {
            if (total <= 0xFFFFFFFFll) r[u] = (uint32_t)t / (uint32_t)kc; else r[u] = t / kc;
            c0[u] = (t - r[u] * kc) << 3;
            if (VEC) load_raw<DT>(x, r[u] * k + c0[u], raw[u]);
            else load_chunk_guarded<DT>(x, r[u] * k, c0[u], k, v[u]);
        }
    }
#pragma unroll
    for (int u = 0; u < kQdqRounds; ++u) {
        const bool live = t0 + u * 256 < total;
        if (VEC) unpack_raw<DT>(raw[u], v[u]);
        if (s && live) {
            if (VEC) {
                float sc[8];
                load_scales8(s, s_dtype, c0[u], sc);
#pragma unroll
                for (int j = 0; j < 8; ++j) v[u][j] = round_to<DT>(v[u][j] * sc[j]);
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    if (c0[u] + j < k)
                        v[u][j] = round_to<DT>(v[u][j] * load_scalar(s, s_dtype, c0[u] + j));
            }
        }
        block_int_qdq_chunk(v[u], lg_g, bound, lo);
        if (!live) continue;
        if (VEC) store_chunk<DT>(y, r[u] * k + c0[u], v[u]);
        else store_chunk_guarded<DT>(y, r[u] * k, c0[u], k, v[u]);
    }
}

// The same for the aligned case (k a multiple of the block, 16-byte aligned operands), where
// chunk t of the tensor is elements [8 t, 8 t + 8): all loads of a lane -- its kQdqRounds chunks
// and their scales -- are issued first, in straight-line code (a lane past the end re-reads the
// last chunk and does not store), so nothing waits behind a store.  SD is the dtype of the
// scale vector, -1 without one.
template <int DT, int SD>
__global__ __launch_bounds__(256) void scale_block_int_qdq_vec_kernel(
    const void* __restrict__ x, int64_t total, int64_t kc, const void* __restrict__ s, int lg_g,
    float bound, float lo, void* __restrict__ y) {
    constexpr int SDT = SD < 0 ? MO_BF16 : SD;
    const int64_t t0 = (int64_t)blockIdx.x * kQdqTileChunks + threadIdx.x;
    const int64_t last = total - 1;
    RawChunk<DT> raw[kQdqRounds];
    RawChunk<SDT> sraw[kQdqRounds];
    // column chunk of the first item by one division, of the others by stepping
    int64_t cc = 0;
    if constexpr (SD >= 0) {
        const int64_t tt = t0 < last ? t0 : last;
        cc = total <= 0xFFFFFFFFll ? (int64_t)((uint32_t)tt % (uint32_t)kc) : tt % kc;
    }
    const int64_t step = 256 % kc;
#pragma unroll
    for (int u = 0; u < kQdqRounds; ++u) {
        const int64_t t = t0 + u * 256;
        load_raw<DT>(x, (t < last ? t : last) << 3, raw[u]);
        if constexpr (SD >= 0) {
            load_raw<SDT>(s, cc << 3, sraw[u]);
            cc += step;
            cc = cc >= kc ? cc - kc : cc;
        }
    }
#pragma unroll
    for (int u = 0; u < kQdqRounds; ++u) {
        const int64_t t = t0 + u * 256;
        float v[8];
        unpack_raw<DT>(raw[u], v);
        if constexpr (SD >= 0) {
            float sc[8];
            unpack_raw<SDT>(sraw[u], sc);
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = round_to<DT>(v[j] * sc[j]);
        }
        block_int_qdq_chunk(v, lg_g, bound, lo);
        if (t <= last) store_chunk<DT>(y, t << 3, v);
    }
}

// acc[c] += sum over rows of f32( T( |x[r, c]| / T(f32(blk_amax[r, c / bs]) + tiny) ) ) when
// blk_amax is given, else of |x[r, c]|.  One thread per column over a slab of rows.
template <int DT>
__global__ __launch_bounds__(256) void abs_colsum_kernel(const void* __restrict__ x, int64_t rows,
                                                         int64_t k, const float* __restrict__ blk_amax,
                                                         int64_t bs, int64_t slab,
                                                         float* __restrict__ acc) {
    const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= k) return;
    const int64_t r0 = (int64_t)blockIdx.y * slab;
    int64_t r1 = r0 + slab;
    if (r1 > rows) r1 = rows;
    const int64_t nb = blk_amax ? (k + bs - 1) / bs : 0;
    // smallest positive normal of T, as torch.finfo(T).tiny
    const float tiny = DT == MO_F16 ? 6.103515625e-05f : 1.17549435e-38f;
    float sum = 0.0f;
    for (int64_t r = r0; r < r1; ++r) {
        float v = __builtin_fabsf(load_elem<DT>(x, r * k + c));
        if (blk_amax) {
            float d = blk_amax[r * nb + c / bs] + tiny;
            if constexpr (DT == MO_BF16) d = bf16_bits_to_f32(f32_to_bf16_bits(d));
            else if constexpr (DT == MO_F16) d = f16_bits_to_f32(f32_to_f16_bits(d));
            v = v / d;
            if constexpr (DT == MO_BF16) v = bf16_bits_to_f32(f32_to_bf16_bits(v));
            else if constexpr (DT == MO_F16) v = f16_bits_to_f32(f32_to_f16_bits(v));
        }
        sum += v;
    }
    atomicAdd(acc + c, sum);
}

// The same sums for k % 8 == 0 (and bs % 8 == 0), without atomics: a lane owns 8 adjacent columns
// and walks down a slab of rows, four 16-byte loads in flight; the workgroup of slab blockIdx.y
// stores its sums to row blockIdx.y of partial[slabs, k], and a second pass adds those rows to
// acc in a fixed order.  The block abs-max of a chunk is one value, so the division becomes one
// reciprocal per chunk and the exact FMA-corrected quotient per element.
template <int DT, bool WITH_AMAX>
__global__ __launch_bounds__(256) void abs_colsum8_kernel(const void* __restrict__ x, int64_t rows,
                                                          int64_t k, const float* __restrict__ blk_amax,
                                                          int64_t bs, int64_t slab,
                                                          float* __restrict__ partial) {
    const int64_t col = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
    if (col >= k) return;
    const int64_t r0 = (int64_t)blockIdx.y * slab;
    int64_t r1 = r0 + slab;
    if (r1 > rows) r1 = rows;
    const int64_t nb = WITH_AMAX ? k / bs : 0, cb = WITH_AMAX ? col / bs : 0;
    const float tiny = DT == MO_F16 ? 6.103515625e-05f : 1.17549435e-38f;
    float sum[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    auto add_row = [&](const RawChunk<DT>& raw, float amax) {
        float v[8];
        unpack_raw<DT>(raw, v);
        if constexpr (WITH_AMAX) {
            const float d = round_to<DT>(amax + tiny);
            const float r = 1.0f / d;
            if (mid_range(d)) {     // |x| <= amax <= d: the quotient cannot overflow
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float a = __builtin_fabsf(v[j]);
                    float q = exact_quotient(a, d, r);   // NaN stays NaN
                    // the correction steps are exact only while nothing underflows
                    if (q < 1.0e-30f && a > 0.0f) {
                        keep_branch();
                        q = a / d;
                    }
                    sum[j] += round_to<DT>(q);
                }
            } else {
                keep_branch();
#pragma unroll
                for (int j = 0; j < 8; ++j) sum[j] += round_to<DT>(__builtin_fabsf(v[j]) / d);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) sum[j] += __builtin_fabsf(v[j]);
        }
    };
    int64_t r = r0;
    constexpr int U = DT == MO_F32 ? 4 : 8;   // rows (16- or 32-byte loads) in flight per lane
    for (; r + U - 1 < r1; r += U) {
        RawChunk<DT> raw[U];
        float am[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            load_raw<DT>(x, (r + u) * k + col, raw[u]);
            am[u] = WITH_AMAX ? blk_amax[(r + u) * nb + cb] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) add_row(raw[u], am[u]);
    }
    for (; r < r1; ++r) {
        RawChunk<DT> raw;
        load_raw<DT>(x, r * k + col, raw);
        add_row(raw, WITH_AMAX ? blk_amax[r * nb + cb] : 0.0f);
    }
    f32x4* out = (f32x4*)(partial + (int64_t)blockIdx.y * k + col);
    const f32x4 a = {sum[0], sum[1], sum[2], sum[3]}, b = {sum[4], sum[5], sum[6], sum[7]};
    out[0] = a;
    out[1] = b;
}

// abs_colsum8_kernel<DT, true> with the block abs-max taken from x itself: the G = bs / 8 lanes
// that own a block of a row exchange the maxima of their chunks (bit patterns, so a NaN wins
// as in torch's amax).  One pass over the weight instead of two and no amax array.
//
// bf16: |x| and d = T(amax + tiny) have 8-bit significands, so the exact quotient differs from
// every rounding boundary of bf16 by at least 1 / (255 * 512) of its value unless it lies on
// one, which it cannot (the boundary's odd 9-bit numerator would have to divide the 8-bit
// numerator of |x|).  A quotient good to 2^-22 -- |x| times the hardware reciprocal -- therefore
// rounds to the same bf16 value as the correctly rounded fp32 quotient does; only quotients in
// fp32's denormal range, where that error bound does not hold, take the division.
#ifndef MO_WS_U
#define MO_WS_U 4
#endif
template <int DT>
__global__ __launch_bounds__(256) void weight_scale_colsum8_kernel(const void* __restrict__ x,
                                                                   int64_t rows, int64_t k, int lg_g,
                                                                   int64_t slab,
                                                                   float* __restrict__ partial) {
    const int64_t col = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
    if (col >= k) return;   // k is a multiple of the block: its lanes leave together
    const int64_t r0 = (int64_t)blockIdx.y * slab;
    int64_t r1 = r0 + slab;
    if (r1 > rows) r1 = rows;
    const float tiny = DT == MO_F16 ? 6.103515625e-05f : 1.17549435e-38f;
    float sum[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    auto add_row = [&](const RawChunk<DT>& raw) {
        float v[8];
        unpack_raw<DT>(raw, v);
        float amax;
        if constexpr (DT == MO_F32) {
            uint32_t m = 0;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t b = f2u(v[j]) & 0x7FFFFFFFu;
                m = b > m ? b : m;
            }
            amax = u2f(group_max_u32(m, lg_g));
        } else {
            const uint32_t mask = 0x7FFF7FFFu;
            const uint32_t p = pk_max_u16(pk_max_u16(raw.a.x & mask, raw.a.y & mask),
                                          pk_max_u16(raw.a.z & mask, raw.a.w & mask));
            uint32_t m = p & 0xFFFFu;
            m = (p >> 16) > m ? (p >> 16) : m;
            m = group_max_u32(m, lg_g);
            amax = DT == MO_BF16 ? u2f(m << 16) : f16_bits_to_f32(m);
        }
        const float d = round_to<DT>(amax + tiny);
        if (mid_range(d)) {     // |x| <= amax <= d: the quotient cannot overflow
            if constexpr (DT == MO_BF16) {
                const float r = __builtin_amdgcn_rcpf(d);
                float q[8];
                bool denormal = false;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    q[j] = __builtin_fabsf(v[j]) * r;                  // NaN stays NaN
                    denormal |= __builtin_amdgcn_classf(q[j], 0x80);   // positive denormal
                }
                if (denormal) {     // one branch per chunk; rare
                    keep_branch();
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        if (__builtin_amdgcn_classf(q[j], 0x80)) q[j] = __builtin_fabsf(v[j]) / d;
                }
                // the pair (0, q) converted leaves bf16(q) as an fp32 bit pattern
#pragma unroll
                for (int j = 0; j < 8; ++j) sum[j] += u2f(f32x2_to_bf16x2(0.0f, q[j]));
            } else {
                const float r = 1.0f / d;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float a = __builtin_fabsf(v[j]);
                    float q = exact_quotient(a, d, r);
                    // the correction steps are exact only while nothing underflows
                    if (q < 1.0e-30f && a > 0.0f) {
                        keep_branch();
                        q = a / d;
                    }
                    sum[j] += round_to<DT>(q);
                }
            }
        } else {
            keep_branch();
#pragma unroll
            for (int j = 0; j < 8; ++j) sum[j] += round_to<DT>(__builtin_fabsf(v[j]) / d);
        }
    };
    int64_t r = r0;
    constexpr int U = DT == MO_F32 ? MO_WS_U / 2 : MO_WS_U;   // rows (16- or 32-byte loads) in flight per lane
    for (; r + U - 1 < r1; r += U) {
        RawChunk<DT> raw[U];
#pragma unroll
        for (int u = 0; u < U; ++u) load_raw<DT>(x, (r + u) * k + col, raw[u]);
#pragma unroll
        for (int u = 0; u < U; ++u) add_row(raw[u]);
    }
    for (; r < r1; ++r) {
        RawChunk<DT> raw;
        load_raw<DT>(x, r * k + col, raw);
        add_row(raw);
    }
    f32x4* out = (f32x4*)(partial + (int64_t)blockIdx.y * k + col);
    const f32x4 a = {sum[0], sum[1], sum[2], sum[3]}, b = {sum[4], sum[5], sum[6], sum[7]};
    out[0] = a;
    out[1] = b;
}

// acc[c] += sum over the rows of partial[rows, k] (k % 4 == 0).  A workgroup owns 64 columns:
// lane = (column quad, one of 16 row groups); a group adds rows g, g + 16, ... in that order,
// four 16-byte loads in flight, and the groups are combined through LDS in group order -- a
// fixed order for a given shape, by one writer per column.
__global__ __launch_bounds__(256) void colsum_fold_partials_kernel(const float* __restrict__ partial,
                                                                   int64_t rows, int64_t k,
                                                                   float* __restrict__ acc) {
    __shared__ f32x4 smem[16][16];
    const int cq = threadIdx.x & 15, g = threadIdx.x >> 4;
    const int64_t col = ((int64_t)blockIdx.x * 16 + cq) * 4;
    f32x4 s = {0.0f, 0.0f, 0.0f, 0.0f};
    if (col < k) {
        int64_t r = g;
        for (; r + 48 < rows; r += 64) {
            f32x4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = *(const f32x4*)(partial + (r + 16 * u) * k + col);
#pragma unroll
            for (int u = 0; u < 4; ++u) s += v[u];
        }
        for (; r < rows; r += 16) s += *(const f32x4*)(partial + r * k + col);
    }
    smem[g][cq] = s;
    __syncthreads();
    if (g == 0 && col < k) {
#pragma unroll
        for (int i = 1; i < 16; ++i) s += smem[i][cq];
        f32x4* out = (f32x4*)(acc + col);
        *out = *out + s;
    }
}

// acc[0] += sum of f32( T(a[i] - b[i]) )^2.  Lanes sum 8-element chunks in fp32, the grid
// combines in double (one atomic per workgroup).
template <int DT>
__global__ __launch_bounds__(256) void sq_diff_sum_kernel(const void* __restrict__ a,
                                                          const void* __restrict__ b, int64_t n,
                                                          int vec, double* __restrict__ acc) {
    __shared__ double smem[4];
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    double sum = 0.0;
    if (vec) {
        const int64_t chunks = n >> 3;
        // 4 chunks of each operand in flight per lane
        for (int64_t c = tid; c < chunks; c += 4 * stride) {
            RawChunk<DT> ra[4], rb[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int64_t cu = c + u * stride;
                zero_raw<DT>(ra[u]);
                zero_raw<DT>(rb[u]);
                if (cu < chunks) {
                    load_raw<DT>(a, cu << 3, ra[u]);
                    load_raw<DT>(b, cu << 3, rb[u]);
                }
            }
            float part = 0.0f;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                float va[8], vb[8];
                unpack_raw<DT>(ra[u], va);
                unpack_raw<DT>(rb[u], vb);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float d = round_to<DT>(va[j] - vb[j]);
                    part += d * d;
                }
            }
            sum += part;
        }
        if (tid < (n & 7)) {
            const int64_t i = (chunks << 3) + tid;
            const float d = round_to<DT>(load_elem<DT>(a, i) - load_elem<DT>(b, i));
            sum += d * d;
        }
    } else {
        for (int64_t i = tid; i < n; i += stride) {
            const float d = round_to<DT>(load_elem<DT>(a, i) - load_elem<DT>(b, i));
            sum += d * d;
        }
    }
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, kWave);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) smem[wave] = sum;
    __syncthreads();
    if (threadIdx.x == 0) atomicAdd(acc, smem[0] + smem[1] + smem[2] + smem[3]);
}

static inline unsigned blocks_for_awq(int64_t items, int64_t cap = 16384) {
    int64_t b = (items + 255) / 256;
    if (b < 1) b = 1;
    if (b > cap) b = cap;
    return (unsigned)b;
}


// ------------------------------------------------------------------------------ scale grid
// The candidate scales of a whole alpha grid: one workgroup per alpha.  Pass 1 writes the clamped
// quotients to `scales` and reduces their maximum and minimum; pass 2 divides every element
// (each lane re-reads what it wrote itself) by sqrt(max * min) and writes the two rounded copies.
__device__ __forceinline__ float grid_power(float base, float exponent, int mode) {
    if (mode == 1) return 1.0f;                      // exponent 0
    if (mode == 2) return base;                      // exponent 1
    if (mode == 3) return __builtin_sqrtf(base);     // exponent 0.5: correctly rounded root
    // the device math library's pow, the one the tensor library calls: the compiler builtin's
    // result differs from it in the last place now and then
    return powf(base, exponent);
}

template <int DT>
__global__ __launch_bounds__(1024) void awq_scale_grid_kernel(
    const float* __restrict__ x_max, const float* __restrict__ w_max,
    const float* __restrict__ exponents, int n_alpha, int k, float* __restrict__ scales,
    void* __restrict__ w_scales, void* __restrict__ x_scales) {
    __shared__ float red_max[16], red_min[16];
    __shared__ int red_nan[16];
    const int a = blockIdx.x;
    const float ea = exponents[a], eb = exponents[n_alpha + a];
    const int ma = (int)exponents[2 * n_alpha + a], mb = (int)exponents[3 * n_alpha + a];
    float* row = scales + (int64_t)a * k;
    float hi = 0.0f, lo = 3.0e38f;
    int nan = 0;
    for (int c = threadIdx.x; c < k; c += blockDim.x) {
        const float num = grid_power(x_max[c], ea, ma);
        const float den = grid_power(w_max[c], eb, mb) + 1.17549435e-38f;
        float v = num / den;
        v = v < 1e-4f ? 1e-4f : v;
        v = v > 1e4f ? 1e4f : v;
        row[c] = v;
        if (v != v) nan = 1;
        else { hi = v > hi ? v : hi; lo = v < lo ? v : lo; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float h2 = __shfl_xor(hi, o, kWave), l2 = __shfl_xor(lo, o, kWave);
        hi = h2 > hi ? h2 : hi;
        lo = l2 < lo ? l2 : lo;
        nan |= __shfl_xor(nan, o, kWave);
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    if (lane == 0) { red_max[wave] = hi; red_min[wave] = lo; red_nan[wave] = nan; }
    __syncthreads();
    for (int w = 0; w < waves; ++w) {
        hi = red_max[w] > hi ? red_max[w] : hi;
        lo = red_min[w] < lo ? red_min[w] : lo;
        nan |= red_nan[w];
    }
    const float norm = nan ? __builtin_nanf("") : __builtin_sqrtf(hi * lo);
    for (int c = threadIdx.x; c < k; c += blockDim.x) {
        const float v = row[c] / norm;
        row[c] = v;
        if (w_scales) store_elem<DT>(w_scales, (int64_t)a * k + c, v);
        if (x_scales) store_elem<DT>(x_scales, (int64_t)a * k + c, 1.0f / v);
    }
}

// The row of the candidate-scale grid whose loss is the first smallest one (what
// min(dict, key=dict.get) picks on the host: a NaN is never smaller than anything, and a NaN in
// front is never replaced), its index, and the three tensors the folding makes of it.  Every
// thread scans the few losses itself; no exchange between workgroups.
template <int DT>
__global__ __launch_bounds__(256) void awq_pick_scale_kernel(
    const double* __restrict__ loss, int n_alpha, const float* __restrict__ scales, int k,
    int64_t* __restrict__ best, float* __restrict__ best_scale, float* __restrict__ pre_quant_scale,
    void* __restrict__ pre_quant_scale_t, float* __restrict__ fold) {
    int b = 0;
    double lowest = loss[0];
    for (int i = 1; i < n_alpha; ++i) {
        const double v = loss[i];
        if (v < lowest) {
            lowest = v;
            b = i;
        }
    }
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c == 0 && best) best[0] = b;
    if (c >= k) return;
    const float s = scales[(int64_t)b * k + c];
    const float p = 1.0f / s;
    if (best_scale) best_scale[c] = s;
    if (pre_quant_scale) pre_quant_scale[c] = p;
    if (pre_quant_scale_t) store_elem<DT>(pre_quant_scale_t, c, p);
    if (fold) fold[c] = 1.0f / p;
}

// SmoothQuant's per-channel scale and everything the smoothing makes of it, one workgroup:
//   ws = T(w_col[c]);  s[c] = f32(T(ws ^ (1 - alpha))) / act[c] ^ alpha          (fp32 division)
//   if min_c s[c] <= 2^-31: s[c] = 1 where act[c] <= 2^-31;  s[c] = clamp(s[c], 1e-4, 1e4)
//   rounded[c] = T(s[c]);  fold[c] = 1 / s[c]
//   act_max = T(max_c act[c]);  smoothed_max = T(max_c f32(T(act[c])) * s[c])
// with the NaN behaviour of the tensor expressions: a NaN scale makes the minimum NaN (no channel
// is reset), passes the clamp, and a NaN operand makes a maximum NaN.
template <int DT>
__global__ __launch_bounds__(1024) void smooth_scales_kernel(
    const float* __restrict__ act, const float* __restrict__ w_col, int k, float exp_w, int mode_w,
    float exp_a, int mode_a, float* __restrict__ scale, void* __restrict__ rounded,
    float* __restrict__ fold, void* __restrict__ act_max, void* __restrict__ smoothed_max) {
    __shared__ float red_a[16], red_b[16];
    __shared__ int red_nan[16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    auto to_t = [](float v) {
        if constexpr (DT == MO_BF16) return round_to_bf16(v);
        else if constexpr (DT == MO_F16) return f16_bits_to_f32(f32_to_f16_bits(v));
        else return v;
    };
    // a = running minimum of the scales, b = running maximum of act; NaNs are carried by flags
    float lo = __builtin_inff(), hi = -__builtin_inff();
    int nan_s = 0, nan_a = 0;
    for (int c = threadIdx.x; c < k; c += blockDim.x) {
        const float a = act[c];
        const float num = to_t(grid_power(to_t(w_col[c]), exp_w, mode_w));
        const float v = num / grid_power(a, exp_a, mode_a);
        scale[c] = v;
        if (v != v) nan_s = 1; else lo = v < lo ? v : lo;
        if (a != a) nan_a = 1; else hi = a > hi ? a : hi;
    }
    auto meet = [&](float& x, float& y, int& flags, bool x_is_min) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float x2 = __shfl_xor(x, o, kWave), y2 = __shfl_xor(y, o, kWave);
            x = x_is_min ? (x2 < x ? x2 : x) : (x2 > x ? x2 : x);
            y = y2 > y ? y2 : y;
            flags |= __shfl_xor(flags, o, kWave);
        }
        __syncthreads();   // the arrays may still be read from the meeting before
        if (lane == 0) { red_a[wave] = x; red_b[wave] = y; red_nan[wave] = flags; }
        __syncthreads();
        for (int w = 0; w < waves; ++w) {
            x = x_is_min ? (red_a[w] < x ? red_a[w] : x) : (red_a[w] > x ? red_a[w] : x);
            y = red_b[w] > y ? red_b[w] : y;
            flags |= red_nan[w];
        }
    };
    int flags = nan_s | (nan_a << 1);
    meet(lo, hi, flags, true);
    const bool reset_dead = !(flags & 1) && lo <= 4.656612873077393e-10f;   // 2^-31
    if (threadIdx.x == 0 && act_max)
        store_elem<DT>(act_max, 0, (flags & 2) ? __builtin_nanf("") : hi);
    float top = -__builtin_inff(), unused = 0.0f;
    int nan_p = 0;
    for (int c = threadIdx.x; c < k; c += blockDim.x) {
        const float a = act[c];
        float v = scale[c];   // each lane re-reads what it wrote itself
        if (reset_dead && a <= 4.656612873077393e-10f) v = 1.0f;
        v = v < 1e-4f ? 1e-4f : v;
        v = v > 1e4f ? 1e4f : v;
        scale[c] = v;
        if (rounded) store_elem<DT>(rounded, c, v);
        if (fold) fold[c] = 1.0f / v;
        const float p = to_t(a) * v;
        if (p != p) nan_p = 1; else top = p > top ? p : top;
    }
    meet(top, unused, nan_p, false);
    if (threadIdx.x == 0 && smoothed_max)
        store_elem<DT>(smoothed_max, 0, nan_p ? __builtin_nanf("") : top);
}

}  // namespace mo

#define DISPATCH_DT(dtype, CALL)          \
    switch (dtype) {                      \
        case MO_F32: CALL(MO_F32); break; \
        case MO_F16: CALL(MO_F16); break; \
        case MO_BF16: CALL(MO_BF16); break; \
        default: return MO_ERR_DTYPE;     \
    }

extern "C" int mo_mul_cols(const void* x, int64_t rows, int64_t k, int dtype, const void* s,
                           int s_dtype, void* y, void* stream) {
    if (rows < 0 || k < 0) return MO_ERR_ARG;
    if (s_dtype < MO_F32 || s_dtype > MO_BF16) return MO_ERR_DTYPE;
    if (rows == 0 || k == 0) return MO_OK;
    if (!x || !s || !y) return MO_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    const bool vec = (k % 8 == 0) && ((((uintptr_t)x | (uintptr_t)y | (uintptr_t)s) & 15u) == 0);
    if (vec) {
        const int64_t gx = (k / 8 + 255) / 256;
        const int64_t blocks = gx * ((rows + mo::kMulRows - 1) / mo::kMulRows);
        if (blocks > 0x7FFFFFFF) return MO_ERR_UNSUPPORTED;
#define CALL_SD(DT, SD) \
    mo::mul_cols8_kernel<DT, SD><<<(unsigned)blocks, 256, mo::ballast_bytes("mul_cols8_kernel", 36), st>>>(x, rows, k, gx, s, y)
#define CALL(DT)                                     \
    if (s_dtype == MO_F32) CALL_SD(DT, MO_F32);      \
    else if (s_dtype == MO_F16) CALL_SD(DT, MO_F16); \
    else CALL_SD(DT, MO_BF16)
        DISPATCH_DT(dtype, CALL)
#undef CALL
#undef CALL_SD
    } else {
        const unsigned g = mo::blocks_for_awq(rows * ((k + 7) >> 3));
#define CALL(DT) mo::mul_cols_kernel<DT><<<g, 256, 0, st>>>(x, rows, k, s, s_dtype, y)
        DISPATCH_DT(dtype, CALL)
#undef CALL
    }
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_scale_block_int_qdq(const void* x, int64_t rows, int64_t k, int dtype,
                                      const void* s, int s_dtype, int64_t block_size, int num_bits,
                                      int is_unsigned, int narrow_range, void* y, void* stream) {
    if (rows < 0 || k < 0 || num_bits < 1 || num_bits > 24) return MO_ERR_ARG;
    if (s_dtype < MO_F32 || s_dtype > MO_BF16) return MO_ERR_DTYPE;
    int lg = 0;
    while ((8 << lg) < block_size && lg < 6) ++lg;
    if ((8 << lg) != block_size) return MO_ERR_UNSUPPORTED;  // 8, 16, ..., 512
    if (rows == 0 || k == 0) return MO_OK;
    if (!x || !y) return MO_ERR_ARG;
    const float bound = (float)((1 << (num_bits - 1 + (is_unsigned ? 1 : 0))) - 1);
    const float lo = is_unsigned ? 0.0f : (narrow_range ? -bound : -bound - 1.0f);
    hipStream_t st = (hipStream_t)stream;
    const int64_t kp = (k + block_size - 1) / block_size * block_size;
    const int64_t total = rows * (kp >> 3);
    const int64_t blocks = (total + mo::kQdqTileChunks - 1) / mo::kQdqTileChunks;
    if (blocks > 0x7FFFFFFF) return MO_ERR_UNSUPPORTED;
    const bool vec = (k % block_size == 0) &&
                     ((((uintptr_t)x | (uintptr_t)y | (uintptr_t)s) & 15u) == 0);
    const unsigned g = (unsigned)blocks;
    const size_t cap = mo::ballast_bytes("scale_block_int_qdq_kernel", 0);
    if (vec) {
        const int64_t kc = k >> 3;
#define CALL_SD(DT, SD)                                                                          \
    mo::scale_block_int_qdq_vec_kernel<DT, SD><<<g, 256, cap, st>>>(x, total, kc, s, lg, bound, lo, y)
#define CALL(DT)                                                                                 \
    if (!s) CALL_SD(DT, -1);                                                                     \
    else if (s_dtype == MO_F32) CALL_SD(DT, MO_F32);                                             \
    else if (s_dtype == MO_F16) CALL_SD(DT, MO_F16);                                             \
    else CALL_SD(DT, MO_BF16)
        DISPATCH_DT(dtype, CALL)
#undef CALL
#undef CALL_SD
        return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
    }
#define CALL(DT)                                                                                      \
    mo::scale_block_int_qdq_kernel<DT, false><<<g, 256, cap, st>>>(x, rows, k, s, s_dtype, lg, bound, lo, y)
    DISPATCH_DT(dtype, CALL)
#undef CALL
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_abs_colsum(const void* x, int64_t rows, int64_t k, int dtype,
                             const float* blk_amax, int64_t block_size, float* acc, void* stream) {
    if (rows < 0 || k < 0 || (blk_amax && block_size <= 0)) return MO_ERR_ARG;
    if (rows == 0 || k == 0) return MO_OK;
    if (!x || !acc) return MO_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    const int64_t gx = (k + 255) / 256;
    int64_t gy = (1024 + gx - 1) / gx;
    int64_t slab = (rows + gy - 1) / gy;
    if (slab < 8) slab = 8;
    gy = (rows + slab - 1) / slab;
    dim3 grid((unsigned)gx, (unsigned)gy);
#define CALL(DT) mo::abs_colsum_kernel<DT><<<grid, 256, 0, st>>>(x, rows, k, blk_amax, block_size, slab, acc)
    DISPATCH_DT(dtype, CALL)
#undef CALL
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_sq_diff_sum(const void* a, const void* b, int64_t n, int dtype, double* acc,
                              void* stream) {
    if (n < 0) return MO_ERR_ARG;
    if (n == 0) return MO_OK;
    if (!a || !b || !acc) return MO_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    // every workgroup ends with one atomic on the same double: 8 chunks per lane before a second
    // workgroup is worth its atomic, and never more than 1024 of them
    // a grid-stride pass by two workgroups per CU: 5.5 - 6.7 TB/s from 134 MB to 470 MB of operands
    // (1024 workgroups: 4.8 - 5.9, 4096: 3.8 - 5.4)
    const unsigned g = mo::blocks_for_awq((n + 63) / 64, (unsigned)mo::tuned("sq_diff_workgroups", 512));
    const int vec = ((((uintptr_t)a | (uintptr_t)b) & 15u) == 0) ? 1 : 0;
#define CALL(DT) mo::sq_diff_sum_kernel<DT><<<g, 256, mo::ballast_bytes("sq_diff_sum_kernel", 53), st>>>(a, b, n, vec, acc)
    DISPATCH_DT(dtype, CALL)
#undef CALL
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

// mo_abs_colsum without atomics (two passes through a caller-provided workspace of
// partial_rows x k floats); MO_ERR_UNSUPPORTED unless k % 8 == 0, block_size % 8 == 0 (when
// blk_amax is given, which also needs block_size to divide k) and the buffers are 16-byte aligned.
extern "C" int mo_abs_colsum_staged(const void* x, int64_t rows, int64_t k, int dtype,
                                    const float* blk_amax, int64_t block_size, float* acc,
                                    float* partial, int64_t partial_rows, void* stream) {
    if (rows < 0 || k < 0 || partial_rows < 1) return MO_ERR_ARG;
    if (dtype < MO_F32 || dtype > MO_BF16) return MO_ERR_DTYPE;
    if (rows == 0 || k == 0) return MO_OK;
    if (!x || !acc || !partial) return MO_ERR_ARG;
    if (k % 8 || ((((uintptr_t)x | (uintptr_t)partial | (uintptr_t)acc) & 15u) != 0))
        return MO_ERR_UNSUPPORTED;
    if (blk_amax && (block_size <= 0 || block_size % 8 || k % block_size)) return MO_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    int64_t slabs = partial_rows < 65535 ? partial_rows : 65535;
    const int64_t slab = (rows + slabs - 1) / slabs;
    slabs = (rows + slab - 1) / slab;
    const dim3 grid((unsigned)((k / 8 + 255) / 256), (unsigned)slabs);
#define CALL(DT)                                                                                  \
    if (blk_amax)                                                                                 \
        mo::abs_colsum8_kernel<DT, true><<<grid, 256, mo::ballast_bytes("abs_colsum8_kernel", 0), st>>>(x, rows, k, blk_amax, block_size,  \
                                                               slab, partial);                    \
    else                                                                                          \
        mo::abs_colsum8_kernel<DT, false><<<grid, 256, mo::ballast_bytes("abs_colsum8_kernel", 0), st>>>(x, rows, k, blk_amax, block_size, \
                                                                slab, partial)
    DISPATCH_DT(dtype, CALL)
#undef CALL
    mo::colsum_fold_partials_kernel<<<(unsigned)((k + 63) / 64), 256, 0, st>>>(partial, slabs, k, acc);
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

// Column sums of |x| / T(block abs-max + tiny) with the block abs-max computed in the same pass
// (two launches: slab sums, then the fold of the partial rows in a fixed order).
extern "C" int mo_weight_scale_colsum(const void* x, int64_t rows, int64_t k, int dtype,
                                      int64_t block_size, float* acc, float* partial,
                                      int64_t partial_rows, void* stream) {
    if (rows < 0 || k < 0 || partial_rows < 1 || block_size <= 0) return MO_ERR_ARG;
    if (dtype < MO_F32 || dtype > MO_BF16) return MO_ERR_DTYPE;
    int lg_g = 0;
    while (lg_g < 6 && (8ll << lg_g) < block_size) ++lg_g;
    if ((8ll << lg_g) != block_size || k % block_size) return MO_ERR_UNSUPPORTED;
    if (rows == 0 || k == 0) return MO_OK;
    if (!x || !acc || !partial) return MO_ERR_ARG;
    if ((((uintptr_t)x | (uintptr_t)partial | (uintptr_t)acc) & 15u) != 0) return MO_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    int64_t slabs = partial_rows < 65535 ? partial_rows : 65535;
    const int64_t slab = (rows + slabs - 1) / slabs;
    slabs = (rows + slab - 1) / slab;
    const dim3 grid((unsigned)((k / 8 + 255) / 256), (unsigned)slabs);
#define CALL(DT)                                                                              \
    mo::weight_scale_colsum8_kernel<DT>                                                       \
        <<<grid, 256, mo::ballast_bytes("weight_scale_colsum8_kernel", 0), st>>>(x, rows, k, lg_g, \
                                                                                 slab, partial)
    DISPATCH_DT(dtype, CALL)
#undef CALL
    mo::colsum_fold_partials_kernel<<<(unsigned)((k + 63) / 64), 256, 0, st>>>(partial, slabs, k, acc);
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

// The AWQ-lite candidate scales for every alpha of the search grid in one launch.
extern "C" int mo_awq_scale_grid(const float* x_max, const float* w_max, const float* exponents,
                                 int64_t n_alpha, int64_t k, float* scales, void* w_scales,
                                 void* x_scales, int dtype, void* stream) {
    if (n_alpha < 0 || k < 0) return MO_ERR_ARG;
    if (dtype < MO_F32 || dtype > MO_BF16) return MO_ERR_DTYPE;
    if (n_alpha == 0 || k == 0) return MO_OK;
    if (!x_max || !w_max || !exponents || !scales) return MO_ERR_ARG;
    if (n_alpha > 65535 || k > 0x7FFFFFFF) return MO_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    const int threads = k >= 4096 ? 1024 : 256;
#define CALL(DT)                                                                                   \
    mo::awq_scale_grid_kernel<DT><<<(unsigned)n_alpha, threads, 0, st>>>(                          \
        x_max, w_max, exponents, (int)n_alpha, (int)k, scales, w_scales, x_scales)
    DISPATCH_DT(dtype, CALL)
#undef CALL
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_awq_pick_scale(const double* loss, int64_t n_alpha, const float* scales, int64_t k,
                                 int64_t* best, float* best_scale, float* pre_quant_scale,
                                 void* pre_quant_scale_t, float* fold, int dtype, void* stream) {
    if (n_alpha < 0 || k < 0) return MO_ERR_ARG;
    if (dtype < MO_F32 || dtype > MO_BF16) return MO_ERR_DTYPE;
    if (n_alpha == 0) return MO_ERR_ARG;   // nothing to pick from
    if (!loss || (k && !scales)) return MO_ERR_ARG;
    if (n_alpha > 65535 || k > 0x7FFFFFFF) return MO_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    const unsigned blocks = k ? (unsigned)((k + 255) / 256) : 1u;
#define CALL(DT)                                                                          \
    mo::awq_pick_scale_kernel<DT><<<blocks, 256, 0, st>>>(loss, (int)n_alpha, scales, (int)k, best, \
                                                          best_scale, pre_quant_scale,   \
                                                          pre_quant_scale_t, fold)
    DISPATCH_DT(dtype, CALL)
#undef CALL
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_smooth_scales(const float* act_amax, const float* weight_col_amax, int64_t k,
                                float exp_w, int mode_w, float exp_a, int mode_a, int dtype,
                                float* pre_quant_scale, void* pre_quant_scale_t, float* fold,
                                void* act_amax_max, void* smoothed_amax, void* stream) {
    if (k < 0 || mode_w < 0 || mode_w > 3 || mode_a < 0 || mode_a > 3) return MO_ERR_ARG;
    if (dtype < MO_F32 || dtype > MO_BF16) return MO_ERR_DTYPE;
    if (k == 0) return MO_ERR_ARG;   // a maximum over nothing
    if (!act_amax || !weight_col_amax || !pre_quant_scale) return MO_ERR_ARG;
    if (k > 0x7FFFFFFF) return MO_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    const int threads = k >= 4096 ? 1024 : 256;
#define CALL(DT)                                                                                    \
    mo::smooth_scales_kernel<DT><<<1, threads, 0, st>>>(act_amax, weight_col_amax, (int)k, exp_w, mode_w, \
                                                        exp_a, mode_a, pre_quant_scale, pre_quant_scale_t, \
                                                        fold, act_amax_max, smoothed_amax)
    DISPATCH_DT(dtype, CALL)
#undef CALL
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}
