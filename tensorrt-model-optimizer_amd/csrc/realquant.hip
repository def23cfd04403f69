// Real (storage) quantisation kernels for gfx950: FP8 / INT8 element casts with scales, the
// INT4 block quantise+pack of the weight-compress path and the INT4 row-pair pack of the AWQ
// export path, plus their inverses.  All HBM-bound elementwise work.
#include "common.h"

namespace mo {

// Round an fp32 value through the dtype torch's type promotion gives the quotient / product.
template <int VIA>
__device__ __forceinline__ float round_via(float v) {
    if constexpr (VIA == MO_BF16) return bf16_bits_to_f32(f32_to_bf16_bits(v));
    else if constexpr (VIA == MO_F16) return f16_bits_to_f32(f32_to_f16_bits(v));
    else return v;
}

__device__ __forceinline__ uint32_t to_int8_byte(float v) {
    float q = __builtin_rintf(v);
    q = q < -128.0f ? -128.0f : q;
    q = q > 127.0f ? 127.0f : q;
    // NaN: torch's float -> int8 cast of NaN is 0 on x86 after the clamp left it NaN
    int i = (q == q) ? (int)q : 0;
    return (uint32_t)i & 0xFFu;
}

// q[i] = fmt( via( f32(x[i]) / f32(scale[a(i)]) ) ),  a(i) = (i / inner) % axis
template <int DT, int VIA, int FMT>
__global__ __launch_bounds__(256) void real_quantize_kernel(const void* __restrict__ x, int64_t n,
                                                            int64_t axis, int64_t inner,
                                                            const void* __restrict__ scale,
                                                            int scale_dtype,
                                                            uint8_t* __restrict__ out) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const bool uniform = axis == 1;
    const float s0 = load_scalar(scale, scale_dtype, 0);
    for (int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; (c << 3) < n; c += stride) {
        const int64_t i0 = c << 3;
        uint32_t lo = 0, hi = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int64_t i = i0 + j;
            uint32_t b = 0;
            if (i < n) {
                const float s = uniform ? s0 : load_scalar(scale, scale_dtype, (i / inner) % axis);
                const float v = round_via<VIA>(load_elem<DT>(x, i) / s);
                b = FMT == 0 ? f32_to_e4m3<false>(v) : to_int8_byte(v);
            }
            if (j < 4) lo |= b << (8 * j); else hi |= b << (8 * (j - 4));
        }
        if (i0 + 8 <= n && (((uintptr_t)out & 7u) == 0)) {
            u32x2 o = {lo, hi};
            *(u32x2*)(out + i0) = o;
        } else {
            for (int j = 0; j < 8 && i0 + j < n; ++j)
                out[i0 + j] = (uint8_t)((j < 4 ? lo >> (8 * j) : hi >> (8 * (j - 4))) & 0xFFu);
        }
    }
}

// y[i] = T( f32(T(q[i])) * f32(T(scale[a(i)])) )
template <int DT, int FMT>
__global__ __launch_bounds__(256) void real_dequantize_kernel(const uint8_t* __restrict__ q,
                                                              int64_t n, int64_t axis,
                                                              int64_t inner,
                                                              const void* __restrict__ scale,
                                                              int scale_dtype,
                                                              void* __restrict__ y) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const float s = round_via<DT>(load_scalar(scale, scale_dtype, axis == 1 ? 0 : (i / inner) % axis));
        const float v = FMT == 0 ? e4m3_to_f32(q[i]) : (float)(int8_t)q[i];
        store_elem<DT>(y, i, round_via<DT>(v) * s);
    }
}

// ------------------------------------------------------------------------------ tiled fast paths
// 16-byte aligned tensors whose scale is shared by the 8 elements of a chunk (per tensor, or
// inner % 8 == 0).  One workgroup per tile of 1024 chunks, 4 per lane, loads issued before the
// math.  The quotient x / s comes from one reciprocal per chunk and the exact FMA correction
// whenever the scale is in range and the largest quotient of the chunk cannot overflow; the
// sign of a zero quotient is restored from x (s is positive on that path).
constexpr int kRealTileChunks = 1024;

// Scale indices of the lane's chunks c0 + 256 u (u < U): one division for the first, the others
// by stepping (256 = step_r * inner_chunks + step_c, at most u carries).
template <int U>
__device__ __forceinline__ void chunk_scale_indices(int64_t c0, int64_t chunks, int64_t inner_chunks,
                                                    int64_t axis, int64_t (&idx)[U]) {
    int64_t row0;
    if (chunks <= 0xFFFFFFFFll) row0 = (uint32_t)c0 / (uint32_t)inner_chunks;
    else row0 = c0 / inner_chunks;
    const int64_t col0 = c0 - row0 * inner_chunks;
    const int64_t step_r = 256 / inner_chunks, step_c = 256 - step_r * inner_chunks;
#pragma unroll
    for (int u = 0; u < U; ++u) {
        int64_t row = row0 + u * step_r, col = col0 + u * step_c;
#pragma unroll
        for (int i = 0; i < u; ++i)
            if (col >= inner_chunks) { col -= inner_chunks; ++row; }
        idx[u] = row < axis ? row : row % axis;
    }
}

// Which scale a chunk takes, three ways (SCALES):
//   kScalePerTensor  one scale; a tile is 1024 consecutive chunks of the flat tensor
//   kScalePerRowTile rows of at least 2048 elements: a workgroup stays inside one row (the last
//                    tile of a row may be short), so the scale, its reciprocal and the range
//                    checks are wavefront-uniform (scalar) as in the per-tensor case
//   kScalePerChunk   anything else: each lane finds the rows of its chunks
//   kScalePerRound   (dequantizer) rows whose length is a multiple of 2048 elements: tiles of
//                    the flat tensor as in the per-tensor case (no half-empty tiles on
//                    4096-wide rows), and the 256 chunks of a round lie inside one row, so the
//                    scale of a round is wavefront-uniform
//   kScalePerBlock2d one scale per two-dimensional block of a matrix: `inner_chunks` is the
//                    length of a matrix row in chunks, `axis` the rows of a block and
//                    `tiles_per_row` the chunks across a block; the scale of the chunk at
//                    (row, col) is scale[(row / axis) * (inner_chunks / tiles_per_row) + col /
//                    tiles_per_row]
constexpr int kScalePerTensor = 0, kScalePerRowTile = 1, kScalePerChunk = 2, kScalePerRound = 3,
              kScalePerBlock2d = 4;

// chunk index, validity and scale of the lane's 4 chunks.  A chunk past the end gets the index
// of the last valid one and ok = false: the kernels load it like any other (all loads in
// straight-line code ahead of the first store, so that no round waits behind a store) and skip
// only its store.
template <int SCALES>
__device__ __forceinline__ void tile_layout(int64_t chunks, int64_t axis, int64_t inner_chunks,
                                            int64_t tiles_per_row, const void* scale,
                                            int scale_dtype, int64_t (&c)[4], bool (&ok)[4],
                                            float (&sv)[4]) {
    if constexpr (SCALES == kScalePerRowTile) {
        const int64_t row = (int64_t)blockIdx.x / tiles_per_row;
        const int64_t tile = (int64_t)blockIdx.x - row * tiles_per_row;
        const float s0 = load_scalar(scale, scale_dtype, row < axis ? row : row % axis);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t local = tile * kRealTileChunks + threadIdx.x + u * 256;
            ok[u] = local < inner_chunks;
            c[u] = row * inner_chunks + (ok[u] ? local : inner_chunks - 1);
            sv[u] = s0;
        }
    } else {
        const int64_t c0 = (int64_t)blockIdx.x * kRealTileChunks + threadIdx.x;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            ok[u] = c0 + u * 256 < chunks;
            c[u] = ok[u] ? c0 + u * 256 : chunks - 1;
        }
        if constexpr (SCALES == kScalePerTensor) {
            sv[0] = sv[1] = sv[2] = sv[3] = load_scalar(scale, scale_dtype, 0);
        } else if constexpr (SCALES == kScalePerRound) {
            // row of the tile's first chunk by one division, of the later rounds by stepping
            // (a round is 256 chunks and a row at least that); rounds past the end of the
            // tensor read some valid scale and store nothing
            const int64_t base = (int64_t)blockIdx.x * kRealTileChunks;
            int64_t row = chunks <= 0xFFFFFFFFll ? (int64_t)((uint32_t)base / (uint32_t)inner_chunks)
                                                 : base / inner_chunks;
            int64_t col = base - row * inner_chunks;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                sv[u] = load_scalar(scale, scale_dtype, row < axis ? row : row % axis);
                col += 256;
                if (col >= inner_chunks) { col -= inner_chunks; ++row; }
            }
        } else if constexpr (SCALES == kScalePerBlock2d) {
            const int64_t across = inner_chunks / tiles_per_row;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int64_t row = c[u] / inner_chunks, col = c[u] - row * inner_chunks;
                sv[u] = load_scalar(scale, scale_dtype, (row / axis) * across + col / tiles_per_row);
            }
        } else {
            int64_t idx[4];
            chunk_scale_indices<4>(c0, chunks, inner_chunks, axis, idx);
#pragma unroll
            for (int u = 0; u < 4; ++u) sv[u] = load_scalar(scale, scale_dtype, idx[u]);
        }
    }
}

template <int DT, int VIA, int FMT, int SCALES>
__global__ __launch_bounds__(256) void real_quantize_tile_kernel(
    const void* __restrict__ x, int64_t chunks, int64_t axis, int64_t inner_chunks,
    int64_t tiles_per_row, const void* __restrict__ scale, int scale_dtype,
    u32x2* __restrict__ out) {
    int64_t cs[4];
    bool ok[4];
    float sv[4];
    tile_layout<SCALES>(chunks, axis, inner_chunks, tiles_per_row, scale, scale_dtype, cs, ok, sv);
    RawChunk<DT> raw[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        // one scale per long row: a row shorter than the tile leaves whole rounds without work,
        // and skipping their loads is worth more than straight-line code (4096-wide rows use
        // half a tile: 30.0 against 30.7 us per 117 MB with the loads skipped)
        if (SCALES == kScalePerRowTile && !ok[u]) {
            zero_raw<DT>(raw[u]);
            continue;
        }
        load_raw<DT>(x, cs[u] << 3, raw[u]);
    }
    float v[4][8];
    float rv = 1.0f;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int64_t c = cs[u];
        // a row of fewer than 1024 chunks leaves part of its workgroup without work: those
        // lanes skip the arithmetic too (only the loads are unconditional)
        if (!ok[u]) continue;
        unpack_raw<DT>(raw[u], v[u]);
        const float s = sv[u];
        // bf16 / bf16 rounded to bf16: both significands have 8 bits, so the exact quotient stays
        // 2^-17 of its value away from every rounding boundary of bf16 (and is never on one) and
        // x times the hardware reciprocal, good to 2^-22, rounds to the same bf16 value as the
        // correctly rounded fp32 quotient.  Where that product is an fp32 denormal the bound
        // does not hold, but both roundings are then far below half the smallest E4M3 / INT8
        // step and give the same (signed) zero.
        const bool narrow = DT == MO_BF16 && VIA == MO_BF16 && (f2u(s) & 0xFFFFu) == 0u;
        float r;
        if (narrow) {
            r = __builtin_amdgcn_rcpf(s);
        } else {
            // the correctly rounded reciprocal (an IEEE division) is taken again only when the
            // scale changes
            if ((SCALES != kScalePerChunk && SCALES != kScalePerBlock2d) || u == 0 || f2u(s) != f2u(sv[u - 1])) rv = 1.0f / s;
            r = rv;
        }
        uint32_t m = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t t = f2u(v[u][j]) & 0x7FFFFFFFu;
            m = t > m ? t : m;
        }
        float q[8];
        const bool fast = mid_range(s) && u2f(m) * r < 1.0e38f;  // a NaN element fails the comparison
        if (fast && narrow) {
#pragma unroll
            for (int j = 0; j < 8; ++j) q[j] = v[u][j] * r;
        } else if (fast) {
#pragma unroll
            for (int j = 0; j < 8; ++j)
                q[j] = __builtin_copysignf(exact_quotient(v[u][j], s, r), v[u][j]);
        } else {
            keep_branch();
#pragma unroll
            for (int j = 0; j < 8; ++j) q[j] = v[u][j] / s;
        }
        uint32_t lo = 0, hi = 0;
        if (FMT == 1 && fast) {
            // finite quotients: clamp with v_med3, round to nearest even by adding 1.5 * 2^23,
            // and the low byte of the sum's mantissa is the two's-complement int8
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float a = __builtin_amdgcn_fmed3f(round_via<VIA>(q[j]), -128.0f, 127.0f);
                const float b = __builtin_amdgcn_fmed3f(round_via<VIA>(q[4 + j]), -128.0f, 127.0f);
                lo |= (f2u(a + 12582912.0f) & 0xFFu) << (8 * j);
                hi |= (f2u(b + 12582912.0f) & 0xFFu) << (8 * j);
            }
        } else if constexpr (FMT == 0) {
            lo = f32x2_to_e4m3x2(round_via<VIA>(q[0]), round_via<VIA>(q[1])) |
                 (f32x2_to_e4m3x2(round_via<VIA>(q[2]), round_via<VIA>(q[3])) << 16);
            hi = f32x2_to_e4m3x2(round_via<VIA>(q[4]), round_via<VIA>(q[5])) |
                 (f32x2_to_e4m3x2(round_via<VIA>(q[6]), round_via<VIA>(q[7])) << 16);
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                lo |= to_int8_byte(round_via<VIA>(q[j])) << (8 * j);
                hi |= to_int8_byte(round_via<VIA>(q[4 + j])) << (8 * j);
            }
        }
        const u32x2 o = {lo, hi};
        __builtin_nontemporal_store(o, out + c);
    }
}

template <int DT, int FMT, int SCALES>
__global__ __launch_bounds__(256) void real_dequantize_tile_kernel(
    const u32x2* __restrict__ q, int64_t chunks, int64_t axis, int64_t inner_chunks,
    int64_t tiles_per_row, const void* __restrict__ scale, int scale_dtype, void* __restrict__ y) {
    int64_t cs[4];
    bool ok[4];
    float sv[4];
    tile_layout<SCALES>(chunks, axis, inner_chunks, tiles_per_row, scale, scale_dtype, cs, ok, sv);
    u32x2 w[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        // (as in the quantizer: rounds past the end of a short row are not loaded)
        w[u] = u32x2{0u, 0u};
        if (SCALES == kScalePerRowTile && !ok[u]) continue;
        w[u] = __builtin_nontemporal_load(q + cs[u]);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int64_t c = cs[u];
        if (!ok[u]) continue;
        const float s = round_via<DT>(sv[u]);
        float v[8];
        // every E4M3 value and every int8 value is exact in bf16, fp16 and fp32
        if constexpr (FMT == 0) {
            const f32pair p0 = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[u].x, false);
            const f32pair p1 = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[u].x, true);
            const f32pair p2 = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[u].y, false);
            const f32pair p3 = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[u].y, true);
            v[0] = p0.x; v[1] = p0.y; v[2] = p1.x; v[3] = p1.y;
            v[4] = p2.x; v[5] = p2.y; v[6] = p3.x; v[7] = p3.y;
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                v[j] = (float)(int8_t)(w[u].x >> (8 * j));
                v[4 + j] = (float)(int8_t)(w[u].y >> (8 * j));
            }
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] *= s;
        store_chunk<DT>(y, c << 3, v);
    }
}

// ------------------------------------------------------------------------------ INT4 compress
// Flat blocks of `bs` elements (the tail block zero padded); one thread per block.
//   scale = T( f32(T(1 / amax)) * 7 )            (torch evaluates `7 / amax` as reciprocal * 7)
//   q     = clamp(rne(T(x * scale)), -8, 7) + 8
//   byte  = q[2i] << 4 | q[2i + 1]
template <int DT>
__global__ __launch_bounds__(256) void int4_block_quantize_kernel(const void* __restrict__ x,
                                                                  int64_t n, int64_t bs,
                                                                  int64_t nblocks,
                                                                  void* __restrict__ scales,
                                                                  int scales_given,
                                                                  uint8_t* __restrict__ packed) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; b < nblocks; b += stride) {
        const int64_t i0 = b * bs;
        uint32_t m = 0;
        for (int64_t j = 0; j < bs; ++j) {
            const float v = i0 + j < n ? load_elem<DT>(x, i0 + j) : 0.0f;
            const uint32_t t = f2u(v) & 0x7FFFFFFFu;
            m = t > m ? t : m;
        }
        const float amax = u2f(m);
        float scale = round_via<DT>(round_via<DT>(1.0f / amax) * 7.0f);
        if (scales_given) scale = load_elem<DT>(scales, b);
        else store_elem<DT>(scales, b, scale);
        for (int64_t j = 0; j < bs; j += 2) {
            uint32_t nib[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const float v = i0 + j + h < n ? load_elem<DT>(x, i0 + j + h) : 0.0f;
                float q = __builtin_rintf(round_via<DT>(v * scale));
                q = q < -8.0f ? -8.0f : q;
                q = q > 7.0f ? 7.0f : q;
                q += 8.0f;
                nib[h] = (q == q) ? ((uint32_t)(int)q & 0xFFu) : 0u;
            }
            packed[(i0 + j) >> 1] = (uint8_t)(((nib[0] << 4) | nib[1]) & 0xFFu);
        }
    }
}

// y[i] = T( f32(nibble - 8) / f32(scale[block]) ), high nibble first
template <int DT>
__global__ __launch_bounds__(256) void int4_block_dequantize_kernel(
    const uint8_t* __restrict__ packed, int64_t nbytes, int64_t bs, const void* __restrict__ scales,
    void* __restrict__ y) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nbytes; i += stride) {
        const uint32_t b = packed[i];
        const float s = load_elem<DT>(scales, (2 * i) / bs);
        store_elem<DT>(y, 2 * i, ((float)(int)(b >> 4) - 8.0f) / s);
        store_elem<DT>(y, 2 * i + 1, ((float)(int)(b & 0xFu) - 8.0f) / s);
    }
}

// ------------------------------------------------------------------------------ INT4 AWQ export
// w[N, K], ws[N, K / bs] fp32; q = int8(clamp(rne(f32(w) / ws), -8, 7));
// out[j, k] = (q[2j, k] & 0xF) | (q[2j + 1, k] << 4).  A lane packs 8 columns of a row pair.
// NARROW: the scales came in the weight's own 16-bit type, so the tensor division of the
// reference rounds the quotient to that type before it is rounded to an integer.
template <int DT, bool NARROW>
__global__ __launch_bounds__(256) void int4_pack_rows_kernel(const void* __restrict__ w,
                                                             int64_t n_rows, int64_t k, int64_t bs,
                                                             const float* __restrict__ ws,
                                                             uint8_t* __restrict__ out) {
    const int64_t kc = (k + 7) >> 3, nsb = k / bs;
    const int64_t total = (n_rows >> 1) * kc;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += stride) {
        const int64_t j = t / kc, c0 = (t - j * kc) << 3;
        for (int e = 0; e < 8 && c0 + e < k; ++e) {
            const int64_t col = c0 + e;
            uint32_t nib[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int64_t row = 2 * j + h;
                float q = load_elem<DT>(w, row * k + col) / ws[row * nsb + col / bs];
                if constexpr (NARROW) q = round_via<DT>(q);
                q = __builtin_rintf(q);
                q = q < -8.0f ? -8.0f : q;
                q = q > 7.0f ? 7.0f : q;
                nib[h] = (q == q) ? ((uint32_t)(int)q & 0xFu) : 0u;
            }
            out[j * k + col] = (uint8_t)(nib[0] | (nib[1] << 4));
        }
    }
}

// ------------------------------------------------------------------------------ INT4 fast paths
// Block sizes of 8 << k elements (k <= 6) on 16-byte aligned tensors: a lane owns a chunk, the
// lanes of a block combine their abs-max with in-wave shuffles.
// clamp(rne(v), -8, 7) as an integer in three operations: v_med3_f32 clamps (and returns the
// smallest operand, -8, for a NaN, which is the "NaN packs as code 0" rule of the kernels above),
// adding 1.5 * 2^23 rounds to nearest even and leaves the integer in the low mantissa bits.
__device__ __forceinline__ int int4_rne(float v) {
    const float t = __builtin_amdgcn_fmed3f(v, -8.0f, 7.0f);
    return (int)f2u(t + 12582912.0f) - 0x4B400000;
}

// chunks per lane (16-byte loads in flight for the quantizer, 4-byte loads for the dequantizer);
// measured on 34 MB - 537 MB tensors: 4 beats 8 for the quantizer by 5 - 10 %, the dequantizer wants 8
constexpr int kInt4QuantRounds = 4;
constexpr int kInt4DequantRounds = 8;

template <int DT>
__global__ __launch_bounds__(256) void int4_block_quantize_tile_kernel(
    const void* __restrict__ x, int64_t chunks, int lanes_per_block, int shift,
    void* __restrict__ scales, int scales_given, uint32_t* __restrict__ packed) {
    constexpr int U = kInt4QuantRounds;
    const int64_t c0 = (int64_t)blockIdx.x * (256 * U) + threadIdx.x;
    RawChunk<DT> raw[U];
    // The loads sit in per-round bounds checks, so the compiler waits for all of them at once
    // and the rounds then compute and store back to back.  The form used elsewhere (clamped
    // straight-line loads, a wait per round) was 4 % slower for this kernel in alternating
    // runs on 117 MB (24.7 against 23.7 us): it stores a fifth of what it loads and no round
    // loads behind a store either way.
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int64_t c = c0 + u * 256;
        zero_raw<DT>(raw[u]);
        if (c < chunks) load_raw<DT>(x, c << 3, raw[u]);
    }
    float v[U][8];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int64_t c = c0 + u * 256;
        unpack_raw<DT>(raw[u], v[u]);
        uint32_t m = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t t = f2u(v[u][j]) & 0x7FFFFFFFu;
            m = t > m ? t : m;
        }
        // chunks is a multiple of lanes_per_block, so the lanes of a block are all in or all out
        m = group_max_u32(m, shift);
        if (c >= chunks) continue;
        float scale = round_via<DT>(round_via<DT>(1.0f / u2f(m)) * 7.0f);
        if (scales_given) scale = load_elem<DT>(scales, c >> shift);
        else if ((threadIdx.x & (lanes_per_block - 1)) == 0) store_elem<DT>(scales, c >> shift, scale);
        // byte = (hi + 8) << 4 | (lo + 8) = 16 * hi + lo + 0x88; the +8s of the four bytes are
        // added once to the assembled word (the borrows of negative bytes cancel exactly)
        int w = 0;
#pragma unroll
        for (int j = 0; j < 8; j += 2) {
            const int hi = int4_rne(round_via<DT>(v[u][j] * scale));
            const int lo = int4_rne(round_via<DT>(v[u][j + 1] * scale));
            w += (hi * 16 + lo) << (4 * j);
        }
        __builtin_nontemporal_store((uint32_t)w + 0x88888888u, packed + c);
    }
}

template <int DT>
__global__ __launch_bounds__(256) void int4_block_dequantize_tile_kernel(
    const uint32_t* __restrict__ packed, int64_t chunks, int shift,
    const void* __restrict__ scales, void* __restrict__ y) {
    constexpr int U = kInt4DequantRounds;
    const int64_t c0 = (int64_t)blockIdx.x * (256 * U) + threadIdx.x;
    uint32_t w[U];
    float sc[U];
    // Codes and scales of all rounds are loaded in straight-line code (a lane past the end
    // re-reads the last chunk) and only the stores are conditional: loads inside per-round
    // branches make the compiler wait for everything outstanding, the previous round's store
    // included, at every join.
#pragma unroll
    for (int u = 0; u < U; ++u) {
        int64_t c = c0 + u * 256;
        c = c < chunks ? c : chunks - 1;
        w[u] = __builtin_nontemporal_load(packed + c);
        sc[u] = load_elem<DT>(scales, c >> shift);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int64_t c = c0 + u * 256;
        const float s = sc[u];
        const float r = 1.0f / s;
        const bool fast = mid_range(s);
        float v[8];   // codes + 8
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v[2 * j] = (float)((w[u] >> (8 * j + 4)) & 0xFu);
            v[2 * j + 1] = (float)((w[u] >> (8 * j)) & 0xFu);
        }
        if (fast && DT == MO_BF16) {
            // a code has 4 significant bits and a bf16 scale 8: the exact quotient stays at
            // least 2^-17 of its value away from every rounding boundary of bf16 (it cannot
            // lie on one: the boundary's odd 9-bit numerator times the scale has more bits than
            // a code), so code times the reciprocal, good to 2^-22, rounds to the same bf16
            // value as the correctly rounded fp32 quotient.  (n - 8) * ra in one FMA: 8 * ra is
            // exact, so the sum is rounded once, and n = 8 gives +0 as 0 / s does.
            const float ra = __builtin_amdgcn_rcpf(s), off = -8.0f * ra;
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = __builtin_fmaf(v[j], ra, off);
        } else if (fast) {
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = exact_quotient(v[j] - 8.0f, s, r);  // 0 / s = +0, s > 0
        } else {
            keep_branch();
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = (v[j] - 8.0f) / s;
        }
        if (c < chunks) store_chunk<DT>(y, c << 3, v);
    }
}

// Row-pair pack with k % 8 == 0 and block_size % 8 == 0: a lane loads the same chunk of
// columns from rows 2j and 2j + 1 and stores 8 bytes.
constexpr int kInt4PackRounds = 2;   // items per lane (two 16-byte loads in flight each); 4 is 10 % slower at 117 MB
template <int DT, bool NARROW>
__global__ __launch_bounds__(256) void int4_pack_rows_tile_kernel(
    const void* __restrict__ w, int64_t pairs, int64_t kc, int64_t chunks_per_scale,
    const float* __restrict__ ws, u32x2* __restrict__ out) {
    constexpr int R = kInt4PackRounds;
    const int64_t total = pairs * kc;
    const int64_t t0 = (int64_t)blockIdx.x * (256 * R) + threadIdx.x;
    const int64_t nsb = kc / chunks_per_scale;
    RawChunk<DT> ra_[R], rb_[R];
    float sa[R], sb[R];
    // (row pair, chunk) of the lane's first item by one division, of the others by stepping
    int64_t j0, cc0;
    if (total <= 0xFFFFFFFFll) {
        j0 = (uint32_t)t0 / (uint32_t)kc;
        cc0 = (uint32_t)t0 - (uint32_t)j0 * (uint32_t)kc;
    } else {
        j0 = t0 / kc;
        cc0 = t0 - j0 * kc;
    }
    const int64_t step_j = 256 / kc, step_c = 256 - step_j * kc;   // 256 = step_j * kc + step_c
    // all loads in straight-line code (an item past the end re-reads the last one and stores
    // nothing), so that no round waits behind the store of the one before
#pragma unroll
    for (int u = 0; u < R; ++u) {
        const int64_t t = t0 + u * 256;
        int64_t j = j0 + u * step_j, c = cc0 + u * step_c;
        // c < kc + u * step_c < (u + 1) * kc: at most u wraps
#pragma unroll
        for (int i = 0; i < u; ++i)
            if (c >= kc) { c -= kc; ++j; }
        if (t >= total) { j = pairs - 1; c = kc - 1; }
        load_raw<DT>(w, ((2 * j) * kc + c) << 3, ra_[u]);
        load_raw<DT>(w, ((2 * j + 1) * kc + c) << 3, rb_[u]);
        const int64_t sc = (uint32_t)c / (uint32_t)chunks_per_scale;  // both below 2^32
        sa[u] = ws[(2 * j) * nsb + sc];
        sb[u] = ws[(2 * j + 1) * nsb + sc];
    }
    float a[R][8], b[R][8];
#pragma unroll
    for (int u = 0; u < R; ++u) {
        const int64_t t = t0 + u * 256;
        unpack_raw<DT>(ra_[u], a[u]);
        unpack_raw<DT>(rb_[u], b[u]);
        uint32_t m = 0;
        if constexpr (DT == MO_BF16) {
            // bit patterns of |x| order like the values: maxima of the 16-bit halves, two per
            // instruction; the fp32 pattern of a bf16 value is its pattern shifted up
            const u32x4 p = ra_[u].a, q = rb_[u].a;
            const uint32_t h = pk_max_u16(
                pk_max_u16(pk_max_u16(p.x & 0x7FFF7FFFu, p.y & 0x7FFF7FFFu), pk_max_u16(p.z & 0x7FFF7FFFu, p.w & 0x7FFF7FFFu)),
                pk_max_u16(pk_max_u16(q.x & 0x7FFF7FFFu, q.y & 0x7FFF7FFFu), pk_max_u16(q.z & 0x7FFF7FFFu, q.w & 0x7FFF7FFFu)));
            const uint32_t top = h >> 16, low = h & 0xFFFFu;
            m = (top > low ? top : low) << 16;
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint32_t ta = f2u(a[u][e]) & 0x7FFFFFFFu, tb = f2u(b[u][e]) & 0x7FFFFFFFu;
                m = ta > m ? ta : m;
                m = tb > m ? tb : m;
            }
        }
        const float ra = 1.0f / sa[u], rb = 1.0f / sb[u];
        const float big = u2f(m);
        // fast: both scales normal and mid-range, every element finite (a NaN or inf element
        // makes `big` NaN or inf and fails the comparisons) -- no quotient can be NaN there
        const bool fast = mid_range(sa[u]) && mid_range(sb[u]) && big * ra < 1.0e38f && big * rb < 1.0e38f;
        uint32_t lo = 0, hi = 0;
        if (fast) {
            // clamp, then add 2^23 + 8: the sum rounds to the nearest integer, ties to even (q and
            // q + 8 have the same parity), and its bit pattern is 0x4B000000 + (q + 8) with
            // q + 8 in 0 .. 15.  The patterns are shifted into place and summed as they are; what
            // the eight 0x4B000000 leave in the low 32 bits (only the shifts by 0 and 4 keep any
            // of it) is taken off once, and flipping the top bit of every nibble turns q + 8 into
            // the two's-complement nibble of q.
            constexpr uint32_t kLeft = 0x4B000000u + (0x4B000000u << 4);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float xa = exact_quotient(a[u][e], sa[u], ra), xb = exact_quotient(b[u][e], sb[u], rb);
                if constexpr (NARROW) {
                    xa = round_via<DT>(xa);
                    xb = round_via<DT>(xb);
                }
                const float qa = __builtin_amdgcn_fmed3f(xa, -8.0f, 7.0f);
                const float qb = __builtin_amdgcn_fmed3f(xb, -8.0f, 7.0f);
                const uint32_t ba = f2u(qa + 8388616.0f), bb = f2u(qb + 8388616.0f);
                if (e < 4) lo += (ba << (8 * e)) + (bb << (8 * e + 4));
                else hi += (ba << (8 * (e - 4))) + (bb << (8 * (e - 4) + 4));
            }
            lo = (lo - kLeft) ^ 0x88888888u;
            hi = (hi - kLeft) ^ 0x88888888u;
        } else {
            keep_branch();
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float qa = a[u][e] / sa[u], qb = b[u][e] / sb[u];
                if constexpr (NARROW) {
                    qa = round_via<DT>(qa);
                    qb = round_via<DT>(qb);
                }
                // a NaN quotient packs as 0 here (what the float -> int8 cast of the CPU path yields)
                const uint32_t na = qa == qa ? (uint32_t)int4_rne(qa) & 0xFu : 0u;
                const uint32_t nb = qb == qb ? (uint32_t)int4_rne(qb) & 0xFu : 0u;
                const uint32_t byte = na | (nb << 4);
                if (e < 4) lo |= byte << (8 * e); else hi |= byte << (8 * (e - 4));
            }
        }
        const u32x2 o = {lo, hi};
        if (t < total) __builtin_nontemporal_store(o, out + t);
    }
}

static inline unsigned blocks_for(int64_t items) {
    int64_t b = (items + 255) / 256;
    if (b < 1) b = 1;
    if (b > 65536) b = 65536;
    return (unsigned)b;
}

}  // namespace mo

#define DISPATCH_DT(dtype, CALL)        \
    switch (dtype) {                    \
        case MO_F32: CALL(MO_F32); break; \
        case MO_F16: CALL(MO_F16); break; \
        case MO_BF16: CALL(MO_BF16); break; \
        default: return MO_ERR_DTYPE;   \
    }

extern "C" int mo_real_quantize(const void* x, int64_t outer, int64_t axis, int64_t inner, int dtype,
                                const void* scale, int scale_dtype, int via_dtype, int format,
                                uint8_t* out, void* stream) {
    if (outer < 0 || axis < 0 || inner < 0) return MO_ERR_ARG;
    if (format != MO_FMT_E4M3 && format != MO_FMT_INT8) return MO_ERR_UNSUPPORTED;
    if (scale_dtype < MO_F32 || scale_dtype > MO_BF16 || via_dtype < MO_F32 || via_dtype > MO_BF16)
        return MO_ERR_DTYPE;
    const int64_t n = outer * axis * inner;
    if (n == 0) return MO_OK;
    if (!x || !scale || !out) return MO_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    const bool tiled = (n % 8 == 0) && (axis == 1 || inner % 8 == 0) &&
                       (((uintptr_t)x & 15u) == 0) && (((uintptr_t)out & 7u) == 0) &&
                       (n / 8 + mo::kRealTileChunks - 1) / mo::kRealTileChunks <= 0x7FFFFFFF;
    if (tiled) {
        const int64_t chunks = n / 8, ic = axis == 1 ? 1 : inner / 8;
        const unsigned gt = (unsigned)((chunks + mo::kRealTileChunks - 1) / mo::kRealTileChunks);
        // rows of at least 2048 elements: one row per workgroup, scale math wavefront-uniform
        const int64_t tpr = (ic + mo::kRealTileChunks - 1) / mo::kRealTileChunks;
        const int64_t row_tiles = outer * axis * tpr;
        const bool by_row = axis > 1 && ic >= 256 && row_tiles <= 0x7FFFFFFF;
        // (flat tiles with one scale per round, which the dequantizer takes for rows that are a
        // multiple of 2048 elements, were 5 % slower here than one row per workgroup: 30.3
        // against 28.7 us per 117 MB, four reciprocals per lane instead of one)
#define TILE4(DT, VIA, FMT)                                                                       \
    if (axis == 1)                                                                                \
        mo::real_quantize_tile_kernel<DT, VIA, FMT, mo::kScalePerTensor><<<gt, 256, mo::ballast_bytes("real_quantize_tile_kernel", 0), s>>>(      \
            x, chunks, axis, ic, 1, scale, scale_dtype, (mo::u32x2*)out);                         \
    else if (by_row)                                                                              \
        mo::real_quantize_tile_kernel<DT, VIA, FMT, mo::kScalePerRowTile>                         \
            <<<(unsigned)row_tiles, 256, mo::ballast_bytes("real_quantize_tile_kernel", 0), s>>>(x, chunks, axis, ic, tpr, scale, scale_dtype,    \
                                                 (mo::u32x2*)out);                                \
    else                                                                                          \
        mo::real_quantize_tile_kernel<DT, VIA, FMT, mo::kScalePerChunk><<<gt, 256, mo::ballast_bytes("real_quantize_tile_kernel", 0), s>>>(       \
            x, chunks, axis, ic, 1, scale, scale_dtype, (mo::u32x2*)out)
#define TILE3(DT, VIA) \
    if (format == MO_FMT_E4M3) { TILE4(DT, VIA, 0); } else { TILE4(DT, VIA, 1); }
#define CALL(DT)                                           \
    if (via_dtype == MO_F32) { TILE3(DT, MO_F32); }        \
    else if (via_dtype == MO_F16) { TILE3(DT, MO_F16); }   \
    else { TILE3(DT, MO_BF16); }
        DISPATCH_DT(dtype, CALL)
#undef CALL
#undef TILE3
#undef TILE4
        return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
    }
    const unsigned g = mo::blocks_for((n + 7) / 8);
#define CALL3(DT, VIA)                                                                             \
    if (format == MO_FMT_E4M3)                                                                     \
        mo::real_quantize_kernel<DT, VIA, 0><<<g, 256, 0, s>>>(x, n, axis, inner, scale, scale_dtype, out); \
    else                                                                                           \
        mo::real_quantize_kernel<DT, VIA, 1><<<g, 256, 0, s>>>(x, n, axis, inner, scale, scale_dtype, out)
#define CALL(DT)                                            \
    if (via_dtype == MO_F32) { CALL3(DT, MO_F32); }         \
    else if (via_dtype == MO_F16) { CALL3(DT, MO_F16); }    \
    else { CALL3(DT, MO_BF16); }
    DISPATCH_DT(dtype, CALL)
#undef CALL
#undef CALL3
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_real_dequantize(const uint8_t* q, int64_t outer, int64_t axis, int64_t inner,
                                  int format, const void* scale, int scale_dtype, void* y,
                                  int dtype, void* stream) {
    if (outer < 0 || axis < 0 || inner < 0) return MO_ERR_ARG;
    if (format != MO_FMT_E4M3 && format != MO_FMT_INT8) return MO_ERR_UNSUPPORTED;
    if (scale_dtype < MO_F32 || scale_dtype > MO_BF16) return MO_ERR_DTYPE;
    const int64_t n = outer * axis * inner;
    if (n == 0) return MO_OK;
    if (!q || !scale || !y) return MO_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    const bool tiled = (n % 8 == 0) && (axis == 1 || inner % 8 == 0) &&
                       (((uintptr_t)y & 15u) == 0) && (((uintptr_t)q & 7u) == 0) &&
                       (n / 8 + mo::kRealTileChunks - 1) / mo::kRealTileChunks <= 0x7FFFFFFF;
    if (tiled) {
        const int64_t chunks = n / 8, ic = axis == 1 ? 1 : inner / 8;
        const unsigned gt = (unsigned)((chunks + mo::kRealTileChunks - 1) / mo::kRealTileChunks);
        const int64_t tpr = (ic + mo::kRealTileChunks - 1) / mo::kRealTileChunks;
        const int64_t row_tiles = outer * axis * tpr;
        const bool by_row = axis > 1 && ic >= 256 && row_tiles <= 0x7FFFFFFF;
        const bool by_round = axis > 1 && ic % 256 == 0;
#define TILE3(DT, FMT)                                                                            \
    if (axis == 1)                                                                                \
        mo::real_dequantize_tile_kernel<DT, FMT, mo::kScalePerTensor><<<gt, 256, mo::ballast_bytes("real_dequantize_tile_kernel", 36), s>>>(         \
            (const mo::u32x2*)q, chunks, axis, ic, 1, scale, scale_dtype, y);                     \
    else if (by_round)                                                                            \
        mo::real_dequantize_tile_kernel<DT, FMT, mo::kScalePerRound><<<gt, 256, mo::ballast_bytes("real_dequantize_tile_kernel", 36), s>>>(          \
            (const mo::u32x2*)q, chunks, axis, ic, 1, scale, scale_dtype, y);                     \
    else if (by_row)                                                                              \
        mo::real_dequantize_tile_kernel<DT, FMT, mo::kScalePerRowTile>                            \
            <<<(unsigned)row_tiles, 256, mo::ballast_bytes("real_dequantize_tile_kernel", 36), s>>>((const mo::u32x2*)q, chunks, axis, ic, tpr,      \
                                                 scale, scale_dtype, y);                          \
    else                                                                                          \
        mo::real_dequantize_tile_kernel<DT, FMT, mo::kScalePerChunk><<<gt, 256, mo::ballast_bytes("real_dequantize_tile_kernel", 36), s>>>(          \
            (const mo::u32x2*)q, chunks, axis, ic, 1, scale, scale_dtype, y)
#define CALL(DT) \
    if (format == MO_FMT_E4M3) { TILE3(DT, 0); } else { TILE3(DT, 1); }
        DISPATCH_DT(dtype, CALL)
#undef CALL
#undef TILE3
        return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
    }
    const unsigned g = mo::blocks_for(n);
#define CALL(DT)                                                                                      \
    if (format == MO_FMT_E4M3)                                                                        \
        mo::real_dequantize_kernel<DT, 0><<<g, 256, 0, s>>>(q, n, axis, inner, scale, scale_dtype, y); \
    else                                                                                              \
        mo::real_dequantize_kernel<DT, 1><<<g, 256, 0, s>>>(q, n, axis, inner, scale, scale_dtype, y)
    DISPATCH_DT(dtype, CALL)
#undef CALL
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

// Storage casts with one scale per two-dimensional block (block sizes on the last two dims).
static int check_real_blocks2d(const void* a, const void* b, const void* scale, int64_t rows, int64_t cols,
                               int64_t block_rows, int64_t block_cols, int format, int scale_dtype) {
    if (rows < 0 || cols < 0 || block_rows <= 0 || block_cols <= 0) return MO_ERR_ARG;
    if (format != MO_FMT_E4M3 && format != MO_FMT_INT8) return MO_ERR_UNSUPPORTED;
    if (scale_dtype < MO_F32 || scale_dtype > MO_BF16) return MO_ERR_DTYPE;
    if (rows == 0 || cols == 0) return MO_OK;
    if (!a || !b || !scale) return MO_ERR_ARG;
    if (rows % block_rows || cols % block_cols || block_cols % 8 ||
        (rows * (cols / 8) + mo::kRealTileChunks - 1) / mo::kRealTileChunks > 0x7FFFFFFF)
        return MO_ERR_UNSUPPORTED;
    return MO_OK;
}

extern "C" int mo_real_quantize_blocks2d(const void* x, int64_t rows, int64_t cols, int64_t block_rows,
                                         int64_t block_cols, int dtype, const void* scale,
                                         int scale_dtype, int via_dtype, int format, uint8_t* out,
                                         void* stream) {
    int rc = check_real_blocks2d(x, out, scale, rows, cols, block_rows, block_cols, format, scale_dtype);
    if (rc != MO_OK || rows == 0 || cols == 0) return rc;
    if (via_dtype < MO_F32 || via_dtype > MO_BF16) return MO_ERR_DTYPE;
    if (((uintptr_t)x & 15u) || ((uintptr_t)out & 7u)) return MO_ERR_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
    const int64_t chunks = rows * (cols / 8);
    const unsigned gt = (unsigned)((chunks + mo::kRealTileChunks - 1) / mo::kRealTileChunks);
#define TILE4(DT, VIA, FMT)                                                                        \
    mo::real_quantize_tile_kernel<DT, VIA, FMT, mo::kScalePerBlock2d><<<gt, 256, 0, s>>>(          \
        x, chunks, block_rows, cols / 8, block_cols / 8, scale, scale_dtype, (mo::u32x2*)out)
#define CALL3(DT, VIA) \
    if (format == MO_FMT_E4M3) { TILE4(DT, VIA, 0); } else { TILE4(DT, VIA, 1); }
#define CALL(DT)                                            \
    if (via_dtype == MO_F32) { CALL3(DT, MO_F32); }         \
    else if (via_dtype == MO_F16) { CALL3(DT, MO_F16); }    \
    else { CALL3(DT, MO_BF16); }
    DISPATCH_DT(dtype, CALL)
#undef CALL
#undef CALL3
#undef TILE4
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_real_dequantize_blocks2d(const uint8_t* q, int64_t rows, int64_t cols,
                                           int64_t block_rows, int64_t block_cols, int format,
                                           const void* scale, int scale_dtype, void* y, int dtype,
                                           void* stream) {
    int rc = check_real_blocks2d(q, y, scale, rows, cols, block_rows, block_cols, format, scale_dtype);
    if (rc != MO_OK || rows == 0 || cols == 0) return rc;
    if (((uintptr_t)y & 15u) || ((uintptr_t)q & 7u)) return MO_ERR_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
    const int64_t chunks = rows * (cols / 8);
    const unsigned gt = (unsigned)((chunks + mo::kRealTileChunks - 1) / mo::kRealTileChunks);
#define TILE3(DT, FMT)                                                                             \
    mo::real_dequantize_tile_kernel<DT, FMT, mo::kScalePerBlock2d><<<gt, 256, 0, s>>>(             \
        (const mo::u32x2*)q, chunks, block_rows, cols / 8, block_cols / 8, scale, scale_dtype, y)
#define CALL(DT) \
    if (format == MO_FMT_E4M3) { TILE3(DT, 0); } else { TILE3(DT, 1); }
    DISPATCH_DT(dtype, CALL)
#undef CALL
#undef TILE3
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_int4_block_quantize(const void* x, int64_t n, int64_t block_size, int dtype,
                                      void* scales, int scales_given, uint8_t* packed,
                                      void* stream) {
    if (n < 0 || block_size <= 0 || (block_size & 1)) return MO_ERR_ARG;
    if (n == 0) return MO_OK;
    if (!x || !scales || !packed) return MO_ERR_ARG;
    const int64_t nblocks = (n + block_size - 1) / block_size;
    hipStream_t s = (hipStream_t)stream;
    int shift = -1;  // block_size == 8 << shift
    for (int k = 0; k <= 6; ++k)
        if (block_size == (8ll << k)) shift = k;
    const int64_t per_tile = 256 * mo::kInt4QuantRounds;
    const int64_t tiles = (n / 8 + per_tile - 1) / per_tile;
    if (shift >= 0 && n % block_size == 0 && (((uintptr_t)x & 15u) == 0) &&
        (((uintptr_t)packed & 3u) == 0) && tiles <= 0x7FFFFFFF) {
#define CALL(DT)                                                                          \
    mo::int4_block_quantize_tile_kernel<DT><<<(unsigned)tiles, 256, mo::ballast_bytes("int4_block_quantize_tile_kernel", 0), s>>>(              \
        x, n / 8, 1 << shift, shift, scales, scales_given, (uint32_t*)packed)
        DISPATCH_DT(dtype, CALL)
#undef CALL
        return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
    }
    const unsigned g = mo::blocks_for(nblocks);
#define CALL(DT) mo::int4_block_quantize_kernel<DT><<<g, 256, 0, s>>>(x, n, block_size, nblocks, scales, scales_given, packed)
    DISPATCH_DT(dtype, CALL)
#undef CALL
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_int4_block_dequantize(const uint8_t* packed, int64_t nbytes, int64_t block_size,
                                        const void* scales, void* y, int dtype, void* stream) {
    if (nbytes < 0 || block_size <= 0 || (block_size & 1)) return MO_ERR_ARG;
    if (nbytes == 0) return MO_OK;
    if (!packed || !scales || !y) return MO_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    int shift = -1;
    for (int k = 0; k <= 40; ++k)
        if (block_size == (8ll << k)) shift = k;
    const int64_t per_tile = 256 * mo::kInt4DequantRounds;
    const int64_t tiles = (nbytes / 4 + per_tile - 1) / per_tile;
    if (shift >= 0 && nbytes % 4 == 0 && (((uintptr_t)y & 15u) == 0) &&
        (((uintptr_t)packed & 3u) == 0) && tiles <= 0x7FFFFFFF) {
#define CALL(DT)                                                                          \
    mo::int4_block_dequantize_tile_kernel<DT><<<(unsigned)tiles, 256, mo::ballast_bytes("int4_block_dequantize_tile_kernel", 0), s>>>(            \
        (const uint32_t*)packed, nbytes / 4, shift, scales, y)
        DISPATCH_DT(dtype, CALL)
#undef CALL
        return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
    }
    const unsigned g = mo::blocks_for(nbytes);
#define CALL(DT) mo::int4_block_dequantize_kernel<DT><<<g, 256, 0, s>>>(packed, nbytes, block_size, scales, y)
    DISPATCH_DT(dtype, CALL)
#undef CALL
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_int4_pack_rows(const void* w, int64_t batch, int64_t n_rows, int64_t k,
                                 int64_t block_size, int dtype, const float* ws, uint8_t* out,
                                 void* stream) {
    return mo_int4_pack_rows_via(w, batch, n_rows, k, block_size, dtype, ws, MO_F32, out, stream);
}

extern "C" int mo_int4_pack_rows_via(const void* w, int64_t batch, int64_t n_rows, int64_t k,
                                     int64_t block_size, int dtype, const float* ws, int via_dtype,
                                     uint8_t* out, void* stream) {
    if (batch < 0 || n_rows < 0 || k < 0 || block_size <= 0) return MO_ERR_ARG;
    if ((n_rows & 1) || (k % block_size)) return MO_ERR_ARG;
    if (dtype < MO_F32 || dtype > MO_BF16 || via_dtype < MO_F32 || via_dtype > MO_BF16) return MO_ERR_DTYPE;
    // the quotient of a tensor division is fp32 or, when both operands share a 16-bit type, that type
    if (via_dtype != MO_F32 && via_dtype != dtype) return MO_ERR_UNSUPPORTED;
    const bool narrow = via_dtype != MO_F32;
    if (batch == 0 || n_rows == 0 || k == 0) return MO_OK;
    if (!w || !ws || !out) return MO_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    // a stack of `batch` matrices is one matrix of batch * n_rows rows (n_rows is even)
    const int64_t rows = batch * n_rows;
    if (k % 8 == 0 && block_size % 8 == 0 && k < (1ll << 34) && (((uintptr_t)w & 15u) == 0) &&
        (((uintptr_t)out & 7u) == 0)) {
        const int64_t per_tile = 256 * mo::kInt4PackRounds;
        const int64_t items = (rows >> 1) * (k / 8), tiles = (items + per_tile - 1) / per_tile;
        if (tiles <= 0x7FFFFFFF) {
#define CALL(DT)                                                                      \
    if (narrow && DT != MO_F32)                                                       \
        mo::int4_pack_rows_tile_kernel<DT, DT != MO_F32><<<(unsigned)tiles, 256, mo::ballast_bytes("int4_pack_rows_tile_kernel", 0), s>>>( \
            w, rows >> 1, k / 8, block_size / 8, ws, (mo::u32x2*)out);                \
    else                                                                              \
        mo::int4_pack_rows_tile_kernel<DT, false><<<(unsigned)tiles, 256, mo::ballast_bytes("int4_pack_rows_tile_kernel", 0), s>>>(        \
            w, rows >> 1, k / 8, block_size / 8, ws, (mo::u32x2*)out)
            DISPATCH_DT(dtype, CALL)
#undef CALL
            return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
        }
    }
    const unsigned g = mo::blocks_for((rows >> 1) * ((k + 7) >> 3));
#define CALL(DT)                                                                                      \
    if (narrow && DT != MO_F32)                                                                       \
        mo::int4_pack_rows_kernel<DT, DT != MO_F32><<<g, 256, 0, s>>>(w, rows, k, block_size, ws, out); \
    else                                                                                              \
        mo::int4_pack_rows_kernel<DT, false><<<g, 256, 0, s>>>(w, rows, k, block_size, ws, out)
    DISPATCH_DT(dtype, CALL)
#undef CALL
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}
