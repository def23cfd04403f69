// NF4 (4-bit table codes, block abs-max scales) quantise+pack and dequantise for gfx950.
// HBM-bound elementwise work; numerics are those of the reference's CPU torch path.
//
// Quantise, per block of `bs` flat elements (zero padded to a whole block):
//   scale = max |x|                                  (stored in the input dtype)
//   v     = T(f32(x) / f32(scale))                   (T = input dtype)
//   code  = first index of the minimum of T(|v - table[i]|), i = 0..15; index 0 when v is NaN
//   byte  = code[2i] << 4 | code[2i + 1]
// The table is the bf16 rounding of the sixteen NF4 constants.  Its entries are at least 0.079
// apart and |v| <= 1, so only the two entries that bracket v can share the minimum, and
// whether the upper one wins is monotone in v: for each pair of neighbours there is one
// threshold t[j] with "upper wins <=> v > t[j]", and code = number of thresholds below v.
// The thresholds depend on T (the differences are rounded to T) and are found on the host by
// bisection on exactly the comparison above; the kernel does a four-step binary search.
#include "common.h"

namespace mo {

struct Nf4Thresholds { float t[15]; };

// bf16(-1, -0.6962, -0.5251, -0.3949, -0.2844, -0.1848, -0.0911, 0, 0.0796, 0.1609, 0.2461,
//      0.3379, 0.4407, 0.5626, 0.7230, 1)
#define MO_NF4_TABLE                                                                           \
    {-1.0f, -0.6953125f, -0.5234375f, -0.39453125f, -0.28515625f, -0.1845703125f,              \
     -0.09130859375f, 0.0f, 0.07958984375f, 0.1611328125f, 0.24609375f, 0.337890625f,          \
     0.44140625f, 0.5625f, 0.72265625f, 1.0f}

__device__ __constant__ float kNf4Table[16] = MO_NF4_TABLE;

template <int VIA>
__device__ __forceinline__ float nf4_round_via(float v) {
    if constexpr (VIA == MO_BF16) return bf16_bits_to_f32(f32_to_bf16_bits(v));
    else if constexpr (VIA == MO_F16) return f16_bits_to_f32(f32_to_f16_bits(v));
    else return v;
}

// The thresholds as fifteen register values.  They are handed on as separate scalars, never
// through a pointer or reference: selecting between two of them must stay a select of values
// (given an address the compiler turns it into a load at a selected address, and the copy of
// the argument struct then lives in scratch memory).
struct Nf4Regs {
    float t0, t1, t2, t3, t4, t5, t6, t7, t8, t9, t10, t11, t12, t13, t14;
};

__device__ __forceinline__ Nf4Regs nf4_regs(const Nf4Thresholds& th) {
    float f[15];
#pragma unroll
    for (int j = 0; j < 15; ++j) {
        f[j] = th.t[j];
        asm volatile("" : "+v"(f[j]));
    }
    return {f[0], f[1], f[2], f[3], f[4], f[5], f[6], f[7], f[8], f[9], f[10], f[11], f[12],
            f[13], f[14]};
}

// number of thresholds below v (NaN: none)
__device__ __forceinline__ uint32_t nf4_code_scalars(float v, float t0, float t1, float t2,
                                                     float t3, float t4, float t5, float t6,
                                                     float t7, float t8, float t9, float t10,
                                                     float t11, float t12, float t13, float t14) {
    const bool b3 = v > t7;
    const bool b2 = v > (b3 ? t11 : t3);
    const float m1 = b3 ? (b2 ? t13 : t9) : (b2 ? t5 : t1);
    const bool b1 = v > m1;
    const float m0 = b3 ? (b2 ? (b1 ? t14 : t12) : (b1 ? t10 : t8))
                        : (b2 ? (b1 ? t6 : t4) : (b1 ? t2 : t0));
    const bool b0 = v > m0;
    return (b3 ? 8u : 0u) | (b2 ? 4u : 0u) | (b1 ? 2u : 0u) | (b0 ? 1u : 0u);
}

#define nf4_code(v, R)                                                                         \
    nf4_code_scalars(v, (R).t0, (R).t1, (R).t2, (R).t3, (R).t4, (R).t5, (R).t6, (R).t7, (R).t8, \
                     (R).t9, (R).t10, (R).t11, (R).t12, (R).t13, (R).t14)

template <int DT>
__device__ __forceinline__ uint32_t nf4_codes8(const float (&v)[8], float amax, Nf4Regs th) {
    const float r = 1.0f / amax;
    const bool fast = mid_range(amax);  // finite, non-zero, no under- or overflow in the FMAs
    uint32_t w = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float q = fast ? exact_quotient(v[j], amax, r) : v[j] / amax;
        const uint32_t c = nf4_code(nf4_round_via<DT>(q), th);
        w |= c << (4 * (j ^ 1));  // even element of a pair in the high nibble of its byte
    }
    return w;
}

// One lane per block: any even block size, zero padding of the last block.
template <int DT>
__global__ __launch_bounds__(256) void nf4_quantize_kernel(const void* __restrict__ x, int64_t n,
                                                           int64_t bs, int64_t nblocks,
                                                           Nf4Thresholds thresholds,
                                                           void* __restrict__ scales,
                                                           uint8_t* __restrict__ packed) {
    const Nf4Regs th = nf4_regs(thresholds);
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
        store_elem<DT>(scales, b, amax);
        for (int64_t j = 0; j < bs; j += 2) {
            uint32_t c[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const float v = i0 + j + h < n ? load_elem<DT>(x, i0 + j + h) : 0.0f;
                c[h] = nf4_code(nf4_round_via<DT>(v / amax), th);
            }
            packed[(i0 + j) >> 1] = (uint8_t)((c[0] << 4) | c[1]);
        }
    }
}

// Tile form: block size 8 << shift with no padding; a lane owns chunks of 8 elements, the
// lanes of a block share their maximum through DPP moves, loads are issued before any math.
constexpr int kNf4TileChunks = 1024;

template <int DT>
__global__ __launch_bounds__(256) void nf4_quantize_tile_kernel(
    const void* __restrict__ x, int64_t chunks, int lanes_per_block, int shift,
    Nf4Thresholds thresholds, void* __restrict__ scales, uint32_t* __restrict__ packed) {
    const Nf4Regs th = nf4_regs(thresholds);
    const int64_t c0 = (int64_t)blockIdx.x * kNf4TileChunks + threadIdx.x;
    RawChunk<DT> raw[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int64_t c = c0 + u * 256;
        zero_raw<DT>(raw[u]);
        if (c < chunks) load_raw<DT>(x, c << 3, raw[u]);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int64_t c = c0 + u * 256;
        float v[8];
        unpack_raw<DT>(raw[u], v);
        uint32_t m = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t t = f2u(v[j]) & 0x7FFFFFFFu;
            m = t > m ? t : m;
        }
        // chunks is a multiple of lanes_per_block, so the lanes of a block are all in or all out
        m = group_max_u32(m, shift);
        if (c >= chunks) continue;
        const float amax = u2f(m);
        if ((threadIdx.x & (lanes_per_block - 1)) == 0) store_elem<DT>(scales, c >> shift, amax);
        __builtin_nontemporal_store(nf4_codes8<DT>(v, amax, th), packed + c);
    }
}

// Table form for the 16-bit dtypes and large inputs.  The scaled value v is itself a 16-bit value
// with |v| <= 1, so its code can be read from a table indexed by its bit pattern: 0x3F81
// magnitudes for bf16 (0 .. 1.0), 0x3C01 for fp16, times two signs -- under 32 KiB of one-byte
// codes.  A small kernel fills the table in device memory from the same thresholds (so the two
// forms agree by construction); a workgroup copies it to LDS once and then converts
// kNf4LutTiles tiles, which replaces the 19-instruction search per element by one LDS read.
// Chunks whose block abs-max is zero, tiny or not finite take the threshold search.
constexpr int kNf4LutBytes = 32768;
constexpr int kNf4LutTiles = 8;
template <int DT> struct Nf4Lut;
template <> struct Nf4Lut<MO_BF16> { static constexpr int half = 0x3F81, slot = 0; };
template <> struct Nf4Lut<MO_F16> { static constexpr int half = 0x3C01, slot = 1; };

__device__ __align__(16) uint8_t g_nf4_lut[2][kNf4LutBytes];

template <int DT>
__global__ __launch_bounds__(256) void nf4_build_lut_kernel(Nf4Thresholds thresholds) {
    const Nf4Regs th = nf4_regs(thresholds);
    constexpr int half = Nf4Lut<DT>::half;
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= kNf4LutBytes) return;
    uint32_t code = 0;
    if (e < 2 * half) {
        const uint32_t sign = e >= half ? 1u : 0u;
        const uint32_t bits = (uint32_t)(e - (int)sign * half) | (sign << 15);
        const float v = DT == MO_BF16 ? bf16_bits_to_f32(bits) : f16_bits_to_f32(bits);
        code = nf4_code(v, th);
    }
    g_nf4_lut[Nf4Lut<DT>::slot][e] = (uint8_t)code;
}

template <int DT>
__global__ __launch_bounds__(256) void nf4_quantize_lut_kernel(
    const void* __restrict__ x, int64_t chunks, int lanes_per_block, int shift,
    Nf4Thresholds thresholds, void* __restrict__ scales, uint32_t* __restrict__ packed) {
    __shared__ __align__(16) uint8_t lut[kNf4LutBytes];
    constexpr int half = Nf4Lut<DT>::half;
    {
        const u32x4* src = (const u32x4*)g_nf4_lut[Nf4Lut<DT>::slot];
        u32x4* dst = (u32x4*)lut;
#pragma unroll
        for (int i = 0; i < kNf4LutBytes / 16 / 256; ++i) dst[threadIdx.x + i * 256] = src[threadIdx.x + i * 256];
    }
    __syncthreads();
    const Nf4Regs th = nf4_regs(thresholds);
    for (int t = 0; t < kNf4LutTiles; ++t) {
        const int64_t c0 = ((int64_t)blockIdx.x * kNf4LutTiles + t) * kNf4TileChunks + threadIdx.x;
        if (c0 - threadIdx.x >= chunks) break;  // uniform: the whole tile is past the end
        RawChunk<DT> raw[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t c = c0 + u * 256;
            zero_raw<DT>(raw[u]);
            if (c < chunks) load_raw<DT>(x, c << 3, raw[u]);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t c = c0 + u * 256;
            float v[8];
            unpack_raw<DT>(raw[u], v);
            uint32_t m = 0;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t a = f2u(v[j]) & 0x7FFFFFFFu;
                m = a > m ? a : m;
            }
            m = group_max_u32(m, shift);
            if (c >= chunks) continue;
            const float amax = u2f(m);
            if ((threadIdx.x & (lanes_per_block - 1)) == 0) store_elem<DT>(scales, c >> shift, amax);
            uint32_t w = 0;
            if (mid_range(amax)) {
                const float r = 1.0f / amax;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float q = exact_quotient(v[j], amax, r);
                    const uint32_t bits = DT == MO_BF16 ? f32_to_bf16_bits(q) : f32_to_f16_bits(q);
                    const uint32_t entry = (bits & 0x7FFFu) + ((bits >> 15) & 1u) * (uint32_t)half;
                    w |= (uint32_t)lut[entry] << (4 * (j ^ 1));
                }
            } else {
                w = nf4_codes8<DT>(v, amax, th);
            }
            __builtin_nontemporal_store(w, packed + c);
        }
    }
}

// y[2i] = T(table[byte >> 4] * f32(scale[block])), y[2i + 1] = T(table[byte & 15] * ...)
template <int DT>
__global__ __launch_bounds__(256) void nf4_dequantize_kernel(const uint8_t* __restrict__ packed,
                                                             int64_t nbytes, int64_t bs,
                                                             const void* __restrict__ scales,
                                                             void* __restrict__ y) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nbytes; i += stride) {
        const uint32_t b = packed[i];
        const float s = load_elem<DT>(scales, (2 * i) / bs);
        store_elem<DT>(y, 2 * i, kNf4Table[b >> 4] * s);
        store_elem<DT>(y, 2 * i + 1, kNf4Table[b & 0xFu] * s);
    }
}

template <int DT>
__global__ __launch_bounds__(256) void nf4_dequantize_tile_kernel(
    const uint32_t* __restrict__ packed, int64_t chunks, int shift,
    const void* __restrict__ scales, void* __restrict__ y) {
    __shared__ float table[16];
    if (threadIdx.x < 16) table[threadIdx.x] = kNf4Table[threadIdx.x];
    __syncthreads();
    const int64_t c0 = (int64_t)blockIdx.x * kNf4TileChunks + threadIdx.x;
    uint32_t w[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int64_t c = c0 + u * 256;
        w[u] = c < chunks ? __builtin_nontemporal_load(packed + c) : 0u;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int64_t c = c0 + u * 256;
        if (c >= chunks) continue;
        const float s = load_elem<DT>(scales, c >> shift);
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = table[(w[u] >> (4 * (j ^ 1))) & 0xFu] * s;
        store_chunk<DT>(y, c << 3, v);
    }
}

// ------------------------------------------------------------------------------ host side
static float host_round(float f, int dtype) {
    if (dtype == MO_F32 || f != f) return f;
    uint32_t u;
    __builtin_memcpy(&u, &f, 4);
    if (dtype == MO_BF16) {
        u += 0x7FFFu + ((u >> 16) & 1u);
        u &= 0xFFFF0000u;
    } else {
        const float a = __builtin_fabsf(f);
        if (a < 6.103515625e-05f) {  // fp16 subnormal range: multiples of 2^-24
            return __builtin_rintf(f * 16777216.0f) * 5.9604644775390625e-08f;
        }
        u += 0xFFFu + ((u >> 13) & 1u);
        u &= 0xFFFFE000u;
        float g;
        __builtin_memcpy(&g, &u, 4);
        if (__builtin_fabsf(g) > 65504.0f) return f < 0 ? -__builtin_inff() : __builtin_inff();
        return g;
    }
    __builtin_memcpy(&f, &u, 4);
    return f;
}

// fp32 values in numeric order <-> integers in the same order
static int64_t ordered_key(float f) {
    uint32_t u;
    __builtin_memcpy(&u, &f, 4);
    return (u & 0x80000000u) ? -(int64_t)(u & 0x7FFFFFFFu) : (int64_t)u;
}

static float from_key(int64_t k) {
    const uint32_t u = k < 0 ? (0x80000000u | (uint32_t)(-k)) : (uint32_t)k;
    float f;
    __builtin_memcpy(&f, &u, 4);
    return f;
}

// t[j] = the largest fp32 p for which table[j] still wins against table[j + 1] at v = T(p)
static Nf4Thresholds nf4_thresholds(int dtype) {
    static const float table[16] = MO_NF4_TABLE;
    Nf4Thresholds th;
    for (int j = 0; j < 15; ++j) {
        auto upper_wins = [&](float p) {
            const float v = host_round(p, dtype);
            const float lo = host_round(__builtin_fabsf(v - table[j]), dtype);
            const float hi = host_round(__builtin_fabsf(v - table[j + 1]), dtype);
            return hi < lo;
        };
        int64_t a = ordered_key(table[j]), b = ordered_key(table[j + 1]);  // false at a, true at b
        while (b - a > 1) {
            const int64_t mid = a + (b - a) / 2;
            if (upper_wins(from_key(mid))) b = mid; else a = mid;
        }
        th.t[j] = from_key(a);
    }
    return th;
}

static inline unsigned nf4_blocks_for(int64_t items) {
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

extern "C" int mo_nf4_quantize(const void* x, int64_t n, int64_t block_size, int dtype,
                               void* scales, uint8_t* packed, void* stream) {
    if (n < 0 || block_size <= 0 || (block_size & 1)) return MO_ERR_ARG;
    if (dtype != MO_F32 && dtype != MO_F16 && dtype != MO_BF16) return MO_ERR_DTYPE;
    if (n == 0) return MO_OK;
    if (!x || !scales || !packed) return MO_ERR_ARG;
    const int64_t nblocks = (n + block_size - 1) / block_size;
    hipStream_t s = (hipStream_t)stream;
    const mo::Nf4Thresholds th = mo::nf4_thresholds(dtype);
    int shift = -1;  // block_size == 8 << shift
    for (int k = 0; k <= 6; ++k)
        if (block_size == (8ll << k)) shift = k;
    const int64_t tiles = (n / 8 + mo::kNf4TileChunks - 1) / mo::kNf4TileChunks;
    if (shift >= 0 && n % block_size == 0 && (((uintptr_t)x & 15u) == 0) &&
        (((uintptr_t)packed & 3u) == 0) && tiles <= 0x7FFFFFFF) {
        if (dtype != MO_F32 && tiles >= 64 * mo::kNf4LutTiles) {  // large 16-bit input: table form
            const unsigned g = (unsigned)((tiles + mo::kNf4LutTiles - 1) / mo::kNf4LutTiles);
            if (dtype == MO_BF16) {
                mo::nf4_build_lut_kernel<MO_BF16><<<mo::kNf4LutBytes / 256, 256, 0, s>>>(th);
                mo::nf4_quantize_lut_kernel<MO_BF16><<<g, 256, 0, s>>>(
                    x, n / 8, 1 << shift, shift, th, scales, (uint32_t*)packed);
            } else {
                mo::nf4_build_lut_kernel<MO_F16><<<mo::kNf4LutBytes / 256, 256, 0, s>>>(th);
                mo::nf4_quantize_lut_kernel<MO_F16><<<g, 256, 0, s>>>(
                    x, n / 8, 1 << shift, shift, th, scales, (uint32_t*)packed);
            }
            return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
        }
#define CALL(DT)                                                                    \
    mo::nf4_quantize_tile_kernel<DT><<<(unsigned)tiles, 256, 0, s>>>(               \
        x, n / 8, 1 << shift, shift, th, scales, (uint32_t*)packed)
        DISPATCH_DT(dtype, CALL)
#undef CALL
        return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
    }
    const unsigned g = mo::nf4_blocks_for(nblocks);
#define CALL(DT) mo::nf4_quantize_kernel<DT><<<g, 256, 0, s>>>(x, n, block_size, nblocks, th, scales, packed)
    DISPATCH_DT(dtype, CALL)
#undef CALL
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_nf4_dequantize(const uint8_t* packed, int64_t nbytes, int64_t block_size,
                                 const void* scales, void* y, int dtype, void* stream) {
    if (nbytes < 0 || block_size <= 0 || (block_size & 1)) return MO_ERR_ARG;
    if (dtype != MO_F32 && dtype != MO_F16 && dtype != MO_BF16) return MO_ERR_DTYPE;
    if (nbytes == 0) return MO_OK;
    if (!packed || !scales || !y) return MO_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    int shift = -1;
    for (int k = 0; k <= 40; ++k)
        if (block_size == (8ll << k)) shift = k;
    const int64_t tiles = (nbytes / 4 + mo::kNf4TileChunks - 1) / mo::kNf4TileChunks;
    if (shift >= 0 && nbytes % 4 == 0 && (((uintptr_t)y & 15u) == 0) &&
        (((uintptr_t)packed & 3u) == 0) && tiles <= 0x7FFFFFFF) {
#define CALL(DT)                                                                    \
    mo::nf4_dequantize_tile_kernel<DT><<<(unsigned)tiles, 256, 0, s>>>(             \
        (const uint32_t*)packed, nbytes / 4, shift, scales, y)
        DISPATCH_DT(dtype, CALL)
#undef CALL
        return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
    }
    const unsigned g = mo::nf4_blocks_for(nbytes);
#define CALL(DT) mo::nf4_dequantize_kernel<DT><<<g, 256, 0, s>>>(packed, nbytes, block_size, scales, y)
    DISPATCH_DT(dtype, CALL)
#undef CALL
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}
