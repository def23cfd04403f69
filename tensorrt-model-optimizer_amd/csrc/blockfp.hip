// Block floating point fake quantisation for gfx950: the MX formats (elements E4M3 / E5M2 / E3M2 /
// E2M3 / E2M1 / INT8 ... with one shared power-of-two E8M0 scale per block) and the two-level
// variant with a minifloat block scale under a global abs-max.
//
// HBM-bound: one read and one write of the tensor (4 bytes per bf16 element).  A lane owns a
// chunk of 8 elements, the 1, 2 or 4 lanes of a block combine their abs-max with DPP moves; one
// workgroup per tile of 1024 chunks, the loads of a lane's 4 chunks issued before the math.
#include "common.h"

namespace mo {

// Nearest value of a small float format with M mantissa bits whose smallest normal number is
// 2^EMIN (below it the quantum stays 2^(EMIN - M)), saturating at fmax; `a` is non-negative,
// infinities and NaN give fmax.  Ties go to the even multiple of the quantum -- the value with
// the even index in the reference's tables -- or away from zero when TIES_AWAY.
template <int M, int EMIN, bool TIES_AWAY>
__device__ __forceinline__ float round_minifloat(float a, float fmax) {
    if (!(a < __builtin_inff())) return fmax;
    int e = (int)(f2u(a) >> 23) - 127;
    e = e > EMIN ? e : EMIN;
    const float t = __builtin_ldexpf(a, M - e);
    const float r = TIES_AWAY ? __builtin_floorf(t + 0.5f) : __builtin_rintf(t);
    const float v = __builtin_ldexpf(r, e - M);
    return v < fmax ? v : fmax;
}

// E5M2: round to nearest even with subnormals (quantum 2^-16), saturating at 57344; NaN stays.
__device__ __forceinline__ float round_e5m2_sat(float a) {
    if (a != a) return a;
    a = a < 57344.0f ? a : 57344.0f;
    int e = (int)(f2u(a) >> 23) - 127;
    e = e > -14 ? e : -14;
    const float v = __builtin_ldexpf(__builtin_rintf(__builtin_ldexpf(a, 2 - e)), e - 2);
    return v < 57344.0f ? v : 57344.0f;
}

template <int FMT>
__device__ __forceinline__ float convert_elem(float a) {  // a >= 0 (or NaN)
    if constexpr (FMT == MO_EF_E4M3) return round_e4m3<true>(a);
    else if constexpr (FMT == MO_EF_E5M2) return round_e5m2_sat(a);
    else if constexpr (FMT == MO_EF_INT8) {
        const float q = __builtin_rintf(a);
        return q > 127.0f ? 127.0f : q;  // NaN stays NaN
    }
    else if constexpr (FMT == MO_EF_E0M3) return round_minifloat<3, 3, false>(a, 7.0f);
    else if constexpr (FMT == MO_EF_E1M2) return round_minifloat<2, 1, false>(a, 3.5f);
    else if constexpr (FMT == MO_EF_E3M0) return round_minifloat<0, -2, true>(a, 16.0f);
    else if constexpr (FMT == MO_EF_E2M1) return round_minifloat<1, 0, false>(a, 6.0f);
    else if constexpr (FMT == MO_EF_E3M2) return round_minifloat<2, -2, false>(a, 28.0f);
    else return round_minifloat<3, 0, false>(a, 7.5f);  // E2M3
}

__device__ __forceinline__ float convert_runtime(float a, int fmt) {
    switch (fmt) {
        case MO_EF_E4M3: return convert_elem<MO_EF_E4M3>(a);
        case MO_EF_E5M2: return convert_elem<MO_EF_E5M2>(a);
        case MO_EF_INT8: return convert_elem<MO_EF_INT8>(a);
        case MO_EF_E0M3: return convert_elem<MO_EF_E0M3>(a);
        case MO_EF_E1M2: return convert_elem<MO_EF_E1M2>(a);
        case MO_EF_E3M0: return convert_elem<MO_EF_E3M0>(a);
        case MO_EF_E2M1: return convert_elem<MO_EF_E2M1>(a);
        case MO_EF_E3M2: return convert_elem<MO_EF_E3M2>(a);
        default: return convert_elem<MO_EF_E2M3>(a);
    }
}

__host__ __device__ __forceinline__ float elem_format_max(int fmt) {
    switch (fmt) {
        case MO_EF_E4M3: return 448.0f;
        case MO_EF_E5M2: return 57344.0f;
        case MO_EF_INT8: return 127.0f;
        case MO_EF_E0M3: return 7.0f;
        case MO_EF_E1M2: return 3.5f;
        case MO_EF_E3M0: return 16.0f;
        case MO_EF_E2M1: return 6.0f;
        case MO_EF_E3M2: return 28.0f;
        default: return 7.5f;
    }
}

struct BlockScale { float scale, unscale; };

// amax: block abs-max with |x| clamped to FLT_MAX and NaN elements ignored.
template <int FMT>
__device__ __forceinline__ BlockScale block_scale(float amax, int scale_fmt, bool has_global,
                                                  float global_amax) {
    BlockScale s = {1.0f, 1.0f};
    if (amax == 0.0f) return s;  // finite by construction
    const float fmax = elem_format_max(FMT);
    if (has_global) {
        // two-level scale: the block's unscale, quantised to scale_fmt relative to the global amax
        if (global_amax == 0.0f || !(__builtin_fabsf(global_amax) < __builtin_inff())) return s;
        const float smax = elem_format_max(scale_fmt);
        const float local_unscale = amax / fmax;
        const double two_level = (double)smax * (double)(fmax / global_amax);
        const double q = (double)convert_runtime((float)((double)local_unscale * two_level), scale_fmt) /
                         two_level;
        s.scale = (float)(1.0 / q);
        s.unscale = (float)q;
    } else if (scale_fmt == MO_EF_E8M0) {
        // unscale = 2^ceil(log2(amax / fmax)), read off the bits of the fp32 quotient
        const uint32_t bits = f2u(amax / fmax), ef = (bits >> 23) & 0xFFu, mant = bits & 0x7FFFFFu;
        const int e = (mant > 0 && ef != 0xFEu && !(ef == 0 && mant <= 0x400000u)) ? (int)ef - 126
                                                                                   : (int)ef - 127;
        s.scale = __builtin_ldexpf(1.0f, -e);
        s.unscale = __builtin_ldexpf(1.0f, e);
    } else {
        const double sc = (double)fmax / (double)amax;
        const double inv = (double)convert_runtime((float)(1.0 / sc), scale_fmt);
        s.scale = (float)(1.0 / inv);
        s.unscale = (float)inv;
    }
    return s;
}

constexpr int kBlockFpTileChunks = 1024;

// x viewed as [rows, kp] chunks with kp = k rounded up to whole blocks (zero padded).
template <int DT, int FMT, bool FLAT>
__global__ __launch_bounds__(256) void block_fp_qdq_kernel(
    const void* __restrict__ x, void* __restrict__ y, int64_t total_chunks, int64_t k, int64_t cpr,
    int lg_g, int scale_fmt, const float* __restrict__ global_amax, int per_row) {
    const int64_t c0 = (int64_t)blockIdx.x * kBlockFpTileChunks + threadIdx.x;
    float v[4][8];
    int64_t base[4], col[4], row[4];
    RawChunk<DT> raw[4];
    float gl[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if constexpr (FLAT) {
        // all loads (the global amax of a chunk's row too) in straight-line code ahead of the
        // first store; a chunk past the end re-reads the last one and is not stored
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            int64_t c = c0 + u * 256;
            c = c < total_chunks ? c : total_chunks - 1;
            col[u] = c << 3;
            base[u] = row[u] = 0;
            load_raw<DT>(x, col[u], raw[u]);
        }
        if (global_amax) {
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                int64_t r = 0;
                if (per_row) {
                    const int64_t c = col[u] >> 3;
                    if (total_chunks <= 0xFFFFFFFFll) r = (uint32_t)c / (uint32_t)cpr;
                    else r = c / cpr;
                }
                gl[u] = global_amax[r];
            }
        }
    } else {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t c = c0 + u * 256;
            base[u] = col[u] = row[u] = 0;
#pragma unroll
            for (int j = 0; j < 8; ++j) v[u][j] = 0.0f;
            if (c < total_chunks) {
                if (total_chunks <= 0xFFFFFFFFll) row[u] = (uint32_t)c / (uint32_t)cpr;
                else row[u] = c / cpr;
                col[u] = (c - row[u] * cpr) << 3;
                base[u] = row[u] * k;
                load_chunk_guarded<DT>(x, base[u], col[u], k, v[u]);
            }
        }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const bool live = c0 + u * 256 < total_chunks;
        if constexpr (FLAT) unpack_raw<DT>(raw[u], v[u]);
        uint32_t m = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            uint32_t t = f2u(v[u][j]) & 0x7FFFFFFFu;
            t = t > 0x7F800000u ? 0u : (t < 0x7F7FFFFFu ? t : 0x7F7FFFFFu);  // drop NaN, clamp inf
            m = t > m ? t : m;
        }
        m = group_max_u32(m, lg_g);  // total_chunks is a multiple of the group size
        if constexpr (!FLAT) {
            if (!live) continue;
        }
        float g = gl[u];
        if constexpr (!FLAT) {
            if (global_amax) g = global_amax[per_row ? row[u] : 0];
        }
        const BlockScale s = block_scale<FMT>(u2f(m), scale_fmt, global_amax != nullptr, g);
        float o[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float q = convert_elem<FMT>(__builtin_fabsf(v[u][j]) * s.scale) * s.unscale;
            o[j] = v[u][j] < 0.0f ? -q : q;
        }
        if constexpr (FLAT) {
            if (live) store_chunk<DT>(y, col[u], o);
        } else {
            store_chunk_guarded<DT>(y, base[u], col[u], k, o);
        }
    }
}

template <int DT, int FMT>
static void launch_block_fp(const void* x, void* y, int64_t rows, int64_t k, int64_t kp, int lg_g,
                            int scale_fmt, const float* global_amax, int per_row, hipStream_t s) {
    const int64_t cpr = kp / 8, total = rows * cpr;
    const unsigned grid = (unsigned)((total + kBlockFpTileChunks - 1) / kBlockFpTileChunks);
    const bool flat = (k == kp) && ((((uintptr_t)x | (uintptr_t)y) & 15u) == 0);
    if (flat)
        block_fp_qdq_kernel<DT, FMT, true><<<grid, 256, mo::ballast_bytes("block_fp_qdq_kernel", 0), s>>>(x, y, total, k, cpr, lg_g, scale_fmt,
                                                                global_amax, per_row);
    else
        block_fp_qdq_kernel<DT, FMT, false><<<grid, 256, mo::ballast_bytes("block_fp_qdq_kernel", 0), s>>>(x, y, total, k, cpr, lg_g, scale_fmt,
                                                                 global_amax, per_row);
}

}  // namespace mo

extern "C" int mo_block_fp_qdq(const void* x, void* y, int64_t rows, int64_t k, int dtype,
                               int block_size, int format, int scale_format,
                               const float* global_amax, int64_t n_global_amax, void* stream) {
    if (rows < 0 || k < 0) return MO_ERR_ARG;
    if (block_size != 8 && block_size != 16 && block_size != 32) return MO_ERR_UNSUPPORTED;
    if (format < MO_EF_E4M3 || format > MO_EF_E2M3) return MO_ERR_UNSUPPORTED;
    if (scale_format < MO_EF_E4M3 || scale_format > MO_EF_E8M0) return MO_ERR_UNSUPPORTED;
    if (global_amax && scale_format == MO_EF_E8M0) return MO_ERR_UNSUPPORTED;
    if (global_amax && n_global_amax != 1 && n_global_amax != rows) return MO_ERR_ARG;
    if (rows == 0 || k == 0) return MO_OK;
    if (!x || !y) return MO_ERR_ARG;
    const int64_t kp = (k + block_size - 1) / block_size * block_size;
    if ((rows * (kp / 8) + mo::kBlockFpTileChunks - 1) / mo::kBlockFpTileChunks > 0x7FFFFFFF)
        return MO_ERR_UNSUPPORTED;
    const int lg_g = block_size == 8 ? 0 : (block_size == 16 ? 1 : 2);
    const int per_row = global_amax && n_global_amax == rows && rows > 1;
    hipStream_t s = (hipStream_t)stream;
#define CALL_FMT(DT)                                                                                  \
    switch (format) {                                                                                 \
        case MO_EF_E4M3: mo::launch_block_fp<DT, MO_EF_E4M3>(x, y, rows, k, kp, lg_g, scale_format, global_amax, per_row, s); break; \
        case MO_EF_E5M2: mo::launch_block_fp<DT, MO_EF_E5M2>(x, y, rows, k, kp, lg_g, scale_format, global_amax, per_row, s); break; \
        case MO_EF_INT8: mo::launch_block_fp<DT, MO_EF_INT8>(x, y, rows, k, kp, lg_g, scale_format, global_amax, per_row, s); break; \
        case MO_EF_E0M3: mo::launch_block_fp<DT, MO_EF_E0M3>(x, y, rows, k, kp, lg_g, scale_format, global_amax, per_row, s); break; \
        case MO_EF_E1M2: mo::launch_block_fp<DT, MO_EF_E1M2>(x, y, rows, k, kp, lg_g, scale_format, global_amax, per_row, s); break; \
        case MO_EF_E3M0: mo::launch_block_fp<DT, MO_EF_E3M0>(x, y, rows, k, kp, lg_g, scale_format, global_amax, per_row, s); break; \
        case MO_EF_E2M1: mo::launch_block_fp<DT, MO_EF_E2M1>(x, y, rows, k, kp, lg_g, scale_format, global_amax, per_row, s); break; \
        case MO_EF_E3M2: mo::launch_block_fp<DT, MO_EF_E3M2>(x, y, rows, k, kp, lg_g, scale_format, global_amax, per_row, s); break; \
        default: mo::launch_block_fp<DT, MO_EF_E2M3>(x, y, rows, k, kp, lg_g, scale_format, global_amax, per_row, s); break;         \
    }
    switch (dtype) {
        case MO_F32: CALL_FMT(MO_F32); break;
        case MO_F16: CALL_FMT(MO_F16); break;
        case MO_BF16: CALL_FMT(MO_BF16); break;
        default: return MO_ERR_DTYPE;
    }
#undef CALL_FMT
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

// ------------------------------------------------------------------------------ element casts
// y[i] = nearest value of `fmt` for x[i], sign carried over: the element conversion on its own
// (no block scale).  E8M0 is a scale-only format and converts to 0, as in the reference.
namespace mo {
__global__ __launch_bounds__(256) void convert_to_format_kernel(const float* __restrict__ x,
                                                                float* __restrict__ y, int64_t n,
                                                                int fmt) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float v = x[i];
    float q = 0.0f;
    if (fmt != MO_EF_E8M0) {
        q = convert_runtime(__builtin_fabsf(v), fmt);
        if (fmt == MO_EF_E4M3 || fmt == MO_EF_E5M2) q = __builtin_copysignf(q, v);
        else if (v < 0.0f) q = -q;
    }
    y[i] = q;
}
}  // namespace mo

extern "C" int mo_convert_to_format(const float* x, float* y, int64_t n, int format, void* stream) {
    if (n < 0) return MO_ERR_ARG;
    if (format < MO_EF_E4M3 || format > MO_EF_E8M0) return MO_ERR_UNSUPPORTED;
    if (n == 0) return MO_OK;
    if (!x || !y) return MO_ERR_ARG;
    const int64_t grid = (n + 255) / 256;
    if (grid > 0x7FFFFFFF) return MO_ERR_UNSUPPORTED;
    mo::convert_to_format_kernel<<<(unsigned)grid, 256, 0, (hipStream_t)stream>>>(x, y, n, format);
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

// ------------------------------------------------------------------------------ MXFP4 storage
// Packed MXFP4: blocks of `block` elements share the E8M0 byte 127 + ceil(log2(amax / 6))
// (clamped below at -127); codes are sign << 3 | ordinal with the ordinal = number of E2M1 bounds
// strictly below |x / 2^e| (ties go to the smaller magnitude) and the sign bit set for every
// element that is not positive -- zero packs as code 8; byte i = code[2i] | code[2i + 1] << 4.
namespace mo {

// ceil(log2(v)) clamped below at -127 for a positive finite fp32 v, read off the bits
__device__ __forceinline__ int ceil_log2_clamped(float v) {
    const uint32_t bits = f2u(v), ef = bits >> 23, mant = bits & 0x7FFFFFu;
    if (ef == 0) return mant > 0x400000u ? -126 : -127;  // subnormal: above 2^-127 or not
    return (int)ef - 127 + (mant != 0);
}

__device__ __forceinline__ uint32_t mxfp4_code(float v) {
    const float a = __builtin_fabsf(v);
    const uint32_t ord = (uint32_t)(a > 0.25f) + (uint32_t)(a > 0.75f) + (uint32_t)(a > 1.25f) +
                         (uint32_t)(a > 1.75f) + (uint32_t)(a > 2.5f) + (uint32_t)(a > 3.5f) +
                         (uint32_t)(a > 5.0f);
    return ord | (v > 0.0f ? 0u : 8u);
}

template <int DT>
__global__ __launch_bounds__(256) void mxfp4_quantize_kernel(const void* __restrict__ x,
                                                             int64_t chunks, int lg_g,
                                                             uint32_t* __restrict__ packed,
                                                             uint8_t* __restrict__ scales) {
    const int64_t c0 = (int64_t)blockIdx.x * kBlockFpTileChunks + threadIdx.x;
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
        m = group_max_u32(m, lg_g);
        if (c >= chunks) continue;
        const float amax = u2f(m);
        // amax == 0: log2(0) = -inf, clamped to -127.  Infinite or NaN amax has no defined byte in
        // the reference (float -> uint8 of inf / NaN); 255 here.
        int e = -127;
        const bool finite = m < 0x7F800000u;
        if (amax > 0.0f && finite) e = ceil_log2_clamped(amax / 6.0f);
        if ((threadIdx.x & ((1 << lg_g) - 1)) == 0) scales[c >> lg_g] = finite ? (uint8_t)(e + 127) : 255;
        uint32_t w = 0;
        // the reference divides by 2^e: identical to the product with 2^-e unless 2^-e itself
        // overflows (e = -127).  One branch per block, so that the common case carries no division
        if (e >= -126 && finite && DT != MO_F32) {
            // 16-bit inputs in a finite block: the hardware E2M1 conversion (round to nearest
            // even, sign from the sign bit) gives the code once two differences are ironed out.
            // Ties: the rule here sends a value that sits exactly on a bound to the smaller
            // magnitude, so the magnitude is moved one fp32 ulp towards zero first -- x / 2^e
            // carries at most 11 significant bits, so nothing sits one fp32 ulp *above* a bound
            // and could be dragged onto it.  Zeros: +0 and -0 both pack as code 8, i.e. -0.
            const float inv = __builtin_ldexpf(1.0f, -e);
#pragma unroll
            for (int j = 0; j < 8; j += 2) {
                const uint32_t a = f2u(v[j] * inv), b = f2u(v[j + 1] * inv);
                const float na = u2f((a << 1) == 0u ? 0x80000000u : a - 1u);
                const float nb = u2f((b << 1) == 0u ? 0x80000000u : b - 1u);
                w = fp4_pair(w, na, nb, j >> 1);
            }
        } else if (e >= -126) {
            const float inv = __builtin_ldexpf(1.0f, -e);
#pragma unroll
            for (int j = 0; j < 8; ++j) w |= mxfp4_code(v[j] * inv) << (4 * j);
        } else {
            const float d = __builtin_ldexpf(1.0f, e);
#pragma unroll
            for (int j = 0; j < 8; ++j) w |= mxfp4_code(v[j] / d) << (4 * j);
        }
        __builtin_nontemporal_store(w, packed + c);
    }
}

template <int DT>
__global__ __launch_bounds__(256) void mxfp4_dequantize_kernel(const uint32_t* __restrict__ packed,
                                                               const uint8_t* __restrict__ scales,
                                                               int64_t chunks, int lg_g,
                                                               void* __restrict__ y) {
    const int64_t c0 = (int64_t)blockIdx.x * kBlockFpTileChunks + threadIdx.x;
    uint32_t w[4], sb[4];
    // loads in straight-line code (a chunk past the end re-reads the last one), stores conditional
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        int64_t c = c0 + u * 256;
        c = c < chunks ? c : chunks - 1;
        w[u] = __builtin_nontemporal_load(packed + c);
        sb[u] = scales[c >> lg_g];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int64_t c = c0 + u * 256;
        const float s = __builtin_ldexpf(1.0f, (int)sb[u] - 127);  // exp2(byte - 127) in fp32
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t code = (w[u] >> (4 * j)) & 0xFu;
            const float mag = e2m1_to_f32(code & 7u);
            v[j] = ((code & 8u) ? -mag : mag) * s;   // code 8 is -0
        }
        if (c < chunks) store_chunk<DT>(y, c << 3, v);
    }
}

}  // namespace mo

static int mxfp4_check(int64_t n, int block_size, int* lg_g) {
    if (n < 0) return MO_ERR_ARG;
    *lg_g = -1;
    for (int k = 0; k <= 6; ++k)
        if (block_size == (8 << k)) *lg_g = k;
    if (*lg_g < 0) return MO_ERR_UNSUPPORTED;
    if (n % block_size) return MO_ERR_ARG;
    if ((n / 8 + mo::kBlockFpTileChunks - 1) / mo::kBlockFpTileChunks > 0x7FFFFFFF) return MO_ERR_UNSUPPORTED;
    return MO_OK;
}

extern "C" int mo_mxfp4_quantize(const void* x, int64_t n, int dtype, int block_size,
                                 uint8_t* packed, uint8_t* scales, void* stream) {
    int lg_g;
    const int rc = mxfp4_check(n, block_size, &lg_g);
    if (rc != MO_OK) return rc;
    if (n == 0) return MO_OK;
    if (!x || !packed || !scales) return MO_ERR_ARG;
    if (((uintptr_t)x & 15u) || ((uintptr_t)packed & 3u)) return MO_ERR_ARG;
    const int64_t chunks = n / 8;
    const unsigned grid = (unsigned)((chunks + mo::kBlockFpTileChunks - 1) / mo::kBlockFpTileChunks);
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case MO_F32: mo::mxfp4_quantize_kernel<MO_F32><<<grid, 256, mo::ballast_bytes("mxfp4_quantize_kernel", 0), s>>>(x, chunks, lg_g, (uint32_t*)packed, scales); break;
        case MO_F16: mo::mxfp4_quantize_kernel<MO_F16><<<grid, 256, mo::ballast_bytes("mxfp4_quantize_kernel", 0), s>>>(x, chunks, lg_g, (uint32_t*)packed, scales); break;
        case MO_BF16: mo::mxfp4_quantize_kernel<MO_BF16><<<grid, 256, mo::ballast_bytes("mxfp4_quantize_kernel", 0), s>>>(x, chunks, lg_g, (uint32_t*)packed, scales); break;
        default: return MO_ERR_DTYPE;
    }
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_mxfp4_dequantize(const uint8_t* packed, const uint8_t* scales, int64_t n,
                                   int block_size, void* y, int dtype, void* stream) {
    int lg_g;
    const int rc = mxfp4_check(n, block_size, &lg_g);
    if (rc != MO_OK) return rc;
    if (n == 0) return MO_OK;
    if (!y || !packed || !scales) return MO_ERR_ARG;
    if (((uintptr_t)y & 15u) || ((uintptr_t)packed & 3u)) return MO_ERR_ARG;
    const int64_t chunks = n / 8;
    const unsigned grid = (unsigned)((chunks + mo::kBlockFpTileChunks - 1) / mo::kBlockFpTileChunks);
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case MO_F32: mo::mxfp4_dequantize_kernel<MO_F32><<<grid, 256, mo::ballast_bytes("mxfp4_dequantize_kernel", 0), s>>>((const uint32_t*)packed, scales, chunks, lg_g, y); break;
        case MO_F16: mo::mxfp4_dequantize_kernel<MO_F16><<<grid, 256, mo::ballast_bytes("mxfp4_dequantize_kernel", 0), s>>>((const uint32_t*)packed, scales, chunks, lg_g, y); break;
        case MO_BF16: mo::mxfp4_dequantize_kernel<MO_BF16><<<grid, 256, mo::ballast_bytes("mxfp4_dequantize_kernel", 0), s>>>((const uint32_t*)packed, scales, chunks, lg_g, y); break;
        default: return MO_ERR_DTYPE;
    }
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}
