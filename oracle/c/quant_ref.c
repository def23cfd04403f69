/* Bit-level C restatement of the reference's quantisation arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY: built by oracle/c/Makefile into oracle/c/libquant_ref.so and loaded
 * by oracle/cref.py for tests/, the smoke check and the CPU baseline of bench.py.  The product
 * never links or loads it.
 *
 * Independent of torch: E4M3 and E2M1 rounding are done on the bit patterns, so a disagreement
 * with the torch restatement (oracle/qtensor.py, oracle/fake_quant.py) exposes a mistake in
 * either.  Paths below are relative to the reference checkout; TQ = modelopt/torch/quantization.
 *
 * Compile with -O2 -ffp-contract=off -fno-fast-math: every fp32 operation must round once.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* number of threads the parallel loops below will use */
int qr_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ------------------------------------------------------------------ storage dtypes <-> fp32 */
enum { QR_F32 = 0, QR_F16 = 1, QR_BF16 = 2 };

static inline float bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* round to nearest even; NaN stays a quiet NaN */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u = f2u(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

static inline float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1Fu, m = h & 0x3FFu;
    if (e == 0x1F) return u2f(sign | 0x7F800000u | (m << 13));
    if (e == 0) return u2f(sign | f2u((float)m * 5.9604644775390625e-8f)); /* m * 2^-24 */
    return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

static inline uint16_t f32_to_f16(float f) {
    uint32_t u = f2u(f), sign = (u >> 16) & 0x8000u, a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u);
    if (a >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);          /* rounds to >= 65520 -> inf */
    if (a < 0x38800000u) {                                            /* below 2^-14: quantum 2^-24 */
        float r = u2f(a) + 0.5f;                                      /* 0.5 aligns 2^-24 to bit 0 */
        return (uint16_t)(sign | (f2u(r) - 0x3F000000u));
    }
    uint32_t t = a + 0xFFFu + ((a >> 13) & 1u);
    return (uint16_t)(sign | ((t - (112u << 23)) >> 13));
}

static inline float load_as_f32(const void* p, int64_t i, int dtype) {
    if (dtype == QR_F32) return ((const float*)p)[i];
    if (dtype == QR_F16) return f16_to_f32(((const uint16_t*)p)[i]);
    return bf16_to_f32(((const uint16_t*)p)[i]);
}

static inline void store_from_f32(void* p, int64_t i, int dtype, float v) {
    if (dtype == QR_F32) ((float*)p)[i] = v;
    else if (dtype == QR_F16) ((uint16_t*)p)[i] = f32_to_f16(v);
    else ((uint16_t*)p)[i] = f32_to_bf16(v);
}

static inline float round_to(float v, int dtype) {
    if (dtype == QR_F16) return f16_to_f32(f32_to_f16(v));
    if (dtype == QR_BF16) return bf16_to_f32(f32_to_bf16(v));
    return v;
}

/* ------------------------------------------------------------------ E4M3 (OCP e4m3fn)
 * What Tensor.to(torch.float8_e4m3fn) does on CPU: round to nearest even, subnormals kept
 * (quantum 2^-9), no saturation: anything that rounds above 448 -- i.e. |f| > 464, the tie at
 * 464 itself going to the even neighbour 448 -- and inf / NaN give the NaN byte 0x7F | sign. */
uint8_t qr_f32_to_e4m3(float f) {
    uint32_t u = f2u(f), sign = (u >> 24) & 0x80u, a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint8_t)(0x7F | sign);
    if (a < 0x3C800000u) {                                             /* < 2^-6 */
        float r = u2f(a) + 16384.0f;                                   /* aligns 2^-9 to bit 0 */
        return (uint8_t)((f2u(r) - 0x46800000u) | sign);
    }
    uint32_t t = a + 0x7FFFFu + ((a >> 20) & 1u);                      /* round mantissa to 3 bits */
    if (t >= 0x43F00000u) return (uint8_t)(0x7F | sign);               /* rounded to 480 or more */
    return (uint8_t)(((t - (120u << 23)) >> 20) | sign);
}

float qr_e4m3_to_f32(uint8_t b) {
    uint32_t sign = (uint32_t)(b & 0x80u) << 24, e = (b >> 3) & 0xFu, m = b & 7u;
    if ((b & 0x7Fu) == 0x7Fu) return u2f(sign | 0x7FC00000u);
    if (e == 0) return u2f(sign | f2u((float)m * 0.001953125f));
    return u2f(sign | ((e + 120u) << 23) | (m << 20));
}

/* ------------------------------------------------------------------ E2M1
 * NVFP4QTensor._cast_fp4, TQ/qtensor/nvfp4_tensor.py:100-141: sign = (v < 0); ordinal =
 * searchsorted([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5], |v|) (count of bounds < |v|), plus one
 * when |v| equals an odd-indexed bound (0.75, 1.75, 3.5): ties go to the even code.  NaN and
 * inf sort after every bound: ordinal 7. */
uint8_t qr_f32_to_e2m1(float v) {
    static const float bound[7] = {0.25f, 0.75f, 1.25f, 1.75f, 2.5f, 3.5f, 5.0f};
    float a = fabsf(v);
    uint32_t ord = 0;
    for (int i = 0; i < 7; ++i) ord += !(a <= bound[i]);               /* NaN counts as above */
    if (a == 0.75f || a == 1.75f || a == 3.5f) ord += 1;
    return (uint8_t)(((v < 0.0f) ? 8u : 0u) | ord);
}

float qr_e2m1_to_f32(uint8_t c) {
    /* e2m1 table of NVFP4QTensor.dequantize, TQ/qtensor/nvfp4_tensor.py:234-297; code 8 is +0 */
    static const float lut[16] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f,
                                  0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};
    return lut[c & 15u];
}

/* ------------------------------------------------------------------ abs-max
 * reduce_amax, TQ/utils.py:156-188: max |x| over everything (NaN propagates, as torch.max). */
float qr_absmax(const void* x, int64_t n, int dtype) {
    float m = 0.0f;
    for (int64_t i = 0; i < n; ++i) {
        float a = fabsf(load_as_f32(x, i, dtype));
        if (a != a) return a;
        m = a > m ? a : m;
    }
    return m;
}

/* ------------------------------------------------------------------ NVFP4 quantize + pack
 * NVFP4QTensor.quantize / get_weights_scaling_factor, TQ/qtensor/nvfp4_tensor.py:63-92,143-232:
 *   wsf2  = f32(amax) / (6 * 448)
 *   bs    = f32(block amax) / (6 * wsf2); 0 -> 1.0; wsf = e4m3(bs)
 *   v     = f32(x) / (f32(wsf) * wsf2); code = e2m1(v); byte = code[2i] | code[2i + 1] << 4
 * x is [rows, k] with k a multiple of `block`; `amax` is the tensor's abs-max. */
void qr_nvfp4_quantize(const void* x, int64_t rows, int64_t k, int dtype, int block, float amax,
                       uint8_t* packed, uint8_t* wsf, float* wsf2_out) {
    const float wsf2 = amax / 2688.0f;
    const float gs6 = 6.0f * wsf2;
    *wsf2_out = wsf2;
    const int64_t nblk = rows * k / block;
    /* blocks are independent; the threads only shorten the CPU baseline's wall time */
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < nblk; ++b) {
        const int64_t i0 = b * block;
        float bmax = 0.0f;
        int nan = 0;
        for (int j = 0; j < block; ++j) {
            float a = fabsf(load_as_f32(x, i0 + j, dtype));
            if (a != a) nan = 1;
            bmax = a > bmax ? a : bmax;
        }
        if (nan) bmax = NAN;
        float bs = bmax / gs6;
        if (bs == 0.0f) bs = 1.0f;
        const uint8_t sb = qr_f32_to_e4m3(bs);
        wsf[b] = sb;
        const float s = qr_e4m3_to_f32(sb) * wsf2;
        for (int j = 0; j < block; j += 2) {
            const uint8_t lo = qr_f32_to_e2m1(load_as_f32(x, i0 + j, dtype) / s);
            const uint8_t hi = qr_f32_to_e2m1(load_as_f32(x, i0 + j + 1, dtype) / s);
            packed[(i0 + j) >> 1] = (uint8_t)(lo | (hi << 4));
        }
    }
}

/* NVFP4QTensor.dequantize, TQ/qtensor/nvfp4_tensor.py:234-297:
 *   y = T( lut[code] * (f32(wsf) * wsf2) ) */
void qr_nvfp4_dequantize(const uint8_t* packed, const uint8_t* wsf, float wsf2, int64_t n,
                         int block, void* y, int dtype) {
    for (int64_t i = 0; i < n; ++i) {
        const uint8_t byte = packed[i >> 1];
        const uint8_t code = (i & 1) ? (byte >> 4) : (byte & 15u);
        const float s = qr_e4m3_to_f32(wsf[i / block]) * wsf2;
        store_from_f32(y, i, dtype, qr_e2m1_to_f32(code) * s);
    }
}

/* ------------------------------------------------------------------ FP8 fake quant, per tensor
 * _fp8_eager, TQ/tensor_quant.py:45-59: scale = 448 / amax (torch evaluates scalar / tensor as
 * reciprocal(amax) * 448), y = T( e4m3(f32(x) * scale) * reciprocal(scale) ); amax NULL: plain
 * round trip through E4M3. */
void qr_fp8_qdq(const void* x, int64_t n, int dtype, const float* amax, void* y) {
    float mul = 1.0f, inv = 1.0f;
    if (amax) {
        mul = (1.0f / amax[0]) * 448.0f;
        inv = 1.0f / mul;
    }
    for (int64_t i = 0; i < n; ++i) {
        float v = load_as_f32(x, i, dtype);
        if (amax) v = v * mul;
        v = qr_e4m3_to_f32(qr_f32_to_e4m3(v));
        if (amax) v = v * inv;
        store_from_f32(y, i, dtype, v);
    }
}

/* ------------------------------------------------------------------ integer fake quant, per tensor
 * _tensor_quant, TQ/tensor_quant.py:574-612 (fp32 math):
 *   bound = 2^(bits - 1 + unsigned) - 1; lo = unsigned ? 0 : (narrow ? -bound : -bound - 1)
 *   scale = bound / amax; amax <= 2^-24: scale 1 and output 0
 *   y = T( clamp(rne(x * scale), lo, bound) / scale ) */
void qr_int_qdq(const void* x, int64_t n, int dtype, float amax, int bits, int is_unsigned,
                int narrow, void* y) {
    const float bound = (float)((1 << (bits - 1 + (is_unsigned ? 1 : 0))) - 1);
    const float lo = is_unsigned ? 0.0f : (narrow ? -bound : -bound - 1.0f);
    const int dead = amax <= 5.9604644775390625e-8f;
    const float scale = bound / amax;
    const float mul = dead ? 0.0f : scale, div = dead ? 1.0f : scale;
    for (int64_t i = 0; i < n; ++i) {
        float q = nearbyintf(load_as_f32(x, i, dtype) * mul);            /* default mode: to even */
        q = q < lo ? lo : q;
        q = q > bound ? bound : q;
        store_from_f32(y, i, dtype, q / div);
    }
}

/* ------------------------------------------------------------------ INT4 block compress
 * INT4QTensor.quantize, TQ/qtensor/int4_tensor.py:40-88 (CPU branch), in dtype T:
 *   scale = T(T(1 / amax_block) * 7)   (torch's scalar / tensor), q = clamp(rne(T(x * scale)), -8, 7)
 *   byte = (q[2i] + 8) << 4 | (q[2i + 1] + 8).  n must be a multiple of `block`. */
void qr_int4_block_quantize(const void* x, int64_t n, int dtype, int block, void* scales,
                            uint8_t* packed) {
    for (int64_t b = 0; b < n / block; ++b) {
        const int64_t i0 = b * block;
        float amax = 0.0f;
        for (int j = 0; j < block; ++j) {
            float a = fabsf(load_as_f32(x, i0 + j, dtype));
            amax = (a > amax || a != a) ? a : amax;
        }
        const float scale = round_to(round_to(1.0f / amax, dtype) * 7.0f, dtype);
        store_from_f32(scales, b, dtype, scale);
        for (int j = 0; j < block; j += 2) {
            uint32_t nib[2];
            for (int h = 0; h < 2; ++h) {
                float q = nearbyintf(round_to(load_as_f32(x, i0 + j + h, dtype) * scale, dtype));
                q = q < -8.0f ? -8.0f : q;
                q = q > 7.0f ? 7.0f : q;
                nib[h] = (q == q) ? (uint32_t)((int)q + 8) : 0u;
            }
            packed[(i0 + j) >> 1] = (uint8_t)((nib[0] << 4) | nib[1]);
        }
    }
}

/* ------------------------------------------------------------------ FP8 / INT8 storage cast
 * FP8QTensor.quantize, TQ/qtensor/fp8_tensor.py:41-113 and INT8QTensor.quantize,
 * TQ/qtensor/int8_tensor.py:36-95, per tensor: q = fmt( via( f32(x) / scale ) ) where `via` is
 * the dtype torch's promotion gives the quotient.  fmt 0: E4M3 byte; fmt 1: int8 (rne, clamp). */
void qr_real_quantize(const void* x, int64_t n, int dtype, float scale, int via, int fmt,
                      uint8_t* out) {
    for (int64_t i = 0; i < n; ++i) {
        const float v = round_to(load_as_f32(x, i, dtype) / scale, via);
        if (fmt == 0) {
            out[i] = qr_f32_to_e4m3(v);
        } else {
            float q = nearbyintf(v);
            q = q < -128.0f ? -128.0f : q;
            q = q > 127.0f ? 127.0f : q;
            out[i] = (q == q) ? (uint8_t)(int8_t)(int)q : 0;
        }
    }
}

/* ------------------------------------------------------------------ block floating point (MX)
 * fused_amax_convert, TQ/src/tensor_quant_mx.cu:35-57,97-186,243-297 with the tables and
 * conversions of TQ/src/tensor_quant_mx.h:38-178, in IEEE fp32 / double (the reference kernel is
 * built with --use_fast_math).  Format numbers follow the reference's enum Types. */
enum { QR_E4M3 = 0, QR_E5M2, QR_INT8, QR_E0M3, QR_E1M2, QR_E3M0, QR_E2M1, QR_E3M2, QR_E2M3, QR_E8M0 };

static const float t_e2m1[8] = {0, 0.5f, 1, 1.5f, 2, 3, 4, 6};
static const float b_e2m1[7] = {0.25f, 0.75f, 1.25f, 1.75f, 2.5f, 3.5f, 5};
static const float t_e1m2[8] = {0, 0.5f, 1, 1.5f, 2, 2.5f, 3, 3.5f};
static const float b_e1m2[7] = {0.25f, 0.75f, 1.25f, 1.75f, 2.25f, 2.75f, 3.25f};
static const float t_e0m3[8] = {0, 1, 2, 3, 4, 5, 6, 7};
static const float b_e0m3[7] = {0.5f, 1.5f, 2.5f, 3.5f, 4.5f, 5.5f, 6.5f};
static const float t_e3m0[8] = {0, 0.25f, 0.5f, 1, 2, 4, 8, 16};
static const float b_e3m0[7] = {0.125f, 0.375f, 0.75f, 1.5f, 3, 6, 12};
static const float t_e3m2[32] = {0, 0.0625f, 0.125f, 0.1875f, 0.25f, 0.3125f, 0.375f, 0.4375f,
                                 0.5f, 0.625f, 0.75f, 0.875f, 1, 1.25f, 1.5f, 1.75f,
                                 2, 2.5f, 3, 3.5f, 4, 5, 6, 7, 8, 10, 12, 14, 16, 20, 24, 28};
static const float t_e2m3[32] = {0, 0.125f, 0.25f, 0.375f, 0.5f, 0.625f, 0.75f, 0.875f, 1, 1.125f,
                                 1.25f, 1.375f, 1.5f, 1.625f, 1.75f, 1.875f, 2, 2.25f, 2.5f, 2.75f,
                                 3, 3.25f, 3.5f, 3.75f, 4, 4.5f, 5, 5.5f, 6, 6.5f, 7, 7.5f};

/* nearest table value; a tie goes to the value with the even index, or up when ties_away */
static float table_round(float x, const float* values, const float* bounds, int n, int ties_away) {
    float sign = 1.0f;
    if (x < 0.0f) { sign = -1.0f; x = -x; }
    if (isinf(x) || isnan(x)) return sign * values[n - 1];
    for (int i = 0; i < n - 1; ++i) {
        const float bound = bounds ? bounds[i] : 0.5f * (values[i] + values[i + 1]);
        if (x < bound) return sign * values[i];
        if (x == bound) return sign * ((ties_away || (i & 1)) ? values[i + 1] : values[i]);
    }
    return sign * values[n - 1];
}

/* fp32 -> E5M2 value (round to nearest even, subnormals kept, saturating at 57344) */
static float round_e5m2_sat(float f) {
    uint32_t u = f2u(f), sign = u & 0x80000000u, a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return f;
    float m = u2f(a);
    if (m > 57344.0f) m = 57344.0f;
    if (m < 6.103515625e-05f) {                                  /* below 2^-14: quantum 2^-16 */
        m = (m + 128.0f) - 128.0f;                               /* 2^7 aligns 2^-16 to bit 0 */
    } else {
        uint32_t b = f2u(m);
        b = (b + 0xFFFFFu + ((b >> 21) & 1u)) & 0xFFE00000u;     /* keep 2 mantissa bits */
        m = u2f(b);
        if (m > 57344.0f) m = 57344.0f;
    }
    return u2f(f2u(m) | sign);
}

float qr_convert_to_types(float x, int fmt) {
    switch (fmt) {
        case QR_E4M3: {
            if (x != x) return x;
            float c = x > 448.0f ? 448.0f : (x < -448.0f ? -448.0f : x);
            return qr_e4m3_to_f32(qr_f32_to_e4m3(c));
        }
        case QR_E5M2: return round_e5m2_sat(x);
        case QR_INT8: {
            float q = nearbyintf(x);
            return q > 127.0f ? 127.0f : (q < -127.0f ? -127.0f : q);
        }
        case QR_E2M1: return table_round(x, t_e2m1, b_e2m1, 8, 0);
        case QR_E0M3: return table_round(x, t_e0m3, b_e0m3, 8, 0);
        case QR_E1M2: return table_round(x, t_e1m2, b_e1m2, 8, 0);
        case QR_E3M0: return table_round(x, t_e3m0, b_e3m0, 8, 1);
        case QR_E3M2: return table_round(x, t_e3m2, NULL, 32, 0);
        case QR_E2M3: return table_round(x, t_e2m3, NULL, 32, 0);
        default: return 0.0f;
    }
}

static float format_max(int fmt) {
    static const float m[9] = {448.0f, 57344.0f, 127.0f, 7.0f, 3.5f, 16.0f, 6.0f, 28.0f, 7.5f};
    return fmt >= 0 && fmt < 9 ? m[fmt] : 0.0f;
}

/* x [rows, k]; blocks of `block` along k, zero padded; global_amax NULL, one value
 * (n_global == 1) or one per row (n_global == rows). */
void qr_block_fp_qdq(const void* x, int64_t rows, int64_t k, int dtype, int block, int fmt,
                     int scale_fmt, const float* global_amax, int64_t n_global, void* y) {
    const int64_t nb = (k + block - 1) / block;
    for (int64_t r = 0; r < rows; ++r) {
        for (int64_t b = 0; b < nb; ++b) {
            float amax = 0.0f;
            for (int j = 0; j < block; ++j) {
                const int64_t c = b * block + j;
                float a = c < k ? fabsf(load_as_f32(x, r * k + c, dtype)) : 0.0f;
                if (a > 3.402823466e+38f) a = 3.402823466e+38f;      /* clamp, :192 */
                amax = fmaxf(amax, a);                               /* drops NaN */
            }
            float scale = 1.0f, unscale = 1.0f;
            const int bad_local = amax == 0.0f || isinf(amax) || isnan(amax);
            if (global_amax) {
                const float g = global_amax[n_global == rows && n_global > 1 ? r : 0];
                if (!(bad_local || g == 0.0f || isinf(g) || isnan(g))) {
                    const float fmax = format_max(fmt), smax = format_max(scale_fmt);
                    const float local_unscale = amax / fmax;
                    const double two_level = (double)smax * (double)(fmax / g);
                    const double q = (double)qr_convert_to_types((float)(local_unscale * two_level),
                                                                 scale_fmt) / two_level;
                    scale = (float)(1.0 / q);
                    unscale = (float)q;
                }
            } else if (!bad_local) {
                if (scale_fmt == QR_E8M0) {
                    const float ratio = amax / format_max(fmt);
                    const uint32_t bits = f2u(ratio), ef = (bits >> 23) & 0xFFu, mant = bits & 0x7FFFFFu;
                    const int e = (mant > 0 && ef != 0xFEu && !(ef == 0 && mant <= 0x400000u))
                                      ? (int)ef - 126 : (int)ef - 127;
                    scale = ldexpf(1.0f, -e);
                    unscale = ldexpf(1.0f, e);
                } else {
                    double s = (double)format_max(fmt) / (double)amax;
                    const double inv = (double)qr_convert_to_types((float)(1.0 / s), scale_fmt);
                    scale = (float)(1.0 / inv);
                    unscale = (float)inv;
                }
            }
            for (int j = 0; j < block; ++j) {
                const int64_t c = b * block + j;
                if (c >= k) break;
                const float v = load_as_f32(x, r * k + c, dtype);
                const float q = qr_convert_to_types(fabsf(v) * scale, fmt) * unscale;
                store_from_f32(y, r * k + c, dtype, v < 0.0f ? -q : q);
            }
        }
    }
}
