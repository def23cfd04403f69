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
        const float scale = round_via<DT>(round_via<DT>(1.0f / amax) * 7.0f);
        store_elem<DT>(scales, b, scale);
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
template <int DT>
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
                float q = __builtin_rintf(load_elem<DT>(w, row * k + col) / ws[row * nsb + col / bs]);
                q = q < -8.0f ? -8.0f : q;
                q = q > 7.0f ? 7.0f : q;
                nib[h] = (q == q) ? ((uint32_t)(int)q & 0xFu) : 0u;
            }
            out[j * k + col] = (uint8_t)(nib[0] | (nib[1] << 4));
        }
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

extern "C" int mo_int4_block_quantize(const void* x, int64_t n, int64_t block_size, int dtype,
                                      void* scales, uint8_t* packed, void* stream) {
    if (n < 0 || block_size <= 0 || (block_size & 1)) return MO_ERR_ARG;
    if (n == 0) return MO_OK;
    if (!x || !scales || !packed) return MO_ERR_ARG;
    const int64_t nblocks = (n + block_size - 1) / block_size;
    hipStream_t s = (hipStream_t)stream;
    const unsigned g = mo::blocks_for(nblocks);
#define CALL(DT) mo::int4_block_quantize_kernel<DT><<<g, 256, 0, s>>>(x, n, block_size, nblocks, scales, packed)
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
    const unsigned g = mo::blocks_for(nbytes);
#define CALL(DT) mo::int4_block_dequantize_kernel<DT><<<g, 256, 0, s>>>(packed, nbytes, block_size, scales, y)
    DISPATCH_DT(dtype, CALL)
#undef CALL
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_int4_pack_rows(const void* w, int64_t batch, int64_t n_rows, int64_t k,
                                 int64_t block_size, int dtype, const float* ws, uint8_t* out,
                                 void* stream) {
    if (batch < 0 || n_rows < 0 || k < 0 || block_size <= 0) return MO_ERR_ARG;
    if ((n_rows & 1) || (k % block_size)) return MO_ERR_ARG;
    if (batch == 0 || n_rows == 0 || k == 0) return MO_OK;
    if (!w || !ws || !out) return MO_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    // a stack of `batch` matrices is one matrix of batch * n_rows rows (n_rows is even)
    const int64_t rows = batch * n_rows;
    const unsigned g = mo::blocks_for((rows >> 1) * ((k + 7) >> 3));
#define CALL(DT) mo::int4_pack_rows_kernel<DT><<<g, 256, 0, s>>>(w, rows, k, block_size, ws, out)
    DISPATCH_DT(dtype, CALL)
#undef CALL
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}
