// Squared quantisation error of a tensor for several candidate amax values in one pass, for
// gfx950: the inner loop of the MSE amax search.
//
// The reference computes, per candidate, fake quantisation of the fp32 tensor, an element-wise
// squared difference and a sum -- five full-size passes per candidate.  Here the tensor is read
// once; every element is quantised against up to 16 candidates held in registers and the squared
// errors are accumulated per candidate.  ALU-bound (about 12 operations per element and
// candidate), not HBM-bound.
#include "common.h"
#include "qdq_ops.h"

namespace mo {

__device__ __forceinline__ float wave_sum_f32(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}

// One scale for the whole tensor.  A capped grid of workgroups strides over tiles of 512 chunks
// (two per lane in flight); one atomic add per candidate and workgroup at the end.
template <int DT, int KN, bool SAT, typename Op>
__global__ __launch_bounds__(256) void sq_err_tensor_kernel(const void* __restrict__ x, int64_t n,
                                                            const float* __restrict__ cand, int K,
                                                            Op op, float* __restrict__ loss) {
    __shared__ float smem[4][KN];
    typename Op::Scale s[KN];
    float part[KN];
#pragma unroll
    for (int k = 0; k < KN; ++k) {
        part[k] = 0.0f;
        s[k] = op.make(cand[k < K ? k : 0]);
    }
    const int64_t chunks = n >> 3;
    for (int64_t c = (int64_t)blockIdx.x * 512 + threadIdx.x; c < chunks; c += (int64_t)gridDim.x * 512) {
        RawChunk<DT> raw[2];
        zero_raw<DT>(raw[1]);
        load_raw<DT>(x, c << 3, raw[0]);
        const bool second = c + 256 < chunks;
        if (second) load_raw<DT>(x, (c + 256) << 3, raw[1]);
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            if (u == 1 && !second) continue;
            float v[8];
            unpack_raw<DT>(raw[u], v);
#pragma unroll
            for (int k = 0; k < KN; ++k) {
                if (k < K) {  // uniform
                    float acc = 0.0f;
                    // one decision per candidate between the branch-free arithmetic and the
                    // general one, not one per element
                    if (Op::is_fast(s[k])) {
#pragma unroll
                        for (int j = 0; j < 8; ++j) {
                            const float d = v[j] - op.template apply_fast<SAT>(v[j], s[k]);
                            acc += d * d;
                        }
                    } else {
#pragma unroll
                        for (int j = 0; j < 8; ++j) {
                            const float d = v[j] - op.template apply<SAT>(v[j], s[k]);
                            acc += d * d;
                        }
                    }
                    part[k] += acc;
                }
            }
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 7)) {  // tail elements
        const float v = load_elem<DT>(x, (chunks << 3) + threadIdx.x);
#pragma unroll
        for (int k = 0; k < KN; ++k) {
            if (k < K) {
                const float d = v - op.template apply<SAT>(v, s[k]);
                part[k] += d * d;
            }
        }
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int k = 0; k < KN; ++k) {
        const float t = wave_sum_f32(part[k]);
        if (lane == 0) smem[wave][k] = t;
    }
    __syncthreads();
    if (threadIdx.x < K)
        atomicAdd(loss + threadIdx.x, (smem[0][threadIdx.x] + smem[1][threadIdx.x]) +
                                          (smem[2][threadIdx.x] + smem[3][threadIdx.x]));
}

// One scale per row of length inner (inner % 8 == 0): a wavefront per row, its lanes striding
// over the row's chunks.  Row r feeds channel r % axis; when every channel has one row
// (`exclusive`) the accumulation is a plain read-modify-write.
template <int DT, int KN, bool SAT, typename Op>
__global__ __launch_bounds__(256) void sq_err_rows_kernel(const void* __restrict__ x,
                                                          int64_t nrows, int64_t inner_chunks,
                                                          int64_t axis, int exclusive,
                                                          const float* __restrict__ cand, int K,
                                                          Op op, float* __restrict__ loss) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int64_t waves = ((int64_t)gridDim.x * blockDim.x) >> 6;
    for (int64_t r = wave; r < nrows; r += waves) {
        const int64_t a = r % axis;
        typename Op::Scale s[KN];
        float part[KN];
#pragma unroll
        for (int k = 0; k < KN; ++k) {
            part[k] = 0.0f;
            s[k] = op.make(cand[(int64_t)(k < K ? k : 0) * axis + a]);
        }
        const int64_t base = r * inner_chunks;
        for (int64_t c = lane; c < inner_chunks; c += 128) {
            RawChunk<DT> raw[2];
            zero_raw<DT>(raw[1]);
            load_raw<DT>(x, (base + c) << 3, raw[0]);
            const bool second = c + 64 < inner_chunks;
            if (second) load_raw<DT>(x, (base + c + 64) << 3, raw[1]);
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                if (u == 1 && !second) continue;
                float v[8];
                unpack_raw<DT>(raw[u], v);
#pragma unroll
                for (int k = 0; k < KN; ++k) {
                    if (k < K) {
                        float acc = 0.0f;
                        if (Op::is_fast(s[k])) {
#pragma unroll
                            for (int j = 0; j < 8; ++j) {
                                const float d = v[j] - op.template apply_fast<SAT>(v[j], s[k]);
                                acc += d * d;
                            }
                        } else {
#pragma unroll
                            for (int j = 0; j < 8; ++j) {
                                const float d = v[j] - op.template apply<SAT>(v[j], s[k]);
                                acc += d * d;
                            }
                        }
                        part[k] += acc;
                    }
                }
            }
        }
#pragma unroll
        for (int k = 0; k < KN; ++k) {
            if (k < K) {
                const float t = wave_sum_f32(part[k]);
                if (lane == 0) {
                    float* dst = loss + (int64_t)k * axis + a;
                    if (exclusive) *dst += t;
                    else atomicAdd(dst, t);
                }
            }
        }
    }
}

template <int DT, int KN, bool SAT, typename Op>
static void launch_sq_err(const void* x, int64_t outer, int64_t axis, int64_t inner,
                          const float* cand, int K, Op op, float* loss, hipStream_t s) {
    const int64_t n = outer * axis * inner;
    if (axis == 1) {
        int64_t g = ((n >> 3) + 511) / 512;
        if (g < 1) g = 1;
        if (g > 2048) g = 2048;
        sq_err_tensor_kernel<DT, KN, SAT, Op><<<(unsigned)g, 256, 0, s>>>(x, n, cand, K, op, loss);
    } else {
        const int64_t nrows = outer * axis;
        int64_t g = (nrows + 3) / 4;
        if (g > 16384) g = 16384;
        sq_err_rows_kernel<DT, KN, SAT, Op><<<(unsigned)g, 256, 0, s>>>(x, nrows, inner >> 3, axis,
                                                                        outer == 1 ? 1 : 0, cand, K,
                                                                        op, loss);
    }
}

template <int DT, bool SAT, typename Op>
static void launch_sq_err_k(const void* x, int64_t outer, int64_t axis, int64_t inner,
                            const float* cand, int K, Op op, float* loss, hipStream_t s) {
    if (K <= 4) launch_sq_err<DT, 4, SAT, Op>(x, outer, axis, inner, cand, K, op, loss, s);
    else if (K <= 8) launch_sq_err<DT, 8, SAT, Op>(x, outer, axis, inner, cand, K, op, loss, s);
    else launch_sq_err<DT, 16, SAT, Op>(x, outer, axis, inner, cand, K, op, loss, s);
}

}  // namespace mo

extern "C" int mo_qdq_sq_err(const void* x, int64_t outer, int64_t axis, int64_t inner, int dtype,
                             const float* cand, int n_cand, int kind, int num_bits,
                             int is_unsigned, int narrow_range, int saturate, float* loss,
                             void* stream) {
    if (outer < 0 || axis < 0 || inner < 0 || n_cand < 0) return MO_ERR_ARG;
    if (kind != 0 && kind != 1) return MO_ERR_UNSUPPORTED;
    if (kind == 0 && (num_bits < 1 || num_bits > 24)) return MO_ERR_ARG;
    if (outer == 0 || axis == 0 || inner == 0 || n_cand == 0) return MO_OK;
    if (!x || !cand || !loss) return MO_ERR_ARG;
    if ((uintptr_t)x & 15u) return MO_ERR_UNSUPPORTED;
    if (axis > 1 && inner % 8 != 0) return MO_ERR_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
    mo::IntOp iop;
    iop.bound = (float)((1 << (num_bits - 1 + (is_unsigned ? 1 : 0))) - 1);
    iop.lo = is_unsigned ? 0.0f : (narrow_range ? -iop.bound : -iop.bound - 1.0f);
    // candidates in groups of at most 16 (the register budget of one launch)
    for (int k0 = 0; k0 < n_cand; k0 += 16) {
        const int K = n_cand - k0 < 16 ? n_cand - k0 : 16;
        const float* c = cand + (int64_t)k0 * axis;
        float* l = loss + (int64_t)k0 * axis;
#define CALL(DT)                                                                                   \
    if (kind == 0) mo::launch_sq_err_k<DT, false>(x, outer, axis, inner, c, K, iop, l, s);         \
    else if (saturate) mo::launch_sq_err_k<DT, true>(x, outer, axis, inner, c, K, mo::Fp8Op<true>(), l, s); \
    else mo::launch_sq_err_k<DT, false>(x, outer, axis, inner, c, K, mo::Fp8Op<true>(), l, s)
        switch (dtype) {
            case MO_F32: CALL(MO_F32); break;
            case MO_F16: CALL(MO_F16); break;
            case MO_BF16: CALL(MO_BF16); break;
            default: return MO_ERR_DTYPE;
        }
#undef CALL
    }
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}
