// The two element-wise quantize-dequantize operators (FP8 E4M3 and N-bit integer) shared by the
// fake-quant kernels and the amax-search kernels.
#pragma once
#include "common.h"

namespace mo {

template <bool HAS_AMAX>
struct Fp8Op {
    static constexpr bool has_amax = HAS_AMAX;
    struct Scale { float mul, inv; };
    __device__ __forceinline__ Scale make(float amax) const {
        Scale s;
        // the reference writes `448.0 / amax`, which torch evaluates as reciprocal(amax) * 448
        // (two roundings), and `1 / scale`, which is reciprocal(scale)
        s.mul = (1.0f / amax) * 448.0f;
        s.inv = 1.0f / s.mul;
        return s;
    }
    template <bool SAT>
    __device__ __forceinline__ float apply(float x, const Scale& s) const {
        if (!has_amax) return round_e4m3<SAT>(x);
        return round_e4m3<SAT>(x * s.mul) * s.inv;
    }
    // every scale takes the same path
    static __device__ __forceinline__ bool is_fast(const Scale&) { return true; }
    template <bool SAT>
    __device__ __forceinline__ float apply_fast(float x, const Scale& s) const { return apply<SAT>(x, s); }
    template <bool SAT>
    __device__ __forceinline__ void apply2_fast(float& a, float& b, const Scale& sa, const Scale& sb) const {
        apply2<SAT>(a, b, sa, sb);
    }
    // two elements per conversion instruction
    template <bool SAT>
    __device__ __forceinline__ void apply2(float& a, float& b, const Scale& sa, const Scale& sb) const {
        if (!has_amax) { round_e4m3_pair<SAT>(a, b); return; }
        a *= sa.mul;
        b *= sb.mul;
        round_e4m3_pair<SAT>(a, b);
        a *= sa.inv;
        b *= sb.inv;
    }
};

struct IntOp {
    float bound, lo;
    // y = clamp(rne(x * mul), lo, bound) / div; when `fast`, the division is the exact
    // reciprocal-and-FMA quotient (|q| <= 2^24 and div in [2^-64, 2^64] cannot over/underflow)
    struct Scale { float mul, div, rdiv; bool fast; };
    __device__ __forceinline__ Scale make(float amax) const {
        Scale s;
        // the CPU path's rule (tensor_quant.py:574-612): amax <= 2^-24 zeroes the scale and divides
        // by 1, so a dead channel gives rint(x * 0) -- -0.0 for negative x, NaN for inf / NaN.
        // (The reference's CUDA kernel uses amax < 2^-24 and returns +0.0; parity here is with
        // the CPU path.)
        const bool dead = amax <= 5.9604644775390625e-8f;  // 2^-24
        const float sc = bound / amax;
        s.mul = dead ? 0.0f : sc;
        s.div = dead ? 1.0f : sc;
        s.rdiv = 1.0f / s.div;
        s.fast = mid_range(s.div);
        return s;
    }
    template <bool>
    __device__ __forceinline__ float apply(float x, const Scale& s) const {
        float q = __builtin_rintf(x * s.mul);  // round half to even
        // clamp the way torch.clamp does: NaN stays NaN
        q = q < lo ? lo : q;
        q = q > bound ? bound : q;
        if (s.fast) return __builtin_copysignf(exact_quotient(q, s.div, s.rdiv), q);
        keep_branch();
        return q / s.div;
    }
    template <bool F>
    __device__ __forceinline__ void apply2(float& a, float& b, const Scale& sa, const Scale& sb) const {
        a = apply<F>(a, sa);
        b = apply<F>(b, sb);
    }
    // for a caller that has checked is_fast() of every scale it holds once, outside its loop
    static __device__ __forceinline__ bool is_fast(const Scale& s) { return s.fast; }
    template <bool>
    __device__ __forceinline__ float apply_fast(float x, const Scale& s) const {
        float q = __builtin_rintf(x * s.mul);
        q = q < lo ? lo : q;
        q = q > bound ? bound : q;
        return __builtin_copysignf(exact_quotient(q, s.div, s.rdiv), q);
    }
    template <bool F>
    __device__ __forceinline__ void apply2_fast(float& a, float& b, const Scale& sa, const Scale& sb) const {
        a = apply_fast<F>(a, sa);
        b = apply_fast<F>(b, sb);
    }
};

}  // namespace mo
