// Device helpers shared by the AWQ kernels (the per-alpha fused weight kernel and the one-launch
// search kernel must quantise a weight block with the same arithmetic in the same order).
#pragma once

#include "common.h"

namespace mo {

// One lane's chunk of a block: abs-max shared over the 1 << lg_g lanes of the block (every lane
// of the group must call this), then quantise-dequantise in place (fp32 values, not yet rounded
// to the storage dtype).
__device__ __forceinline__ void block_int_qdq_chunk(float (&v)[8], int lg_g, float bound, float lo) {
    uint32_t m = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t a = f2u(v[j]) & 0x7FFFFFFFu;
        m = a > m ? a : m;
    }
    m = group_max_u32(m, lg_g);
    const float amax = u2f(m);
    const bool dead = amax <= 5.9604644775390625e-8f;
    const float sc = bound / amax;
    const float mul = dead ? 0.0f : sc, div = dead ? 1.0f : sc;
    const float rdiv = 1.0f / div;
    const bool fast = mid_range(div);
    if (fast && lo < 0.0f) {
        // mid-range scale: the block holds no NaN or inf (either would be its abs-max), so the
        // clamp is a plain median (signed grids only: with lo = +0 the median of (-0, +0, bound)
        // need not keep the -0 that the comparison keeps) and the quotient the exact
        // reciprocal-and-FMA one
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float q = __builtin_amdgcn_fmed3f(__builtin_rintf(v[j] * mul), lo, bound);
            v[j] = __builtin_copysignf(exact_quotient(q, div, rdiv), q);
        }
    } else if (fast) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            float q = __builtin_rintf(v[j] * mul);
            q = q < lo ? lo : q;
            q = q > bound ? bound : q;
            v[j] = __builtin_copysignf(exact_quotient(q, div, rdiv), q);
        }
    } else {
        keep_branch();
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            float q = __builtin_rintf(v[j] * mul);
            q = q < lo ? lo : q;            // the way torch.clamp does: NaN stays NaN
            q = q > bound ? bound : q;
            v[j] = q / div;
        }
    }
}

}  // namespace mo
