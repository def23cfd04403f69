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
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        float q = __builtin_rintf(v[j] * mul);
        q = q < lo ? lo : q;
        v[j] = q > bound ? bound : q;
    }
    if (fast) {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = __builtin_copysignf(exact_quotient(v[j], div, rdiv), v[j]);
    } else {
        keep_branch();
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = v[j] / div;
    }
}

}  // namespace mo
