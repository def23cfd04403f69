// AWQ-lite scale search for gfx950: for every alpha of the grid, the loss of the layer output
// with a scaled, INT-N block quantised weight, in one launch.
//
//   loss[a] += sum over (t, n) of f32( bf16( bf16(sum_k xs[a, t, k] * q_a[n, k]) - ref[t, n] ) )^2
//   q_a = block INT-N quantise-dequantise (blocks of bs along k) of bf16(w * s[a])
//
// This is the per-alpha body of the reference's search forward (weight pre-quant scale ->
// dynamic block amax -> fake quant -> linear -> squared error against the unquantised output,
// TQ/model_calib.py:645-690) with the activations already multiplied by 1 / s[a].
//
// A workgroup of 8 wavefronts owns a column tile of 128 (or 96) output features for one alpha and
// all T <= 512 tokens, so every weight element is scaled and quantised exactly once per alpha.  Every
// wavefront does both jobs: it multiplies its 64 (or 32) token rows with the quantised tile of
// the current k block (B operand of v_mfma_f32_32x32x16_bf16 from LDS, A operand straight from a
// chunk-major copy of the activations, in which the lanes of an operand read adjacent memory)
// and, between those matrix instructions, quantises its share of the tile of the next k block
// into the other LDS buffer.  Two wavefronts share a SIMD, so one's vector work and LDS waits
// run under the other's matrix instructions; an activation fragment is used for all 128
// columns, which halves the traffic of the A operand through L2 against a 64-column tile (a
// wider tile does not fit the registers: 512 tokens x 256 columns of fp32 is the whole register
// file of a compute unit).  The 32 compute units that share an L2 each pull the whole activation
// matrix of their alpha through it once per column tile (4 MB per tile, 16 KB per step of 16 k):
// 11 - 12 TB/s over the chip, a third of what a load-only kernel draws through the same path, so
// it is the latency of the loads, not their bytes, that the loop has to hide.  Three things do
// that, each measured: the loads of a step stay in that step (a scheduling barrier per step; the
// compiler otherwise gathers them and drains the in-order load counter mid-block), the raw
// weights of the tile after the next are asked for seven steps ahead, as soon as their
// registers fall free, and they are plain loads so that the next alpha finds them in the
// last-level cache.  The output tile never leaves the registers: it is rounded to bf16, compared
// with the reference output and reduced to one double per workgroup.
//
// The integer codes follow the reference's arithmetic (bound / amax, one IEEE multiply, round
// half to even) with bound / amax from the hardware reciprocal and one FMA correction step,
// which is the correctly rounded quotient except for quotients that lie within about 2^-40 of
// the midpoint of two floats; the dequantised value is code * (amax / bound) instead of the
// reference's division by bound / amax: the fp32 results differ by at most an ulp, which
// survives the rounding to bf16 for about one weight in 10^4, far below the 1e-3 tolerance of
// the per-alpha losses.  The weights that are kept after the search come from the
// exact kernels.
#include <atomic>
#include <mutex>
#include <type_traits>

#include "awq_ops.h"
#include "common.h"

namespace mo {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int kSearchTileN = 128;   // output features per workgroup
constexpr int kSearchBlockK = 128;  // k elements per step of the outer loop: 16 chunks of 8
constexpr int kSearchWaves = 8;
constexpr int kXcds = 8;            // accelerator dies of the chip, each with its own L2

// One column tile of 32 * NG output features (NG = 4 or 3) for alpha `a`, starting at feature n0.
// RB = 32-row blocks per wavefront; the workgroup covers 8 * 32 * RB token rows.
template <int RB, int NG, bool BIAS>
__device__ __forceinline__ void awq_search_tile(
    const uint16_t* __restrict__ xs,   // [A][K / 8][T][8] bf16, activations * (1 / s[a])
    const uint16_t* __restrict__ w,    // [N, K] bf16
    const uint16_t* __restrict__ s,    // [A, K] bf16
    const uint16_t* __restrict__ ref,  // [T, N] bf16
    const uint16_t* __restrict__ bias, // [N] bf16, read when BIAS: added to the fp32 sums before rounding
    int T, int N, int K, int a, int n0, int lg_g, float bound, double* __restrict__ loss,
    u32x4 (&tile)[2][kSearchTileN][16], double (&red)[kSearchWaves]) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nkb = K / kSearchBlockK;

    // ---- producer side: chunk qc of rows qr + 32 u of the tile (u = 0..3), two chunks at a time.
    // Addresses are a wave-uniform base plus a 32-bit byte offset per lane (128 rows of K bf16
    // stay below 4 GiB: K < 2^24 is checked by the launcher), so advancing along k costs no
    // vector instruction.
    const int qc = threadIdx.x & 15, qr = threadIdx.x >> 4;
    const char* wtile = (const char*)(w + (int64_t)n0 * K);
    uint32_t woff = ((uint32_t)qr * (uint32_t)K + (uint32_t)qc * 8u) * 2u;
    const uint32_t wstride = 32u * (uint32_t)K * 2u;  // between the rows of two of a lane's chunks
    const char* srow = (const char*)(s + (int64_t)a * K);
    uint32_t soff = (uint32_t)qc * 16u;
    u32x4 wraw[NG], sraw;   // raw weight chunks and scales of the block to quantise next
    float sf[8];            // the scales of the block being quantised
    uint32_t vp[2][4];      // the pair of chunks being quantised: bf16(w * s), packed
    float mul[2], rdiv[2];  // per chunk: bound / amax and amax / bound

    // Raw weights and scales of k block kb, in two halves: row groups 2 h and 2 h + 1 and, with
    // the first half, the scales.  Plain loads, not streaming ones: the next alpha reads the
    // same weights again, and with the streaming hint they come from HBM every time instead
    // of from the last-level cache (7 % of the launch, measured).  The asm statement emits
    // nothing; it keeps the zero extension of the lane offset inside the loop body, where
    // instruction selection folds it into the load's (scalar base, 32-bit lane offset) form
    // instead of a 64-bit vector add per load.
    auto fetch_half = [&](int kb, int h) {
        const uint32_t k0 = (uint32_t)(kb < nkb ? kb : nkb - 1) * (kSearchBlockK * 2);
        asm volatile("" : "+v"(woff), "+v"(soff));
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int u = 2 * h + i;
            if (u >= NG) continue;   // a tile of 96 features has three row groups
            wraw[u] = *(const u32x4*)(wtile + k0 + u * wstride + woff);
        }
        if (h == 0) sraw = *(const u32x4*)(srow + k0 + soff);
    };
    auto scale_pair = [&](int h) {  // chunks 2 h, 2 h + 1: bf16(w * s), two values a word
        if (h == 0) {
            const uint32_t sw[4] = {sraw.x, sraw.y, sraw.z, sraw.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                sf[2 * j] = u2f(sw[j] << 16);
                sf[2 * j + 1] = u2f(sw[j] & 0xFFFF0000u);
            }
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            if (2 * h + i >= NG) continue;   // a tile of 96 features has three row groups
            const u32x4 r = wraw[2 * h + i];
            const uint32_t ww[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
            for (int j = 0; j < 4; ++j)
                vp[i][j] = f32x2_to_bf16x2(u2f(ww[j] << 16) * sf[2 * j],
                                           u2f(ww[j] & 0xFFFF0000u) * sf[2 * j + 1]);
        }
    };
    const float inv_bound = 1.0f / bound;
    auto block_scales = [&](int h) {  // block abs-max over the lanes of a block, then the two factors
        typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            if (2 * h + i >= NG) continue;
            // |bf16| bit patterns order like the magnitudes: 16-bit integer maxima, two a word
            u16x2 m2 = {0, 0};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t t = vp[i][j] & 0x7FFF7FFFu;
                u16x2 t2;
                __builtin_memcpy(&t2, &t, 4);
                m2 = __builtin_elementwise_max(m2, t2);
            }
            uint32_t m = (uint32_t)(m2.x > m2.y ? m2.x : m2.y) << 16;   // as fp32 bits
            // abs-max over the 1 << lg_g (4, 8 or 16) lanes of a block; selects instead of
            // branches keep the loop body one basic block
#define MO_DPP_STEP(CTRL, ON)                                                                 \
    {                                                                                         \
        const uint32_t t = (uint32_t)__builtin_amdgcn_mov_dpp((int)m, CTRL, 0xF, 0xF, true);  \
        m = ((ON) && t > m) ? t : m;                                                          \
    }
            MO_DPP_STEP(0xB1, true)        // quad_perm [1, 0, 3, 2]
            MO_DPP_STEP(0x4E, true)        // quad_perm [2, 3, 0, 1]
            MO_DPP_STEP(0x141, lg_g >= 3)  // row_half_mirror
            MO_DPP_STEP(0x140, lg_g >= 4)  // row_mirror
#undef MO_DPP_STEP
            const float amax = u2f(m);
            const bool dead = amax <= 5.9604644775390625e-8f;  // 2^-24
            // bound / amax: hardware reciprocal and one FMA correction step, without the
            // branches of the full division sequence
            const float r = __builtin_amdgcn_rcpf(amax);
            const float q0 = bound * r;
            const float q1 = __builtin_fmaf(__builtin_fmaf(-q0, amax, bound), r, q0);
            mul[i] = dead ? 0.0f : q1;
            rdiv[i] = dead ? 1.0f : amax * inv_bound;
        }
    };
    // |v| <= amax, so the rounded code never leaves [-bound, bound]: no clamp is needed
    auto quantise_store = [&](int h, int i, int buf) {
        if (2 * h + i >= NG) return;
        float y[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            y[2 * j] = __builtin_rintf(u2f(vp[i][j] << 16) * mul[i]) * rdiv[i];
            y[2 * j + 1] = __builtin_rintf(u2f(vp[i][j] & 0xFFFF0000u) * mul[i]) * rdiv[i];
        }
        u32x4 o;
        o.x = f32x2_to_bf16x2(y[0], y[1]);
        o.y = f32x2_to_bf16x2(y[2], y[3]);
        o.z = f32x2_to_bf16x2(y[4], y[5]);
        o.w = f32x2_to_bf16x2(y[6], y[7]);
        const int r = qr + 32 * (2 * h + i);
        tile[buf][r][qc ^ (r & 15)] = o;
    };
    // the work on one tile in eight slices (one per step of the matrix loop)
    auto produce_slice = [&](int j, int kb_next, int buf) {
        const int h = j >> 2;
        switch (j & 3) {
            // a half's raw registers are free once scale_pair(h) has read them: the data of
            // the block after the next is asked for right then, seven steps before its use
            case 0: scale_pair(h); break;
            case 1: block_scales(h); fetch_half(kb_next + 1, h); break;
            case 2: quantise_store(h, 0, buf); break;
            default: quantise_store(h, 1, buf); break;
        }
    };

    // ---- consumer side.  v_mfma_f32_32x32x16_bf16: lane (fr, kg) = (lane & 31, lane >> 5)
    // supplies row fr of the A block and column fr of the B block, elements [8 kg, 8 kg + 8) of
    // the 16 k of a step, and receives rows 8 (i / 4) + 4 kg + i % 4 (i = 0..15) of column fr.
    const int fr = lane & 31, kg = lane >> 5;
    const int row_base = wave * (RB * 32);
    const bool has_rows = row_base < T;  // wavefronts past T only produce
    const uint16_t* xa = xs + (int64_t)a * T * K;
    f32x16_t acc[RB][NG];
#pragma unroll
    for (int mb = 0; mb < RB; ++mb)
#pragma unroll
        for (int nb = 0; nb < NG; ++nb)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0.0f;
    // Element offsets of this lane's A fragments.  xs is chunk-major: [K / 8][T][8], i.e. the 16
    // bytes of chunk c of row t sit at ((c * T) + t) * 8, so the 32 lanes fr of a k-group read
    // 512 contiguous bytes.  Rows past T repeat row T - 1 (masked in the epilogue); T * K < 2^31
    // is checked by the launcher.
    uint32_t aoff[RB];  // in bytes, added to a wave-uniform address of the step
#pragma unroll
    for (int mb = 0; mb < RB; ++mb) {
        int t = row_base + mb * 32 + fr;
        t = t < T ? t : T - 1;
        aoff[mb] = ((uint32_t)kg * (uint32_t)T + (uint32_t)t) * 16u;
    }
    const uint32_t step_stride = 2u * (uint32_t)T * 16u;  // one step of 16 k = 2 chunks, in bytes
    const char* xab = (const char*)xa;
    const int steps = nkb * 8;
    // activation fragments are fetched this many steps ahead (a divisor of the 8 steps of a k
    // block, so that a step's register slot j % PF is the same in every block).  Four steps and
    // the one-at-a-time B fragments below measured 5 - 6 % faster than two steps with all four B
    // fragments of a step loaded up front; eight steps are slower again (255 registers, no room
    // left for the scheduler).
    constexpr int PF = 4;
    static_assert(8 % PF == 0, "slot of a step must not depend on the k block");
    u32x4 af[RB][PF];

    // ---- prologue: tile 0 into buffer 0, raw weights of block 1 fetched on the way.  Those
    // must have landed before the loop is entered and the activation prefetch must be issued
    // after them (the empty asm statements and the scheduling barriers see to both): the
    // compiler's wait counts inside the loop are the more cautious of "entered from here" and
    // "came round from the last step", and with the weights still in flight behind the
    // activations at the entry every k block would begin by draining all of its loads.
    fetch_half(0, 0);
    fetch_half(0, 1);
#pragma unroll
    for (int j = 0; j < 8; ++j) produce_slice(j, 0, 0);
#pragma unroll
    for (int u = 0; u < NG; ++u) asm volatile("" ::"v"(wraw[u]));
    asm volatile("" ::"v"(sraw));
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < PF; ++j)
#pragma unroll
        for (int mb = 0; mb < RB; ++mb)
            af[mb][j] = *(const u32x4*)(xab + (uint32_t)j * step_stride + aoff[mb]);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();

    // One k block: 8 steps of 16 k against the tile in buffer kb & 1; with MORE, one eighth of
    // the work on the next tile (into the other buffer) follows each step's matrix instructions.
    // No branches inside, so the whole block is scheduled as one: wavefronts whose rows lie past
    // T multiply their clamped rows as well and are left out of the sum.
    auto k_block = [&](int kb, auto more_tag) {
        constexpr bool MORE = decltype(more_tag)::value;
        const int buf = kb & 1;
        u32x4 bfirst;   // the first B fragment of the next step, read under this step's tail
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int c = j * 2 + kg;
            // B fragments one at a time, the next one's LDS read issued ahead of the current
            // one's matrix instructions: 8 registers of fragments live instead of 16, which is
            // what lets the activation prefetch above reach four steps without spilling
            bf16x8_t afrag[RB];
#pragma unroll
            for (int mb = 0; mb < RB; ++mb) __builtin_memcpy(&afrag[mb], &af[mb][j % PF], 16);
            u32x4 bnext = j == 0 ? tile[buf][fr][c ^ (fr & 15)] : bfirst;
#pragma unroll
            for (int nb = 0; nb < NG; ++nb) {
                bf16x8_t bcur;
                __builtin_memcpy(&bcur, &bnext, 16);
                if (nb + 1 < NG) {
                    const int r = (nb + 1) * 32 + fr;
                    bnext = tile[buf][r][c ^ (r & 15)];
                }
#pragma unroll
                for (int mb = 0; mb < RB; ++mb)
                    acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(afrag[mb], bcur,
                                                                          acc[mb][nb], 0, 0, 0);
            }
            int g = kb * 8 + j + PF;
            g = g < steps ? g : steps - 1;
            const char* xstep = xab + (uint32_t)g * step_stride;   // wave-uniform
#pragma unroll
            for (int mb = 0; mb < RB; ++mb) {
                asm volatile("" : "+v"(aoff[mb]));   // scalar base + lane offset form, as in fetch_half
                af[mb][j % PF] = *(const u32x4*)(xstep + aoff[mb]);
            }
            if constexpr (MORE) produce_slice(j, kb + 1, buf ^ 1);
            if (j < 7) bfirst = tile[buf][fr][(c + 2) ^ (fr & 15)];
            // Nothing moves across a step's end.  Left alone, the scheduler gathers the loads of
            // several steps in one place, and the in-order load counter then has to be waited
            // down to zero in the middle of the block.
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
    };
    for (int kb = 0; kb + 1 < nkb; ++kb) k_block(kb, std::true_type{});
    k_block(nkb - 1, std::false_type{});

    // ---- epilogue: bf16(out) - ref in bf16, squared in fp32 (rows past T read row T - 1 and are
    // masked out of the sum)
    float part = 0.0f;
    if (has_rows) {
        // the column's bias is fetched here, behind a statement the compiler may not move work
        // across: computed any earlier its address would sit in registers through the k loop
        int col = n0 + fr;
        if constexpr (BIAS) asm volatile("" : "+v"(col));
#pragma unroll
        for (int mb = 0; mb < RB; ++mb)
#pragma unroll
            for (int nb = 0; nb < NG; ++nb) {
                const uint16_t* rcol = ref + n0 + nb * 32 + fr;
                float add = 0.0f;
                if constexpr (BIAS) add = bf16_bits_to_f32(bias[col + nb * 32]);
                uint16_t rv[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    int t = row_base + mb * 32 + 8 * (i / 4) + 4 * kg + (i % 4);
                    t = t < T ? t : T - 1;
                    rv[i] = rcol[(int64_t)t * N];
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int t = row_base + mb * 32 + 8 * (i / 4) + 4 * kg + (i % 4);
                    const float o = round_to_bf16(BIAS ? acc[mb][nb][i] + add : acc[mb][nb][i]);
                    const float d = round_to_bf16(o - bf16_bits_to_f32(rv[i]));
                    part += t < T ? d * d : 0.0f;
                }
            }
    }
    double sum = (double)part;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, kWave);
    if (lane == 0) red[wave] = sum;
    __syncthreads();
    if (threadIdx.x == 0) {
        double total = 0.0;
#pragma unroll
        for (int i = 0; i < kSearchWaves; ++i) total += red[i];
        atomicAdd(loss + a, total);
    }
}

// Every alpha's n columns are cut into `wide` tiles of 128 features followed by `narrow` tiles of
// 96 (128 wide + 96 narrow = n).  A launch whose 128-wide tiles do not fill the chip's last round
// (21 alphas x 32 tiles = 672 workgroups on 256 compute units that hold one each: 2.6 rounds)
// trades some wide tiles for narrow ones, so that a unit's last tile is a short one.
//
// Workgroup L of a launch runs on XCD L % 8, and each XCD has its own L2.  All column tiles of
// an alpha read the same activations, so tiles are dealt out in contiguous runs in alpha-major
// order: XCD x takes wide tiles [x * per_wide, (x + 1) * per_wide) first and then narrow tiles
// [x * per_narrow, (x + 1) * per_narrow) -- both runs cover about the same alphas, the column
// tiles of one alpha run side by side on one XCD, and the 4 MB of activations they walk through
// in step are fetched into that L2 once instead of once per XCD.  The grid is
// 8 * (per_wide + per_narrow) workgroups; surplus ones leave at once.
template <int RB, bool BIAS>
__global__ __launch_bounds__(512) void awq_search_kernel(
    const uint16_t* __restrict__ xs, const uint16_t* __restrict__ w, const uint16_t* __restrict__ s,
    const uint16_t* __restrict__ ref, const uint16_t* __restrict__ bias, int T, int N, int K,
    int n_alpha, int wide, int narrow,
    int per_wide, int per_narrow, int lg_g, float bound, double* __restrict__ loss) {
    // quantised weight tile, two buffers: [128 rows][16 chunk slots] of 16 bytes; the slot of
    // chunk c in row r is c ^ (r & 15) so that both the writers (16 lanes per row) and the
    // readers (lanes along rows) spread over all banks
    __shared__ u32x4 tile[2][kSearchTileN][16];
    __shared__ double red[kSearchWaves];
    const int xcd = blockIdx.x % kXcds, slot = blockIdx.x / kXcds;
    if (slot < per_wide) {
        const int i = xcd * per_wide + slot;
        if (i >= n_alpha * wide) return;
        awq_search_tile<RB, 4, BIAS>(xs, w, s, ref, bias, T, N, K, i / wide, (i % wide) * 128, lg_g, bound,
                               loss, tile, red);
    } else {
        const int i = xcd * per_narrow + (slot - per_wide);
        if (i >= n_alpha * narrow) return;
        awq_search_tile<RB, 3, BIAS>(xs, w, s, ref, bias, T, N, K, i / narrow, wide * 128 + (i % narrow) * 96,
                               lg_g, bound, loss, tile, red);
    }
}

// How many 96-wide tiles per alpha (a multiple of 4: four of them replace three 128-wide ones)
// make the launch end soonest: tiles are handed to the compute units of an XCD in launch order
// as units fall free, a tile costs its width plus a fixed part (prologue and epilogue, about 10
// columns' worth), and the launch ends when the slowest XCD does.
static inline int narrow_tiles_per_alpha_uncached(int64_t n_alpha, int64_t n, int units_per_xcd) {
    int best = 0;
    double best_end = 0.0;
    double free_at[64];
    if (units_per_xcd < 1) units_per_xcd = 1;
    if (units_per_xcd > 64) units_per_xcd = 64;
    for (int narrow = 0; narrow * 96ll <= n; narrow += 4) {
        const int64_t wide = (n - narrow * 96ll) / 128;
        const int64_t per_wide = (n_alpha * wide + kXcds - 1) / kXcds;
        const int64_t per_narrow = (n_alpha * narrow + kXcds - 1) / kXcds;
        for (int u = 0; u < units_per_xcd; ++u) free_at[u] = 0.0;
        double end = 0.0;
        for (int64_t t = 0; t < per_wide + per_narrow; ++t) {   // the fullest XCD
            int first = 0;
            for (int u = 1; u < units_per_xcd; ++u)
                if (free_at[u] < free_at[first]) first = u;
            free_at[first] += (t < per_wide ? 128.0 : 96.0) + 10.0;
            if (free_at[first] > end) end = free_at[first];
        }
        // narrower tiles re-read the activations more often: they must pay for themselves
        if (narrow == 0 || end < best_end * 0.97) {
            best = narrow;
            best_end = end;
        }
        if (narrow >= 64) break;
    }
    return best;
}

// The answer for the last few (alphas, features, units) asked about: a search step of every layer
// of a model asks the same handful of questions, and the simulation costs as much host time as
// the kernel it plans takes on the device.
static inline int narrow_tiles_per_alpha(int64_t n_alpha, int64_t n, int units_per_xcd) {
    struct Entry { int64_t n_alpha, n; int units, narrow; };
    static std::mutex lock;
    static Entry memo[16];
    static int used = 0, next = 0;
    {
        std::lock_guard<std::mutex> hold(lock);
        for (int i = 0; i < used; ++i)
            if (memo[i].n_alpha == n_alpha && memo[i].n == n && memo[i].units == units_per_xcd)
                return memo[i].narrow;
    }
    const int narrow = narrow_tiles_per_alpha_uncached(n_alpha, n, units_per_xcd);
    std::lock_guard<std::mutex> hold(lock);
    memo[next] = Entry{n_alpha, n, units_per_xcd, narrow};
    next = (next + 1) % 16;
    if (used < 16) ++used;
    return narrow;
}

// xs[a][c][t][0..8) = bf16(x[t][8 c ..] * inv_s[a][8 c ..]) for every alpha: the activations the
// search kernel multiplies, in its chunk-major layout.  A wavefront owns one chunk column c and
// 64 consecutive tokens (its scales are wave-uniform, its stores contiguous: 1 KiB per alpha).
__global__ __launch_bounds__(256) void awq_scale_activations_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ inv_s, int A, int T, int K,
    uint16_t* __restrict__ xs) {
    const int lane = threadIdx.x & 63;
    const int c = blockIdx.y * 4 + (threadIdx.x >> 6);  // chunk column
    const int t = blockIdx.x * 64 + lane;
    const int kc = K >> 3;
    if (c >= kc || t >= T) return;
    const u32x4 raw = *(const u32x4*)(x + (int64_t)t * K + c * 8);
    const uint32_t xw[4] = {raw.x, raw.y, raw.z, raw.w};
    float v[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        v[2 * j] = u2f(xw[j] << 16);
        v[2 * j + 1] = u2f(xw[j] & 0xFFFF0000u);
    }
    for (int a = 0; a < A; ++a) {
        const u32x4 sr = *(const u32x4*)(inv_s + (int64_t)a * K + c * 8);
        const uint32_t sw[4] = {sr.x, sr.y, sr.z, sr.w};
        u32x4 o;
        o.x = f32x2_to_bf16x2(v[0] * u2f(sw[0] << 16), v[1] * u2f(sw[0] & 0xFFFF0000u));
        o.y = f32x2_to_bf16x2(v[2] * u2f(sw[1] << 16), v[3] * u2f(sw[1] & 0xFFFF0000u));
        o.z = f32x2_to_bf16x2(v[4] * u2f(sw[2] << 16), v[5] * u2f(sw[2] & 0xFFFF0000u));
        o.w = f32x2_to_bf16x2(v[6] * u2f(sw[3] << 16), v[7] * u2f(sw[3] & 0xFFFF0000u));
        *(u32x4*)(xs + (((int64_t)a * kc + c) * T + t) * 8) = o;
    }
}

}  // namespace mo

extern "C" int mo_awq_search_losses(const void* xs, const void* w, const void* s, const void* ref,
                                    int64_t n_alpha, int64_t tokens, int64_t n, int64_t k,
                                    int dtype, int64_t block_size, int num_bits, int is_unsigned,
                                    int narrow_range, double* loss, void* stream) {
    return mo_awq_search_losses_biased(xs, w, s, ref, nullptr, n_alpha, tokens, n, k, dtype, block_size,
                                       num_bits, is_unsigned, narrow_range, loss, stream);
}

extern "C" int mo_awq_search_losses_biased(const void* xs, const void* w, const void* s, const void* ref,
                                           const void* bias, int64_t n_alpha, int64_t tokens, int64_t n,
                                           int64_t k, int dtype, int64_t block_size, int num_bits,
                                           int is_unsigned, int narrow_range, double* loss, void* stream) {
    if (n_alpha < 0 || tokens < 0 || n < 0 || k < 0 || num_bits < 2 || num_bits > 16) return MO_ERR_ARG;
    if (dtype != MO_BF16) return MO_ERR_UNSUPPORTED;
    if (n_alpha == 0 || tokens == 0 || n == 0 || k == 0) return MO_OK;
    if (!xs || !w || !s || !ref || !loss) return MO_ERR_ARG;
    int lg_g = -1;
    if (block_size == 32) lg_g = 2;
    else if (block_size == 64) lg_g = 3;
    else if (block_size == 128) lg_g = 4;
    if (lg_g < 0 || tokens > 512 || n % mo::kSearchTileN || k % mo::kSearchBlockK ||
        n_alpha > 65535 || n > 0x7FFFFFFF || tokens * k > 0x7FFFFFFF || k >= (1 << 24) ||
        (n_alpha + 8) * (n / mo::kSearchTileN) > 0x7FFFFFFF)
        return MO_ERR_UNSUPPORTED;
    if ((((uintptr_t)xs | (uintptr_t)w | (uintptr_t)s) & 15u) || (((uintptr_t)ref | (uintptr_t)bias) & 1u))
        return MO_ERR_UNSUPPORTED;
    const float bound = (float)((1 << (num_bits - 1 + (is_unsigned ? 1 : 0))) - 1);
    // signed grids only: the kernel relies on |w * s| <= block amax keeping every code inside
    // [-bound, bound] (so narrow_range makes no difference); an unsigned grid would have to clamp
    // negative weights to 0
    if (is_unsigned) return MO_ERR_UNSUPPORTED;
    (void)narrow_range;
    hipStream_t st = (hipStream_t)stream;
    // compute units that share an L2 (one workgroup each), per device
    static std::atomic<int> units_of_device[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return MO_ERR_LAUNCH;
    int units_per_xcd = units_of_device[dev].load(std::memory_order_relaxed);
    if (units_per_xcd == 0) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < mo::kXcds)
            cus = 256;
        units_per_xcd = cus / mo::kXcds;
        units_of_device[dev].store(units_per_xcd, std::memory_order_relaxed);
    }
    int narrow = (int)mo::tuned("search_narrow_tiles", -1);
    if (narrow < 0) narrow = mo::narrow_tiles_per_alpha(n_alpha, n, units_per_xcd);
    if (narrow % 4 || narrow * 96ll > n) return MO_ERR_ARG;
    const int64_t wide = (n - narrow * 96ll) / 128;
    const int64_t per_wide = (n_alpha * wide + mo::kXcds - 1) / mo::kXcds;
    const int64_t per_narrow = (n_alpha * narrow + mo::kXcds - 1) / mo::kXcds;
    const dim3 grid((unsigned)((per_wide + per_narrow) * mo::kXcds));
#define CALL(RB, BIAS)                                                                     \
    mo::awq_search_kernel<RB, BIAS><<<grid, 512, 0, st>>>(                                 \
        (const uint16_t*)xs, (const uint16_t*)w, (const uint16_t*)s, (const uint16_t*)ref, \
        (const uint16_t*)bias, (int)tokens, (int)n, (int)k, (int)n_alpha, (int)wide, narrow, \
        (int)per_wide, (int)per_narrow, lg_g, bound, loss)
    if (tokens <= 256) {
        if (bias) CALL(1, true);
        else CALL(1, false);
    } else {
        if (bias) CALL(2, true);
        else CALL(2, false);
    }
#undef CALL
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_awq_scale_activations(const void* x, const void* inv_s, int64_t n_alpha,
                                        int64_t tokens, int64_t k, int dtype, void* xs,
                                        void* stream) {
    if (n_alpha < 0 || tokens < 0 || k < 0) return MO_ERR_ARG;
    if (dtype != MO_BF16 || k % 8) return MO_ERR_UNSUPPORTED;
    if (n_alpha == 0 || tokens == 0 || k == 0) return MO_OK;
    if (!x || !inv_s || !xs) return MO_ERR_ARG;
    if ((((uintptr_t)x | (uintptr_t)inv_s | (uintptr_t)xs) & 15u)) return MO_ERR_UNSUPPORTED;
    const int64_t gx = (tokens + 63) / 64, gy = (k / 8 + 3) / 4;
    if (gx > 0x7FFFFFFF || gy > 65535 || tokens * k > 0x7FFFFFFF || n_alpha > 0x7FFFFFFF)
        return MO_ERR_UNSUPPORTED;
    mo::awq_scale_activations_kernel<<<dim3((unsigned)gx, (unsigned)gy), 256, 0, (hipStream_t)stream>>>(
        (const uint16_t*)x, (const uint16_t*)inv_s, (int)n_alpha, (int)tokens, (int)k, (uint16_t*)xs);
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}
