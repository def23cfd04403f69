// AWQ clip search for gfx950: for every weight block and every clip ratio, the squared error the
// clipped, fake-quantised block makes on the block's partial outputs over the calibration
// tokens -- one launch per batch of tokens instead of (ratios x row batches) broadcast products.
//
// What is computed, in the dtype T of the weight (all as the tensor expression would round):
//   org[t]  = T( sum_j T(x[t, j] * w[j]) )                 j over the block, fp32 accumulation
//   cur[t]  = T( sum_j T(x[t, j] * wq_r[j]) )              wq_r = T(qdq(w; T(f32(amax) * r)))
//   loss[r] += ( sum_t f32(T(cur[t] - org[t]))^2 ) / tokens
//
// Work decomposition: a lane owns one (output row, block).  The block of the quantised weight
// stays in the lane's registers as fp32; the activations of a token are the same for every
// lane, so they are read through uniform (scalar) loads and cost the vector ALU nothing.  The
// org[] values of a lane live in LDS ([token][lane], conflict-free).  VALU-bound: each product
// is one multiply, one rounding to T and one add (bf16: two products share the rounding and the
// add, see token_dots).
//
// A weight with few (row, block) pairs does not fill the chip with one wavefront per 64 pairs
// (1024 x 4096 in blocks of 128 is 512 wavefronts for 1024 SIMDs, and a lone wavefront on a
// SIMD runs at two thirds of the rate three of them reach together), so a workgroup may hold
// 2 or 4 wavefronts that own the same 64 pairs and share the tokens of a pass between them;
// their partial sums meet in LDS and wavefront 0 adds them in wavefront order, so the result
// does not depend on timing.
#include "common.h"
#include "qdq_ops.h"

namespace mo {

constexpr int kClipMaxRatios = 32;
constexpr int kClipTokens = 64;   // tokens per wavefront and pass over the ratios (org[] in LDS)
constexpr int kClipLanes = 64;
constexpr int kClipMaxSplit = 4;  // wavefronts that may share the tokens of one (row, block) set

struct ClipRatios {
    float r[kClipMaxRatios];
    int count;
};

template <int DT>
__device__ __forceinline__ float clip_round(float v) {
    if constexpr (DT == MO_BF16) return round_to_bf16(v);
    else if constexpr (DT == MO_F16) return f16_bits_to_f32(f32_to_f16_bits(v));
    else return v;
}

// For each of `tc` tokens, T( sum_j T(x[t, j] * w[j]) ) -- products rounded to T one by one,
// summed in fp32 in index order -- handed to fn(t, value).
//
// x is uniform over the wavefront: it is read through scalar loads, 16 elements a group, and
// unpacking 16-bit pairs is scalar-ALU work.  The loads are software-pipelined one group ahead
// (across token boundaries too); scalar loads return out of order, so a wait covers every load
// in flight, hence the order "use the group that has arrived, then issue the next load, then
// do the vector work", which the scheduling barriers pin down.
template <int DT, int BS, typename Fn>
__device__ __forceinline__ void token_dots(const void* __restrict__ x, int64_t x0, int64_t stride,
                                           int tc, const float (&w)[BS], Fn fn) {
    constexpr int NG = BS / 16;
    constexpr int WORDS = DT == MO_F32 ? 16 : 8;   // dwords per group of 16 elements
    const uint32_t* xp = (const uint32_t*)((const char*)x + x0 * Elem<DT>::bytes);
    const int64_t stride_words = stride * Elem<DT>::bytes / 4;
    uint32_t cur[WORDS];
#pragma unroll
    for (int j = 0; j < WORDS; ++j) cur[j] = xp[j];
    for (int t = 0; t < tc; ++t) {
        const uint32_t* row = xp + (int64_t)t * stride_words;
        // the group after the last one of this token: the first of the next token (of this
        // token again after the last, a valid address whose data is not used)
        const uint32_t* next_row = t + 1 < tc ? row + stride_words : row;
        // four partial sums: the order of the fp32 accumulation is free, a single chain of
        // dependent adds is not
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            float xs[16];
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                if constexpr (DT == MO_F32) xs[j] = u2f(cur[j]);
                else if constexpr (DT == MO_BF16)
                    xs[j] = (j & 1) ? u2f(cur[j / 2] & 0xFFFF0000u) : u2f(cur[j / 2] << 16);
                else
                    xs[j] = f16_bits_to_f32((j & 1) ? cur[j / 2] >> 16 : cur[j / 2] & 0xFFFFu);
            }
            __builtin_amdgcn_sched_barrier(0);
            const uint32_t* nxt = g + 1 < NG ? row + (g + 1) * WORDS : next_row;
#pragma unroll
            for (int j = 0; j < WORDS; ++j) cur[j] = nxt[j];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < 16; j += 2) {
                if constexpr (DT == MO_BF16) {
                    // both rounded products in one word (one conversion for the pair), added to
                    // a running sum by one instruction: v_dot2c_f32_bf16(pair, (1, 1), acc) =
                    // acc + pair.lo + pair.hi.  Four vector instructions per two products where
                    // multiply, round and add one by one take six.  The instruction's add is
                    // not a correctly rounded fp32 add (about 2e-6 relative at worst) and it
                    // flushes bf16 denormals; the sum is rounded to bf16 below, and measured
                    // against the CPU's arithmetic the losses come out bit-equal as often as
                    // with exact adds (the difference that shows is the order of the adds).
                    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
                    const uint32_t pk = f32x2_to_bf16x2(xs[j] * w[16 * g + j], xs[j + 1] * w[16 * g + j + 1]);
                    const uint32_t one2 = 0x3F803F80u;   // (1.0, 1.0)
                    bf16x2_t pv, ov;
                    __builtin_memcpy(&pv, &pk, 4);
                    __builtin_memcpy(&ov, &one2, 4);
                    acc[(j / 2) & 3] = __builtin_amdgcn_fdot2_f32_bf16(pv, ov, acc[(j / 2) & 3], false);
                } else {
                    acc[j & 3] += clip_round<DT>(xs[j] * w[16 * g + j]);
                    acc[(j + 1) & 3] += clip_round<DT>(xs[j + 1] * w[16 * g + j + 1]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        fn(t, clip_round<DT>((acc[0] + acc[1]) + (acc[2] + acc[3])));
    }
}

// org[] of a lane in LDS, [token][lane] (conflict-free), stored in the tensor dtype (the values
// are rounded to it anyway).
template <int DT> struct OrgStore { typedef uint16_t type; };
template <> struct OrgStore<MO_F32> { typedef float type; };

template <int DT>
__device__ __forceinline__ typename OrgStore<DT>::type org_pack(float v) {
    if constexpr (DT == MO_F32) return v;
    else if constexpr (DT == MO_BF16) return (uint16_t)(f2u(v) >> 16);
    else return (uint16_t)f32_to_f16_bits(v);
}

template <int DT>
__device__ __forceinline__ float org_unpack(typename OrgStore<DT>::type v) {
    if constexpr (DT == MO_F32) return v;
    else if constexpr (DT == MO_BF16) return u2f((uint32_t)v << 16);
    else return f16_bits_to_f32(v);
}

template <int DT, int BS>
__global__ __launch_bounds__(kClipLanes * kClipMaxSplit) void awq_clip_loss_kernel(
    const void* __restrict__ x, int tokens, const void* __restrict__ w, int n, int k,
    const void* __restrict__ w_amax, int amax_dtype, ClipRatios ratios, IntOp op,
    float* __restrict__ loss) {
    constexpr int NC = BS / 8;
    constexpr int GC = NC < 4 ? NC : 4;   // chunks loaded together
    typedef typename OrgStore<DT>::type org_t;
    // dynamic LDS: org[pass_tokens][64] in the tensor dtype, then part[2][split][64] fp32
    extern __shared__ __align__(16) unsigned char clip_smem[];
    const int split = blockDim.x / kClipLanes;
    const int pass_tokens = split * kClipTokens;
    org_t (*org)[kClipLanes] = (org_t (*)[kClipLanes])clip_smem;
    float (*part)[kClipLanes] =
        (float (*)[kClipLanes])(clip_smem + (size_t)pass_tokens * kClipLanes * sizeof(org_t));
    const int lane = threadIdx.x % kClipLanes;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kClipLanes);
    const int nblk = k / BS;
    const int b = blockIdx.y;
    int row = blockIdx.x * kClipLanes + lane;
    const bool active = row < n;
    if (!active) row = n - 1;
    const int64_t w0 = (int64_t)row * k + (int64_t)b * BS;
    const int64_t xb = (int64_t)b * BS;
    const float amax = load_scalar(w_amax, amax_dtype, (int64_t)row * nblk + b);
    float wv[BS];
    // wv <- f(original block): the block is read again from memory (L2) every time, GC chunks
    // of loads in flight, rather than kept in a second set of registers
    auto refill = [&](auto f) {
        // opaque to the optimiser, or it would hoist the (loop-invariant) loads out of the
        // ratio loop and keep the whole block live in registers after all
        int64_t base = w0;
        asm volatile("" : "+v"(base));
#pragma unroll
        for (int c0 = 0; c0 < NC; c0 += GC) {
            RawChunk<DT> raw[GC];
#pragma unroll
            for (int c = 0; c < GC; ++c) load_raw<DT>(w, base + 8 * (c0 + c), raw[c]);
#pragma unroll
            for (int c = 0; c < GC; ++c) {
                float v[8];
                unpack_raw<DT>(raw[c], v);
#pragma unroll
                for (int j = 0; j < 8; ++j) wv[8 * (c0 + c) + j] = f(v[j]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    int flip = 0;   // part[] is double-buffered: one barrier per ratio is enough
    for (int t0 = 0; t0 < tokens; t0 += pass_tokens) {
        const int tc = tokens - t0 < pass_tokens ? tokens - t0 : pass_tokens;
        // this wavefront's share of the pass: tokens [lo, lo + mine)
        const int lo = (int)((int64_t)tc * wave / split);
        const int mine = (int)((int64_t)tc * (wave + 1) / split) - lo;
        const int64_t x0 = (int64_t)(t0 + lo) * k + xb;
        refill([](float v) { return v; });
        token_dots<DT, BS>(x, x0, k, mine, wv,
                           [&](int t, float v) { org[lo + t][lane] = org_pack<DT>(v); });
        for (int r = 0; r < ratios.count; ++r) {
            // `w_amax * ratio` on a tensor: fp32 product rounded to the dtype of the amax
            float clipped = amax * ratios.r[r];
            if (amax_dtype == MO_BF16) clipped = clip_round<MO_BF16>(clipped);
            else if (amax_dtype == MO_F16) clipped = clip_round<MO_F16>(clipped);
            IntOp::Scale s = op.make(clipped);
            // the choice between the exact-reciprocal quotient and a division is per block, not
            // per element: one branch around the whole loop
            if (s.fast) {
                s.fast = true;
                refill([&](float v) { return clip_round<DT>(op.apply<false>(v, s)); });
            } else {
                s.fast = false;
                refill([&](float v) { return clip_round<DT>(op.apply<false>(v, s)); });
            }
            float sum = 0.0f;
            token_dots<DT, BS>(x, x0, k, mine, wv, [&](int t, float cur) {
                const float d = clip_round<DT>(cur - org_unpack<DT>(org[lo + t][lane]));
                sum += d * d;
            });
            if (split > 1) {
                part[flip * split + wave][lane] = sum;
                __syncthreads();
                if (wave == 0) {
                    sum = part[flip * split][lane];
                    for (int v = 1; v < split; ++v) sum += part[flip * split + v][lane];
                }
                flip ^= 1;
            }
            if (active && wave == 0) {
                float* out = loss + ((int64_t)r * n + row) * nblk + b;
                *out += sum / (float)tokens;
            }
        }
    }
}

}  // namespace mo

// loss[r, row, b] += mean over tokens of the squared error of block (row, b) clipped at
// ratios[r] * w_amax[row, b]; see the header for the contract.
extern "C" int mo_awq_clip_losses(const void* x, int64_t tokens, const void* w, int64_t n,
                                  int64_t k, int dtype, int64_t block_size, const void* w_amax,
                                  int amax_dtype, const float* ratios, int n_ratios, int num_bits,
                                  int is_unsigned, int narrow_range, float* loss, void* stream) {
    if (tokens < 0 || n < 0 || k < 0 || n_ratios < 0) return MO_ERR_ARG;
    if (dtype < MO_F32 || dtype > MO_BF16) return MO_ERR_DTYPE;
    if (amax_dtype < MO_F32 || amax_dtype > MO_BF16) return MO_ERR_DTYPE;
    if (num_bits < 2 || num_bits > 16) return MO_ERR_ARG;
    if (block_size != 16 && block_size != 32 && block_size != 64 && block_size != 128)
        return MO_ERR_UNSUPPORTED;
    if (n_ratios > mo::kClipMaxRatios || k % block_size) return MO_ERR_UNSUPPORTED;
    if (tokens > 0x7FFFFFFF || n > 0x7FFFFFFF || k > 0x7FFFFFFF || k / block_size > 65535)
        return MO_ERR_UNSUPPORTED;
    if (tokens == 0 || n == 0 || k == 0 || n_ratios == 0) return MO_OK;
    if (!x || !w || !w_amax || !ratios || !loss) return MO_ERR_ARG;
    if ((((uintptr_t)x | (uintptr_t)w) & 15u) || ((uintptr_t)loss & 3u)) return MO_ERR_ARG;
    mo::ClipRatios rr;
    for (int i = 0; i < mo::kClipMaxRatios; ++i) rr.r[i] = i < n_ratios ? ratios[i] : 0.0f;
    rr.count = n_ratios;
    mo::IntOp op;
    op.bound = (float)((1 << (num_bits - 1 + (is_unsigned ? 1 : 0))) - 1);
    op.lo = is_unsigned ? 0.0f : (narrow_range ? -op.bound : -op.bound - 1.0f);
    const dim3 grid((unsigned)((n + mo::kClipLanes - 1) / mo::kClipLanes),
                    (unsigned)(k / block_size));
    // Wavefronts per 64 (row, block) pairs.  Measured on 4096-wide rows, 64 tokens, bf16: up to
    // about 2048 such sets (two wavefronts per SIMD) a workgroup of four -- one wavefront on
    // each SIMD of a compute unit -- is faster (1024 rows: 848 -> 406 us, 2048 rows: 870 ->
    // 729 us, 3072 rows: 1349 -> 1043 us); from 2048 sets on the single wavefront is (4096 rows:
    // 1359 us either way, 14336 rows: 4017 against 4642 us).  Eight are slower than four
    // everywhere.  Each wavefront should still get 8 tokens or more.
    const int64_t sets = (int64_t)grid.x * grid.y;
    int split = sets < mo::tuned("clip_split_below_sets", 2048) ? mo::kClipMaxSplit : 1;
    while (split > 1 && tokens < 8 * split) split /= 2;
    const size_t elem = dtype == MO_F32 ? 4 : 2;
    if (dtype == MO_F32 && split > 2) split = 2;   // org[] of a pass stays within 64 KB of LDS
    split = (int)mo::tuned("clip_split", split);
    const size_t smem = (size_t)split * mo::kClipTokens * mo::kClipLanes * elem +
                        (split > 1 ? (size_t)2 * split * mo::kClipLanes * sizeof(float) : 0);
    hipStream_t s = (hipStream_t)stream;
#define CALL(DT, BS)                                                                       \
    mo::awq_clip_loss_kernel<DT, BS><<<grid, mo::kClipLanes * split, smem, s>>>(           \
        x, (int)tokens, w, (int)n, (int)k, w_amax, amax_dtype, rr, op, loss)
#define BY_BS(DT)                                                         \
    switch (block_size) {                                                 \
        case 16: CALL(DT, 16); break;                                     \
        case 32: CALL(DT, 32); break;                                     \
        case 64: CALL(DT, 64); break;                                     \
        default: CALL(DT, 128); break;                                    \
    }
    switch (dtype) {
        case MO_F32: BY_BS(MO_F32) break;
        case MO_F16: BY_BS(MO_F16) break;
        default: BY_BS(MO_BF16) break;
    }
#undef BY_BS
#undef CALL
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}
