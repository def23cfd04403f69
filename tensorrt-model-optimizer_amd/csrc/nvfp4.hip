// NVFP4 (E2M1 codes, E4M3 block scales, fp32 global scale) kernels for gfx950:
// quantize + pack, unpack + rescale, and the fused quantize-dequantize.
//
// Work decomposition: a lane owns one chunk (8 elements); a block of BS elements is owned by
// G = BS / 8 adjacent lanes that combine their abs-max with in-wave shuffles, so a wavefront
// load instruction reads 1 KiB (bf16) of contiguous memory and a wavefront store writes 256
// contiguous bytes of codes.  No LDS, no cross-wave traffic.
//
// Algorithmic bytes per element (bf16 in): quantize 2 + 1/2 + 1/16; dequantize 1/2 + 1/16 + 2;
// quantize-dequantize 2 + 2.
#include "common.h"

namespace mo {

// E4M3 byte of a block scale bs = bmax / gs6 (0 -> 1.0).  When the quotient is NaN because of
// an invalid operation (0/0, inf/inf) the x86 reference produces the negative default NaN and
// therefore the byte 0xFF; a NaN that comes from a NaN operand keeps that operand's (positive)
// sign and gives 0x7F.  `cap` is +inf for the reference's cast (a quotient above E4M3's range
// becomes the NaN byte) or 448 to saturate instead (flag MO_FLAG_SATURATE_BLOCK_SCALE).
__device__ __forceinline__ uint32_t block_scale_byte(float bmax, float gs6,
                                                     float cap = __builtin_inff()) {
    float bs = bmax / gs6;
    if (bs == 0.0f) bs = 1.0f;
    if (bs != bs) return (bmax != bmax || gs6 != gs6) ? 0x7Fu : 0xFFu;
    return f32_to_e4m3<false>(bs < cap ? bs : cap);
}

// bits of the `opts` kernel argument
constexpr int kOptForceExact = 1, kOptSaturateScale = 2;
__device__ __forceinline__ float scale_cap(int opts) {
    return (opts & kOptSaturateScale) ? 448.0f : __builtin_inff();
}

template <int G>
__device__ __forceinline__ uint32_t group_max(uint32_t m) {
#pragma unroll
    for (int o = G >> 1; o > 0; o >>= 1) {
        uint32_t t = (uint32_t)__shfl_xor((int)m, o, kWave);
        m = t > m ? t : m;
    }
    return m;
}

__device__ __forceinline__ uint32_t chunk_absmax_bits(const float (&v)[8]) {
    uint32_t m = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        uint32_t t = f2u(v[j]) & 0x7FFFFFFFu;
        m = t > m ? t : m;
    }
    return m;
}

// Chunk c of the zero-padded [rows, kp] view -> loads from the real [rows, k] tensor.
template <int DT, bool FLAT>
__device__ __forceinline__ void load_padded(const void* x, int64_t c, int64_t k, int64_t cpr,
                                            float (&v)[8], int64_t& base, int64_t& col) {
    if constexpr (FLAT) {
        base = 0; col = c << 3;
        load_chunk<DT>(x, col, v);
    } else {
        const int64_t row = c / cpr;
        col = (c - row * cpr) << 3;
        base = row * k;
        load_chunk_guarded<DT>(x, base, col, k, v);
    }
}

// ------------------------------------------------------------------------------ quantize
template <int DT, int BS, bool FLAT>
__global__ __launch_bounds__(256) void nvfp4_quantize_kernel(
    const void* __restrict__ x, int64_t total_chunks, int64_t k, int64_t cpr,
    const float* __restrict__ amax, int amax_is_wsf2, const uint8_t* __restrict__ wsf_in,
    uint32_t* __restrict__ packed, uint8_t* __restrict__ wsf_out, float* __restrict__ wsf2_out,
    int opts) {
    constexpr int G = BS / 8;
    const float wsf2 = amax_is_wsf2 ? amax[0] : amax[0] / 2688.0f;  // 6 * 448
    const float gs6 = 6.0f * wsf2;
    const float cap = scale_cap(opts);
    if (wsf2_out && blockIdx.x == 0 && threadIdx.x == 0) wsf2_out[0] = wsf2;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; c < total_chunks;
         c += stride) {
        float v[8];
        int64_t base, col;
        load_padded<DT, FLAT>(x, c, k, cpr, v, base, col);
        uint32_t byte;
        if (wsf_in) {
            byte = wsf_in[c / G];
        } else {
            const float bmax = u2f(group_max<G>(chunk_absmax_bits(v)));
            byte = block_scale_byte(bmax, gs6, cap);
            if (wsf_out && (threadIdx.x & (G - 1)) == 0) wsf_out[c / G] = (uint8_t)byte;
        }
        const float s = e4m3_to_f32(byte) * wsf2;
        uint32_t w = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) w |= f32_to_e2m1(v[j] / s) << (4 * j);
        __builtin_nontemporal_store(w, packed + c);
    }
}

// ------------------------------------------------------------------------------ dequantize
template <int DT, int BS>
__global__ __launch_bounds__(256) void nvfp4_dequantize_kernel(
    const uint32_t* __restrict__ packed, const uint8_t* __restrict__ wsf,
    const float* __restrict__ wsf2p, int64_t total_chunks, void* __restrict__ y) {
    constexpr int G = BS / 8;
    const float wsf2 = wsf2p[0];
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; c < total_chunks;
         c += stride) {
        const uint32_t w = __builtin_nontemporal_load(packed + c);
        const float s = e4m3_to_f32(wsf[c / G]) * wsf2;
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = e2m1_to_f32((w >> (4 * j)) & 0xFu) * s;
        store_chunk<DT>(y, c << 3, v);
    }
}

// ------------------------------------------------------------------------------ QDQ
// MODE 0: threshold ladder with clamped block scale; MODE 1: quantize -> dequantize.
template <int DT, int BS, int MODE, bool FLAT>
__global__ __launch_bounds__(256) void nvfp4_qdq_kernel(const void* __restrict__ x,
                                                        void* __restrict__ y,
                                                        int64_t total_chunks, int64_t k,
                                                        int64_t cpr, const void* amax,
                                                        int amax_dtype) {
    constexpr int G = BS / 8;
    const float gs = load_scalar(amax, amax_dtype, 0) / 2688.0f;
    const float gs_safe = gs > 0.0f ? gs : 1e-12f;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; c < total_chunks;
         c += stride) {
        float v[8];
        int64_t base, col;
        load_padded<DT, FLAT>(x, c, k, cpr, v, base, col);
        const float bmax = u2f(group_max<G>(chunk_absmax_bits(v)));
        float o[8];
        if constexpr (MODE == 0) {
            float sc = bmax / (6.0f * gs_safe);
            if (sc == sc) sc = sc < 448.0f ? sc : 448.0f;
            float q = round_e4m3<false>(sc) * gs;
            q = q >= 1e-5f ? q : 1.0f;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float r = __builtin_fabsf(v[j]) / q;
                float lvl = 6.0f;
                lvl = r <= 5.0f ? 4.0f : lvl;
                lvl = r < 3.5f ? 3.0f : lvl;
                lvl = r <= 2.5f ? 2.0f : lvl;
                lvl = r < 1.75f ? 1.5f : lvl;
                lvl = r <= 1.25f ? 1.0f : lvl;
                lvl = r < 0.75f ? 0.5f : lvl;
                lvl = r <= 0.25f ? 0.0f : lvl;
                const float t = lvl * q;
                o[j] = v[j] >= 0.0f ? t : -t;
            }
        } else {
            const uint32_t byte = block_scale_byte(bmax, 6.0f * gs);
            const float s = e4m3_to_f32(byte) * gs;
#pragma unroll
            for (int j = 0; j < 8; ++j) o[j] = e2m1_to_f32(f32_to_e2m1(v[j] / s)) * s;
        }
        if constexpr (FLAT) store_chunk<DT>(y, col, o);
        else store_chunk_guarded<DT>(y, base, col, k, o);
    }
}

// ------------------------------------------------------------------------------ fast path
// bf16 input, 16-element blocks, chunk-aligned tensor: a lane owns a whole block (two 16-byte
// loads, one 8-byte store of codes, one scale byte).
//
// The reference divides every element by the block's scale s with an IEEE fp32 division and
// rounds the quotient to E2M1 (ties to even).  The quotient is reproduced exactly, without the
// general division sequence, from one correctly rounded reciprocal per block:
//     r  = RN(1 / s)                       (IEEE division, once per block)
//     q0 = RN(x * r)                       error <= 1.5 ulp
//     q1 = RN(q0 + RN(x - s * q0) * r)     faithful (the residual is exact in an FMA)
//     q  = RN(q1 + RN(x - s * q1) * r)     = RN(x / s)   (Markstein's theorem: a faithful
//                                          quotient and a correctly rounded reciprocal give the
//                                          correctly rounded quotient after one FMA correction)
// valid when nothing over- or underflows; blocks whose scale is outside [2^-64, 2^10], whose
// abs-max is not finite or whose largest quotient would overflow take the general division.
// The hardware E2M1 conversion (round to nearest even, saturating) of q then yields the
// reference's code; a -0.0 input is the one place where the reference's sign rule (v < 0)
// and the hardware's (sign bit) differ, and q is +0.0 there because x - s * q0 is +0.0.

__device__ __forceinline__ uint32_t exact_codes8(const uint32_t (&w)[4], float s) {
    uint32_t o = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        o |= f32_to_e2m1(u2f(w[j] << 16) / s) << (8 * j);
        o |= f32_to_e2m1(u2f(w[j] & 0xFFFF0000u) / s) << (8 * j + 4);
    }
    return o;
}

// One 16-element bf16 block held as 8 packed words -> scale byte and 64 bits of codes.
__device__ __forceinline__ void quantize_block16_bf16(const uint32_t (&w)[8], float wsf2, float gs6,
                                                      int opts, uint32_t& byte,
                                                      uint32_t& c_lo, uint32_t& c_hi) {
    const bool force_exact = opts & kOptForceExact;
    uint32_t m = w[0] & 0x7FFF7FFFu;
#pragma unroll
    for (int j = 1; j < 8; ++j) m = pk_max_u16(m, w[j] & 0x7FFF7FFFu);
    const uint32_t h = (m & 0xFFFFu) > (m >> 16) ? (m & 0xFFFFu) : (m >> 16);
    const float bmax = u2f(h << 16);
    byte = block_scale_byte(bmax, gs6, scale_cap(opts));
    const float s = e4m3_to_f32(byte) * wsf2;
    const uint32_t sb = f2u(s);
    const float r = 1.0f / s;
    const bool fast = !force_exact && sb >= 0x1F800000u && sb <= 0x44800000u && h < 0x7F80u &&
                      (bmax * r < 1.0e38f);
    if (fast) {
        uint32_t lo = 0, hi = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float q0 = exact_quotient(u2f(w[j] << 16), s, r);
            const float q1 = exact_quotient(u2f(w[j] & 0xFFFF0000u), s, r);
            if (j < 4) lo = fp4_pair(lo, q0, q1, j);
            else hi = fp4_pair(hi, q0, q1, j - 4);
        }
        c_lo = lo; c_hi = hi;
    } else {
        const uint32_t w0[4] = {w[0], w[1], w[2], w[3]}, w1[4] = {w[4], w[5], w[6], w[7]};
        c_lo = exact_codes8(w0, s);
        c_hi = exact_codes8(w1, s);
    }
}

// Tiles of kTileBlocks 16-element blocks handled by a workgroup of 256 lanes.
//
// Loads are fully coalesced (lane t of a round reads chunk t, so a wavefront instruction reads
// 1 KiB of contiguous memory); a block's two chunks then sit in adjacent lanes.  Rounds are
// processed in pairs (A, B): the even lane of each pair keeps its A chunk and takes its
// neighbour's A chunk (it now owns a whole round-A block), the odd lane keeps B and takes the
// neighbour's B chunk.  The swap is one DPP move per dword (no LDS).  Every lane therefore
// does the per-block work once for 16 elements, and stores 8 bytes of codes + 1 scale byte.
constexpr int kTileBlocks = MO_NVFP4_TILE_ELEMS / 16;

__device__ __forceinline__ uint32_t swap_adjacent_lanes(uint32_t v) {
    // quad_perm [1, 0, 3, 2]
    return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0xB1, 0xF, 0xF, true);
}

constexpr int kTileRoundPairs = kTileBlocks / 256;

// the raw chunks of one tile: lane t holds chunks t + 512 p (a) and t + 256 + 512 p (b)
struct TileRaw { u32x4 a[kTileRoundPairs], b[kTileRoundPairs]; };

__device__ __forceinline__ void load_tile_bf16(const uint16_t* __restrict__ x, int64_t nblocks,
                                               int64_t tile, TileRaw& r) {
    const int64_t nchunks = nblocks * 2;
    const int64_t c0 = tile * (kTileBlocks * 2) + threadIdx.x;
#pragma unroll
    for (int p = 0; p < kTileRoundPairs; ++p) {
        const int64_t ca = c0 + p * 512, cb = ca + 256;
        const u32x4 zero = {0, 0, 0, 0};
        r.a[p] = ca < nchunks ? __builtin_nontemporal_load(as_global((const u32x4*)(x + ca * 8))) : zero;
        r.b[p] = cb < nchunks ? __builtin_nontemporal_load(as_global((const u32x4*)(x + cb * 8))) : zero;
    }
}

__device__ __forceinline__ void quantize_loaded_tile_bf16(const TileRaw& r, int64_t nblocks,
                                                          int64_t tile, float wsf2, float gs6,
                                                          int opts, u32x2* __restrict__ packed,
                                                          uint8_t* __restrict__ wsf) {
    const int64_t nchunks = nblocks * 2;
    const int64_t c0 = tile * (kTileBlocks * 2) + threadIdx.x;
    const bool odd = threadIdx.x & 1;
#pragma unroll
    for (int p = 0; p < kTileRoundPairs; ++p) {
        const int64_t ca = c0 + p * 512, cb = ca + 256;
        const u32x4 send = odd ? r.a[p] : r.b[p];
        u32x4 recv;
        recv.x = swap_adjacent_lanes(send.x);
        recv.y = swap_adjacent_lanes(send.y);
        recv.z = swap_adjacent_lanes(send.z);
        recv.w = swap_adjacent_lanes(send.w);
        const u32x4 first = odd ? recv : r.a[p], second = odd ? r.b[p] : recv;
        const uint32_t w[8] = {first.x, first.y, first.z, first.w,
                               second.x, second.y, second.z, second.w};
        uint32_t byte, lo, hi;
        quantize_block16_bf16(w, wsf2, gs6, opts, byte, lo, hi);
        const int64_t mine = odd ? cb : ca;  // odd: chunks (cb - 1, cb); even: (ca, ca + 1)
        if (mine < nchunks) {
            const int64_t blk = mine >> 1;
            u32x2 o = {lo, hi};
            __builtin_nontemporal_store(o, as_global(packed + blk));
            *as_global(wsf + blk) = (uint8_t)byte;
        }
    }
}

__device__ __forceinline__ void quantize_tile_bf16(const uint16_t* __restrict__ x,
                                                   int64_t nblocks, int64_t tile, float wsf2,
                                                   float gs6, int opts,
                                                   u32x2* __restrict__ packed,
                                                   uint8_t* __restrict__ wsf) {
    TileRaw r;
    load_tile_bf16(x, nblocks, tile, r);
    quantize_loaded_tile_bf16(r, nblocks, tile, wsf2, gs6, opts, packed, wsf);
}

__global__ __launch_bounds__(256) void nvfp4_quantize_fast_kernel(
    const uint16_t* __restrict__ x, int64_t nblocks, int64_t tiles,
    const float* __restrict__ amax, int amax_is_wsf2, int opts,
    u32x2* __restrict__ packed, uint8_t* __restrict__ wsf_out, float* __restrict__ wsf2_out) {
    const float wsf2 = amax_is_wsf2 ? amax[0] : amax[0] / 2688.0f;
    const float gs6 = 6.0f * wsf2;
    if (wsf2_out && blockIdx.x == 0 && threadIdx.x == 0) wsf2_out[0] = wsf2;
    quantize_tile_bf16(x, nblocks, blockIdx.x, wsf2, gs6, opts, packed, wsf_out);
}

// Many tensors, one launch.  One workgroup per tile, dispatched in tile order so the set of
// tiles in flight stays a compact window of memory (a persistent grid drifts apart over a
// multi-gigabyte pass and loses ~10 % of the bandwidth).  tile_job[t] names the tensor of tile
// t; without it the job is found by binary search over tile_begin.
__global__ __launch_bounds__(256) void nvfp4_quantize_multi_kernel(
    const mo_nvfp4_job* __restrict__ jobs, int njobs, const int32_t* __restrict__ tile_job,
    int amax_is_wsf2, int opts) {
    const int64_t t = blockIdx.x;
    int lo;
    if (tile_job) {
        lo = tile_job[t];
    } else {
        lo = 0;
        int hi = njobs - 1;
        while (lo < hi) {  // last job with tile_begin <= t
            const int mid = (lo + hi + 1) >> 1;
            if (jobs[mid].tile_begin <= t) lo = mid; else hi = mid - 1;
        }
    }
    const mo_nvfp4_job jb = jobs[lo];
    // The amax is fetched with a vector load through the generic pointer, and the global scale
    // stored, before the tile's loads go out.  Measured against this in alternating runs:
    // issuing the tile's loads first (they do not depend on the amax) is 2 % slower at every
    // occupancy cap, and fetching the amax through the scalar cache (a much shorter round trip)
    // 5 % slower; an explicit sleep of 0.5 us or more at the start is slower too.  The launch is
    // short of memory bandwidth, not of requests in flight, and the round trip of this one load
    // happens to space the workgroups' bursts well.
    const float a = jb.amax[0];
    const float wsf2 = amax_is_wsf2 ? a : a / 2688.0f;
    if (jb.wsf2_out && t == jb.tile_begin && threadIdx.x == 0) jb.wsf2_out[0] = wsf2;
    quantize_tile_bf16((const uint16_t*)jb.x, jb.elems >> 4, t - jb.tile_begin, wsf2, 6.0f * wsf2,
                       opts, (u32x2*)jb.packed, jb.wsf);
}

// Abs-max and quantize + pack in ONE launch that reads the tensor once: workgroup w loads tiles
// w, w + G, ... (TP of them) into registers, the workgroups agree on the global abs-max
// (grid_max_exchange) and each quantises the tiles it holds.
template <int TP>
__global__ __launch_bounds__(256) void nvfp4_quantize_fused_kernel(
    const uint16_t* __restrict__ x, int64_t nblocks, int64_t tiles, int opts,
    u32x2* __restrict__ packed, uint8_t* __restrict__ wsf_out, float* __restrict__ wsf2_out,
    float* __restrict__ amax_out, uint32_t* __restrict__ ws, uint32_t spin_limit) {
    __shared__ uint32_t smem[8];
    TileRaw r[TP];
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < TP; ++i) {
        const int64_t t = (int64_t)i * gridDim.x + blockIdx.x;
        load_tile_bf16(x, nblocks, t < tiles ? t : tiles, r[i]);  // past the end: all zero
    }
#pragma unroll
    for (int i = 0; i < TP; ++i)
#pragma unroll
        for (int p = 0; p < kTileRoundPairs; ++p) {
            const u32x4 a = r[i].a[p], b = r[i].b[p];
            m = pk_max_u16(m, pk_max_u16(pk_max_u16(a.x & 0x7FFF7FFFu, a.y & 0x7FFF7FFFu),
                                         pk_max_u16(a.z & 0x7FFF7FFFu, a.w & 0x7FFF7FFFu)));
            m = pk_max_u16(m, pk_max_u16(pk_max_u16(b.x & 0x7FFF7FFFu, b.y & 0x7FFF7FFFu),
                                         pk_max_u16(b.z & 0x7FFF7FFFu, b.w & 0x7FFF7FFFu)));
        }
    const uint32_t h = (m & 0xFFFFu) > (m >> 16) ? (m & 0xFFFFu) : (m >> 16);
    uint32_t gbits;
    if (!grid_max_exchange(ws, h << 16, gridDim.x, spin_limit, smem, gbits)) {
        // the wait for the other workgroups expired: take the abs-max of the whole tensor here
        // (16-element blocks of bf16 = two 16-byte units each)
        keep_branch();
        gbits = workgroup_absmax_bits<false>(x, nblocks * 2, 0u, smem) << 16;
    }
    const float amax = u2f(gbits);
    const float wsf2 = amax / 2688.0f;
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        if (amax_out) amax_out[0] = amax;
        if (wsf2_out) wsf2_out[0] = wsf2;
    }
#pragma unroll
    for (int i = 0; i < TP; ++i) {
        const int64_t t = (int64_t)i * gridDim.x + blockIdx.x;
        if (t < tiles) quantize_loaded_tile_bf16(r[i], nblocks, t, wsf2, 6.0f * wsf2, opts, packed, wsf_out);
    }
}

template <int TP>
static int launch_quantize_fused(const uint16_t* x, int64_t nblocks, int64_t tiles, int opts,
                                 u32x2* packed, uint8_t* wsf_out, float* wsf2_out, float* amax_out,
                                 uint32_t* ws, uint32_t spin_limit, hipStream_t s) {
    static int limit[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return MO_ERR_LAUNCH;
    if (!limit[dev]) {
        const int l = resident_grid_limit(nvfp4_quantize_fused_kernel<TP>, 256);
        limit[dev] = l > 0 ? l : -1;
    }
    if (limit[dev] < 0) return MO_ERR_UNSUPPORTED;
    const int64_t grid = (tiles + TP - 1) / TP;
    if (grid > limit[dev]) return MO_ERR_TOO_LARGE;
    nvfp4_quantize_fused_kernel<TP><<<dim3((unsigned)grid), 256, 0, s>>>(
        x, nblocks, tiles, opts, packed, wsf_out, wsf2_out, amax_out, ws, spin_limit);
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

// ------------------------------------------------------------------------------ fast dequantize
// bf16 output, 16-element blocks: a lane owns a chunk (4 bytes of codes in, 16 bytes out, the
// scale byte shared with the neighbouring lane), so loads and stores of a wavefront are
// contiguous.  Codes are decoded by v_cvt_scalef32_pk_f32_fp4; "+ 0.0f" turns the hardware's
// -0.0 for code 8 into the table's +0.0.
typedef float f32x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void decode8(uint32_t codes, float s, float (&v)[8]) {
#define MO_DEC(SEL)                                                                     \
    {                                                                                   \
        f32x2_t p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(codes, 1.0f, SEL);         \
        v[2 * SEL] = (p.x + 0.0f) * s;                                                  \
        v[2 * SEL + 1] = (p.y + 0.0f) * s;                                              \
    }
    MO_DEC(0) MO_DEC(1) MO_DEC(2) MO_DEC(3)
#undef MO_DEC
}

constexpr int kDequantRounds = 8;  // chunks per lane (4 measures the same, 2 is 15 % slower)

__global__ __launch_bounds__(256) void nvfp4_dequantize_fast_kernel(
    const uint32_t* __restrict__ packed, const uint8_t* __restrict__ wsf,
    const float* __restrict__ wsf2p, int64_t nchunks, uint16_t* __restrict__ y) {
    constexpr int R = kDequantRounds;
    const float wsf2 = wsf2p[0];
    const int64_t c0 = (int64_t)blockIdx.x * (256 * R) + threadIdx.x;
    uint32_t c[R], sb[R];
    // every load in straight-line code (a lane past the end re-reads the last chunk), only the
    // stores conditional: with the loads inside per-round branches the compiler waits at every
    // join for all memory operations in flight, the previous round's store among them
#pragma unroll
    for (int r = 0; r < R; ++r) {
        int64_t ch = c0 + r * 256;
        ch = ch < nchunks ? ch : nchunks - 1;
        c[r] = __builtin_nontemporal_load(packed + ch);
        sb[r] = wsf[ch >> 1];
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int64_t ch = c0 + r * 256;
        float v[8];
        decode8(c[r], e4m3_to_f32(sb[r]) * wsf2, v);
        if (ch < nchunks) store_chunk<MO_BF16>(y, ch * 8, v);
    }
}

// ------------------------------------------------------------------------------ fast QDQ
// bf16 in/out, 16-element blocks, aligned, no padding: same data movement as the quantize fast
// path (coalesced chunk loads, lane-pair exchange so a lane owns a block), the quotient by the
// exact reciprocal-and-FMA division, E2M1 rounding and decoding by the hardware converts.
template <int MODE>
__device__ __forceinline__ void qdq_block16_bf16(const uint32_t (&w)[8], float gs, float gs_safe,
                                                 float (&lo)[8], float (&hi)[8]) {
    uint32_t m = w[0] & 0x7FFF7FFFu;
#pragma unroll
    for (int j = 1; j < 8; ++j) m = pk_max_u16(m, w[j] & 0x7FFF7FFFu);
    const uint32_t h = (m & 0xFFFFu) > (m >> 16) ? (m & 0xFFFFu) : (m >> 16);
    const float bmax = u2f(h << 16);
    float x[16];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        x[2 * j] = u2f(w[j] << 16);
        x[2 * j + 1] = u2f(w[j] & 0xFFFF0000u);
    }
    float s;  // the value one code unit stands for
    if constexpr (MODE == 0) {
        float sc = bmax / (6.0f * gs_safe);
        if (sc == sc) sc = sc < 448.0f ? sc : 448.0f;
        s = round_e4m3<false>(sc) * gs;
        s = s >= 1e-5f ? s : 1.0f;
    } else {
        s = e4m3_to_f32(block_scale_byte(bmax, 6.0f * gs)) * gs;
    }
    const float r = 1.0f / s;
    const uint32_t sb = f2u(s);
    const bool fast = sb >= 0x1F800000u && sb <= 0x44800000u && h < 0x7F80u && (bmax * r < 1.0e38f);
    float o[16];
    if (fast) {
        uint32_t c0 = 0, c1 = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float a = MODE == 0 ? __builtin_fabsf(x[2 * j]) : x[2 * j];
            const float b = MODE == 0 ? __builtin_fabsf(x[2 * j + 1]) : x[2 * j + 1];
            const float qa = exact_quotient(a, s, r), qb = exact_quotient(b, s, r);
            if (j < 4) c0 = fp4_pair(c0, qa, qb, j);
            else c1 = fp4_pair(c1, qa, qb, j - 4);
        }
        float d0[8], d1[8];
        decode8(c0, s, d0);
        decode8(c1, s, d1);
#pragma unroll
        for (int j = 0; j < 8; ++j) { o[j] = d0[j]; o[8 + j] = d1[j]; }
        if constexpr (MODE == 0) {
#pragma unroll
            for (int j = 0; j < 16; ++j) o[j] = x[j] >= 0.0f ? o[j] : -o[j];
        }
    } else {
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            if constexpr (MODE == 0) {
                const float q = __builtin_fabsf(x[j]) / s;
                float lvl = 6.0f;
                lvl = q <= 5.0f ? 4.0f : lvl;
                lvl = q < 3.5f ? 3.0f : lvl;
                lvl = q <= 2.5f ? 2.0f : lvl;
                lvl = q < 1.75f ? 1.5f : lvl;
                lvl = q <= 1.25f ? 1.0f : lvl;
                lvl = q < 0.75f ? 0.5f : lvl;
                lvl = q <= 0.25f ? 0.0f : lvl;
                const float t = lvl * s;
                o[j] = x[j] >= 0.0f ? t : -t;
            } else {
                o[j] = e2m1_to_f32(f32_to_e2m1(x[j] / s)) * s;
            }
        }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) { lo[j] = o[j]; hi[j] = o[8 + j]; }
}

// RP = pairs of 16-byte loads per lane (a workgroup handles RP * 256 blocks).  Measured: one pair
// beats four from 50 MB of input (8192 x 4096: 5.4 - 5.7 TB/s against 5.0; 537 MB: 6.45 against
// 6.0) and ties at 34 MB; smaller tensors keep four (fewer workgroups to launch).
template <int MODE, int RP>
__global__ __launch_bounds__(256) void nvfp4_qdq_fast_kernel(const uint16_t* __restrict__ x,
                                                             uint16_t* __restrict__ y,
                                                             int64_t nblocks, const void* amax,
                                                             int amax_dtype) {
    const float gs = load_scalar(amax, amax_dtype, 0) / 2688.0f;
    const float gs_safe = gs > 0.0f ? gs : 1e-12f;
    const int64_t nchunks = nblocks * 2;
    const int64_t c0 = (int64_t)blockIdx.x * (RP * 512) + threadIdx.x;
    const bool odd = threadIdx.x & 1;
    u32x4 a[RP], b[RP];
#pragma unroll
    for (int p = 0; p < RP; ++p) {
        const int64_t ca = c0 + p * 512, cb = ca + 256;
        const u32x4 zero = {0, 0, 0, 0};
        a[p] = ca < nchunks ? __builtin_nontemporal_load((const u32x4*)(x + ca * 8)) : zero;
        b[p] = cb < nchunks ? __builtin_nontemporal_load((const u32x4*)(x + cb * 8)) : zero;
    }
#pragma unroll
    for (int p = 0; p < RP; ++p) {
        const int64_t ca = c0 + p * 512, cb = ca + 256;
        const u32x4 send = odd ? a[p] : b[p];
        u32x4 recv;
        recv.x = swap_adjacent_lanes(send.x);
        recv.y = swap_adjacent_lanes(send.y);
        recv.z = swap_adjacent_lanes(send.z);
        recv.w = swap_adjacent_lanes(send.w);
        const u32x4 first = odd ? recv : a[p], second = odd ? b[p] : recv;
        const uint32_t w[8] = {first.x, first.y, first.z, first.w,
                               second.x, second.y, second.z, second.w};
        float lo[8], hi[8];
        qdq_block16_bf16<MODE>(w, gs, gs_safe, lo, hi);
        // back to the load layout, so that the stores are contiguous across the wavefront:
        // the even lane hands over the second chunk of its round-A block and receives the
        // first chunk of the neighbour's round-B block; the odd lane the other way round.
        u32x4 o0, o1;
        o0.x = f32x2_to_bf16x2(lo[0], lo[1]); o0.y = f32x2_to_bf16x2(lo[2], lo[3]);
        o0.z = f32x2_to_bf16x2(lo[4], lo[5]); o0.w = f32x2_to_bf16x2(lo[6], lo[7]);
        o1.x = f32x2_to_bf16x2(hi[0], hi[1]); o1.y = f32x2_to_bf16x2(hi[2], hi[3]);
        o1.z = f32x2_to_bf16x2(hi[4], hi[5]); o1.w = f32x2_to_bf16x2(hi[6], hi[7]);
        const u32x4 give = odd ? o0 : o1;
        u32x4 got;
        got.x = swap_adjacent_lanes(give.x);
        got.y = swap_adjacent_lanes(give.y);
        got.z = swap_adjacent_lanes(give.z);
        got.w = swap_adjacent_lanes(give.w);
        const u32x4 out_a = odd ? got : o0, out_b = odd ? o1 : got;
        if (ca < nchunks) __builtin_nontemporal_store(out_a, (u32x4*)(y + ca * 8));
        if (cb < nchunks) __builtin_nontemporal_store(out_b, (u32x4*)(y + cb * 8));
    }
}

static inline unsigned grid_for(int64_t chunks) {
    int64_t b = (chunks + 255) / 256;
    if (b < 1) b = 1;
    if (b > 16384) b = 16384;
    return (unsigned)b;
}

template <int DT, int BS>
static void launch_quantize(const void* x, int64_t rows, int64_t k, int64_t kp, const float* amax,
                            int is_wsf2, const uint8_t* wsf_in, uint8_t* packed, uint8_t* wsf_out,
                            float* wsf2_out, int opts, hipStream_t s) {
    const int64_t cpr = kp / 8, total = rows * cpr;
    const bool flat = (k == kp) && (((uintptr_t)x & 15u) == 0);
    if (flat)
        nvfp4_quantize_kernel<DT, BS, true><<<grid_for(total), 256, 0, s>>>(
            x, total, k, cpr, amax, is_wsf2, wsf_in, (uint32_t*)packed, wsf_out, wsf2_out, opts);
    else
        nvfp4_quantize_kernel<DT, BS, false><<<grid_for(total), 256, 0, s>>>(
            x, total, k, cpr, amax, is_wsf2, wsf_in, (uint32_t*)packed, wsf_out, wsf2_out, opts);
}

template <int DT, int BS>
static void launch_qdq(const void* x, void* y, int64_t rows, int64_t k, int64_t kp,
                       const void* amax, int amax_dtype, int mode, hipStream_t s) {
    const int64_t cpr = kp / 8, total = rows * cpr;
    const bool flat = (k == kp) && (((uintptr_t)x & 15u) == 0) && (((uintptr_t)y & 15u) == 0);
    const unsigned g = grid_for(total);
    if (mode == 0) {
        if (flat) nvfp4_qdq_kernel<DT, BS, 0, true><<<g, 256, 0, s>>>(x, y, total, k, cpr, amax, amax_dtype);
        else nvfp4_qdq_kernel<DT, BS, 0, false><<<g, 256, 0, s>>>(x, y, total, k, cpr, amax, amax_dtype);
    } else {
        if (flat) nvfp4_qdq_kernel<DT, BS, 1, true><<<g, 256, 0, s>>>(x, y, total, k, cpr, amax, amax_dtype);
        else nvfp4_qdq_kernel<DT, BS, 1, false><<<g, 256, 0, s>>>(x, y, total, k, cpr, amax, amax_dtype);
    }
}

}  // namespace mo

static_assert(mo::kOptForceExact == MO_FLAG_FORCE_EXACT &&
              mo::kOptSaturateScale == MO_FLAG_SATURATE_BLOCK_SCALE, "flag bits");
constexpr int kKnownFlags = MO_FLAG_FORCE_EXACT | MO_FLAG_SATURATE_BLOCK_SCALE;

#define MO_DISPATCH_DT_BS(dtype, bs, CALL)                                            \
    switch (dtype) {                                                                  \
        case MO_F32:                                                                  \
            if (bs == 8) { CALL(MO_F32, 8); } else if (bs == 16) { CALL(MO_F32, 16); } \
            else { CALL(MO_F32, 32); }                                                \
            break;                                                                    \
        case MO_F16:                                                                  \
            if (bs == 8) { CALL(MO_F16, 8); } else if (bs == 16) { CALL(MO_F16, 16); } \
            else { CALL(MO_F16, 32); }                                                \
            break;                                                                    \
        case MO_BF16:                                                                 \
            if (bs == 8) { CALL(MO_BF16, 8); } else if (bs == 16) { CALL(MO_BF16, 16); } \
            else { CALL(MO_BF16, 32); }                                               \
            break;                                                                    \
        default: return MO_ERR_DTYPE;                                                 \
    }

extern "C" int mo_nvfp4_quantize(const void* x, int64_t rows, int64_t k, int dtype, int block_size,
                                 const float* amax, int amax_is_wsf2, const uint8_t* wsf_in,
                                 uint8_t* packed, uint8_t* wsf_out, float* wsf2_out,
                                 int flags, void* stream) {
    if (rows < 0 || k < 0 || (flags & ~kKnownFlags)) return MO_ERR_ARG;
    if (block_size != 8 && block_size != 16 && block_size != 32) return MO_ERR_UNSUPPORTED;
    if (rows == 0 || k == 0) return MO_OK;
    if (!x || !amax || !packed || (!wsf_in && !wsf_out)) return MO_ERR_ARG;
    if ((uintptr_t)packed & 3u) return MO_ERR_ARG;
    const int64_t kp = (k + block_size - 1) / block_size * block_size;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == MO_BF16 && block_size == 16 && k == kp && !wsf_in &&
        (((uintptr_t)x & 15u) == 0) && (((uintptr_t)packed & 7u) == 0)) {
        const int64_t nblocks = rows * k / 16;
        const int64_t tiles = (nblocks + mo::kTileBlocks - 1) / mo::kTileBlocks;
        if (tiles > 0x7FFFFFFF) return MO_ERR_UNSUPPORTED;
        // the occupancy cap pays above about a gigabyte; below, the shorter ramp of a full chip wins
        const int cap_kb = tiles >= 32768 ? 36 : 0;
        mo::nvfp4_quantize_fast_kernel<<<(unsigned)tiles, 256, mo::ballast_bytes("nvfp4_quantize_fast_kernel", cap_kb), s>>>(
            (const uint16_t*)x, nblocks, tiles, amax, amax_is_wsf2, flags,
            (mo::u32x2*)packed, wsf_out, wsf2_out);
        return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
    }
#define CALL(DT, BS) \
    mo::launch_quantize<DT, BS>(x, rows, k, kp, amax, amax_is_wsf2, wsf_in, packed, wsf_out, wsf2_out, \
                                flags, s)
    MO_DISPATCH_DT_BS(dtype, block_size, CALL)
#undef CALL
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_nvfp4_dequantize(const uint8_t* packed, const uint8_t* wsf, const float* wsf2,
                                   int64_t rows, int64_t kp, int block_size, void* y, int dtype,
                                   void* stream) {
    if (rows < 0 || kp < 0) return MO_ERR_ARG;
    if (block_size != 8 && block_size != 16 && block_size != 32) return MO_ERR_UNSUPPORTED;
    if (rows == 0 || kp == 0) return MO_OK;
    if (!packed || !wsf || !wsf2 || !y || kp % block_size) return MO_ERR_ARG;
    if (((uintptr_t)packed & 3u) || ((uintptr_t)y & 15u)) return MO_ERR_ARG;
    const int64_t total = rows * (kp / 8);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == MO_BF16 && block_size == 16) {
        const int64_t per_tile = 256 * mo::kDequantRounds;
        const int64_t tiles = (total + per_tile - 1) / per_tile;
        if (tiles > 0x7FFFFFFF) return MO_ERR_UNSUPPORTED;
        mo::nvfp4_dequantize_fast_kernel<<<(unsigned)tiles, 256, mo::ballast_bytes("nvfp4_dequantize_fast_kernel", 0), s>>>(
            (const uint32_t*)packed, wsf, wsf2, total, (uint16_t*)y);
        return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
    }
#define CALL(DT, BS)                                                                      \
    mo::nvfp4_dequantize_kernel<DT, BS><<<mo::grid_for(total), 256, 0, s>>>(              \
        (const uint32_t*)packed, wsf, wsf2, total, y)
    MO_DISPATCH_DT_BS(dtype, block_size, CALL)
#undef CALL
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_nvfp4_qdq(const void* x, void* y, int64_t rows, int64_t k, int dtype,
                            const void* amax, int amax_dtype, int block_size, int mode,
                            void* stream) {
    if (rows < 0 || k < 0 || (mode != 0 && mode != 1)) return MO_ERR_ARG;
    if (block_size != 8 && block_size != 16 && block_size != 32) return MO_ERR_UNSUPPORTED;
    if (amax_dtype < MO_F32 || amax_dtype > MO_BF16) return MO_ERR_DTYPE;
    if (rows == 0 || k == 0) return MO_OK;
    if (!x || !y || !amax) return MO_ERR_ARG;
    const int64_t kp = (k + block_size - 1) / block_size * block_size;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == MO_BF16 && block_size == 16 && k == kp &&
        ((((uintptr_t)x | (uintptr_t)y) & 15u) == 0)) {
        const int64_t nblocks = rows * k / 16;
        const bool big = nblocks >= mo::tuned("nvfp4_qdq_big_blocks", 1ll << 20);   // 16 Mi elements = 32 MB of bf16
        const int64_t per_tile = (big ? 1 : 4) * 256;         // blocks per workgroup
        const int64_t tiles = (nblocks + per_tile - 1) / per_tile;
        if (tiles > 0x7FFFFFFF) return MO_ERR_UNSUPPORTED;
        const unsigned g = (unsigned)tiles;
        const size_t cap = mo::ballast_bytes("nvfp4_qdq_fast_kernel", 0);
        const uint16_t* xi = (const uint16_t*)x;
        uint16_t* yo = (uint16_t*)y;
        if (mode == 0 && big) mo::nvfp4_qdq_fast_kernel<0, 1><<<g, 256, cap, s>>>(xi, yo, nblocks, amax, amax_dtype);
        else if (mode == 0) mo::nvfp4_qdq_fast_kernel<0, 4><<<g, 256, cap, s>>>(xi, yo, nblocks, amax, amax_dtype);
        else if (big) mo::nvfp4_qdq_fast_kernel<1, 1><<<g, 256, cap, s>>>(xi, yo, nblocks, amax, amax_dtype);
        else mo::nvfp4_qdq_fast_kernel<1, 4><<<g, 256, cap, s>>>(xi, yo, nblocks, amax, amax_dtype);
        return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
    }
#define CALL(DT, BS) mo::launch_qdq<DT, BS>(x, y, rows, k, kp, amax, amax_dtype, mode, s)
    MO_DISPATCH_DT_BS(dtype, block_size, CALL)
#undef CALL
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_nvfp4_quantize_multi(const mo_nvfp4_job* jobs_dev, int njobs,
                                       const int32_t* tile_job_dev, int64_t total_tiles,
                                       int dtype, int block_size, int amax_is_wsf2,
                                       int flags, void* stream) {
    if (njobs < 0 || total_tiles < 0 || total_tiles > 0x7FFFFFFF || (flags & ~kKnownFlags))
        return MO_ERR_ARG;
    if (dtype != MO_BF16 || block_size != 16) return MO_ERR_UNSUPPORTED;
    if (njobs == 0 || total_tiles == 0) return MO_OK;
    if (!jobs_dev) return MO_ERR_ARG;
    const int cap_kb = total_tiles >= 32768 ? 36 : 0;
    mo::nvfp4_quantize_multi_kernel<<<(unsigned)total_tiles, 256, mo::ballast_bytes("nvfp4_quantize_multi_kernel", cap_kb), (hipStream_t)stream>>>(
        jobs_dev, njobs, tile_job_dev, amax_is_wsf2, flags);
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_nvfp4_quantize_fused(const void* x, int64_t rows, int64_t k, int dtype,
                                       int block_size, uint8_t* packed, uint8_t* wsf_out,
                                       float* wsf2_out, float* amax_out, int flags,
                                       void* workspace, int64_t spin_limit, void* stream) {
    if (rows < 0 || k < 0 || (flags & ~kKnownFlags) || spin_limit < 0) return MO_ERR_ARG;
    if (dtype != MO_BF16 || block_size != 16 || k % 16) return MO_ERR_UNSUPPORTED;
    if (rows == 0 || k == 0) return MO_OK;
    if (!x || !packed || !wsf_out || !workspace) return MO_ERR_ARG;
    if (((uintptr_t)x & 15u) || ((uintptr_t)packed & 7u) || ((uintptr_t)workspace & 127u))
        return MO_ERR_UNSUPPORTED;
    const int64_t nblocks = rows * k / 16;
    const int64_t tiles = (nblocks + mo::kTileBlocks - 1) / mo::kTileBlocks;
    const uint32_t spins = spin_limit > 0xFFFFFFFFll ? 0xFFFFFFFFu : (uint32_t)spin_limit;
    hipStream_t s = (hipStream_t)stream;
    // the fewer workgroups meet at the exchange, the cheaper it is: as many tiles per workgroup
    // (1, 2, 4) as keep the grid at two workgroups per compute unit, more workgroups after that
    int rc = MO_ERR_TOO_LARGE;
    if (tiles <= 512)
        rc = mo::launch_quantize_fused<1>((const uint16_t*)x, nblocks, tiles, flags, (mo::u32x2*)packed,
                                          wsf_out, wsf2_out, amax_out, (uint32_t*)workspace, spins, s);
    if (rc == MO_ERR_TOO_LARGE && tiles <= 1024)
        rc = mo::launch_quantize_fused<2>((const uint16_t*)x, nblocks, tiles, flags, (mo::u32x2*)packed,
                                          wsf_out, wsf2_out, amax_out, (uint32_t*)workspace, spins, s);
    if (rc == MO_ERR_TOO_LARGE)
        rc = mo::launch_quantize_fused<4>((const uint16_t*)x, nblocks, tiles, flags, (mo::u32x2*)packed,
                                          wsf_out, wsf2_out, amax_out, (uint32_t*)workspace, spins, s);
    return rc;
}

// ------------------------------------------------------------------------------ E2M1 codes
// One code byte per element: sign << 3 | ordinal of the nearest E2M1 magnitude, ties to the even
// code (NVFP4QTensor._cast_fp4, TQ/qtensor/nvfp4_tensor.py:120-140).
namespace mo {
template <int DT>
__global__ __launch_bounds__(256) void cast_fp4_kernel(const void* __restrict__ x, int64_t n,
                                                       uint8_t* __restrict__ codes) {
    const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i0 >= n) return;
    if (i0 + 4 <= n && (((uintptr_t)codes) & 3u) == 0) {
        uint32_t w = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) w |= f32_to_e2m1(load_elem<DT>(x, i0 + j)) << (8 * j);
        *(uint32_t*)(codes + i0) = w;
    } else {
        for (int64_t i = i0; i < n && i < i0 + 4; ++i) codes[i] = (uint8_t)f32_to_e2m1(load_elem<DT>(x, i));
    }
}
}  // namespace mo

extern "C" int mo_cast_fp4(const void* x, int64_t n, int dtype, uint8_t* codes, void* stream) {
    if (n < 0) return MO_ERR_ARG;
    if (dtype < MO_F32 || dtype > MO_BF16) return MO_ERR_DTYPE;
    if (n == 0) return MO_OK;
    if (!x || !codes) return MO_ERR_ARG;
    const int64_t grid = (n + 1023) / 1024;
    if (grid > 0x7FFFFFFF) return MO_ERR_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case MO_F32: mo::cast_fp4_kernel<MO_F32><<<(unsigned)grid, 256, 0, s>>>(x, n, codes); break;
        case MO_F16: mo::cast_fp4_kernel<MO_F16><<<(unsigned)grid, 256, 0, s>>>(x, n, codes); break;
        default: mo::cast_fp4_kernel<MO_BF16><<<(unsigned)grid, 256, 0, s>>>(x, n, codes); break;
    }
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}
