// Shared device helpers for the gfx950 quantization kernels.
//
// Conventions used by every kernel in this directory:
//  * one "chunk" = 8 consecutive elements of the innermost dimension; a lane loads a chunk with
//    one 16-byte access for 16-bit inputs (two for fp32), so a wavefront instruction touches
//    1 KiB of contiguous memory when the tensor is chunk aligned;
//  * all rounding that decides an output bit is done in software on integer bit patterns or
//    with IEEE fp32 operations (no approximate reciprocal decides a bit on its own);
//  * abs-max values travel as the uint32 bit pattern of a non-negative fp32: unsigned integer
//    order equals numeric order there and every NaN pattern sorts above +inf, so an integer max
//    propagates NaN exactly like torch.max does.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#ifdef MO_TUNING
#include <stdio.h>
#include <stdlib.h>
#endif

#include "../../include/modelopt_hip.h"

namespace mo {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;

// Occupancy cap of the streaming kernels.  A launch asks for `kb` KiB of dynamic LDS that the
// kernel never touches: a CU has 160 KiB, so floor(160 / kb) workgroups fit on it instead of the
// 7 or 8 the register budget would allow.  With every lane keeping 4 to 8 16-byte loads in
// flight, 4 workgroups per CU (about 32 MB in flight over the chip) already cover the memory
// latency, and more concurrent streams only cost DRAM efficiency: the mixed read/write kernels
// gain 5 - 11 % from the cap.  0 = no cap.  A build with -DMO_TUNING reads
// MO_BALLAST_<kernel> / MO_BALLAST_ALL from the environment at every launch (sweeps only).
inline size_t ballast_bytes(const char* kernel, int kb) {
#ifdef MO_TUNING
    char key[160];
    snprintf(key, sizeof key, "MO_BALLAST_%s", kernel);
    if (const char* e = getenv(key)) return (size_t)atoi(e) << 10;
    if (const char* e = getenv("MO_BALLAST_ALL")) return (size_t)atoi(e) << 10;
#else
    (void)kernel;
#endif
    return (size_t)kb << 10;
}

// A launch parameter (grid size, rows per slab ...): `value` in the product build; a build with
// -DMO_TUNING reads MO_TUNE_<name> from the environment at every launch (sweeps only).
inline int64_t tuned(const char* name, int64_t value) {
#ifdef MO_TUNING
    char key[160];
    snprintf(key, sizeof key, "MO_TUNE_%s", name);
    if (const char* e = getenv(key)) return atoll(e);
#else
    (void)name;
#endif
    return value;
}

// A pointer known to address device (global) memory, as one of that address space: loads and
// stores through it are global_* instructions.  Kernel arguments are recognised as such by the
// compiler; pointers read from memory (a job table) are generic and would use flat_* ones.
template <typename T>
__device__ __forceinline__ __attribute__((address_space(1))) T* as_global(T* p) {
    return (__attribute__((address_space(1))) T*)(uintptr_t)p;
}

__device__ __forceinline__ uint32_t f2u(float f) { return __float_as_uint(f); }
__device__ __forceinline__ float u2f(uint32_t u) { return __uint_as_float(u); }

// ---------------------------------------------------------------- 16-bit float <-> fp32

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return u2f(h << 16); }

// fp32 -> bf16 bits, round to nearest even (v_cvt_pk_bf16_f32 on gfx950); NaN stays NaN.
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    __bf16 h = (__bf16)f;
    uint16_t b;
    __builtin_memcpy(&b, &h, 2);
    return b;
}

// two fp32 -> packed bf16 pair (lo in bits 0..15)
__device__ __forceinline__ uint32_t f32x2_to_bf16x2(float lo, float hi) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    f32x2 v = {lo, hi};
    bf16x2 h = __builtin_convertvector(v, bf16x2);
    uint32_t b;
    __builtin_memcpy(&b, &h, 4);
    return b;
}

// fp32 rounded to the nearest bf16 / fp16 value, as fp32
// (Converting the pair (0, f) would leave bf16(f) as an fp32 bit pattern in one instruction instead
// of two; kernels that are short of vector-ALU slots do that by hand.  As the general form it
// made no streaming kernel faster and raised the register count of the clip search kernel from
// 156 to 278, two wavefronts per SIMD fewer.)
__device__ __forceinline__ float round_to_bf16(float f) { return u2f(f32_to_bf16_bits(f) << 16); }

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
    _Float16 v;
    uint16_t b = (uint16_t)h;
    __builtin_memcpy(&v, &b, 2);
    return (float)v;
}

__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
    // The empty asm keeps the compiler from merging a preceding multiply into
    // v_fma_mixlo_f16 a, b, 0 -- the +0 addend would turn a -0.0 product into +0.0.
    asm volatile("" : "+v"(f));
    _Float16 v = (_Float16)f;  // v_cvt_f16_f32: IEEE round to nearest even
    uint16_t b;
    __builtin_memcpy(&b, &v, 2);
    return b;
}

// ---------------------------------------------------------------- chunk load / store by dtype
// A chunk is always presented to the math as 8 fp32 values.  `abs16` style tricks live in the
// kernels that need them; these helpers are the generic path.

template <int DT> struct Elem;
template <> struct Elem<MO_F32> { static constexpr int bytes = 4; };
template <> struct Elem<MO_F16> { static constexpr int bytes = 2; };
template <> struct Elem<MO_BF16> { static constexpr int bytes = 2; };

template <int DT>
__device__ __forceinline__ float load_elem(const void* p, int64_t i) {
    if constexpr (DT == MO_F32) return ((const float*)p)[i];
    else if constexpr (DT == MO_F16) return f16_bits_to_f32(((const uint16_t*)p)[i]);
    else return bf16_bits_to_f32(((const uint16_t*)p)[i]);
}

template <int DT>
__device__ __forceinline__ void store_elem(void* p, int64_t i, float v) {
    if constexpr (DT == MO_F32) ((float*)p)[i] = v;
    else if constexpr (DT == MO_F16) ((uint16_t*)p)[i] = (uint16_t)f32_to_f16_bits(v);
    else ((uint16_t*)p)[i] = (uint16_t)f32_to_bf16_bits(v);
}

// Aligned chunk (8 elements starting at element index i, i % 8 == 0, base 16-byte aligned).
template <int DT>
__device__ __forceinline__ void load_chunk(const void* p, int64_t i, float (&v)[8]) {
    if constexpr (DT == MO_F32) {
        const f32x4* q = (const f32x4*)((const float*)p + i);
        f32x4 a = __builtin_nontemporal_load(q), b = __builtin_nontemporal_load(q + 1);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
        v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
        u32x4 w = __builtin_nontemporal_load((const u32x4*)((const uint16_t*)p + i));
        uint32_t r[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if constexpr (DT == MO_BF16) {
                v[2 * j] = u2f(r[j] << 16);
                v[2 * j + 1] = u2f(r[j] & 0xFFFF0000u);
            } else {
                v[2 * j] = f16_bits_to_f32(r[j] & 0xFFFFu);
                v[2 * j + 1] = f16_bits_to_f32(r[j] >> 16);
            }
        }
    }
}

// The same load split in two, so that a kernel can issue the loads of several chunks before
// the first conversion has to wait for data: RawChunk holds the registers as loaded.
template <int DT> struct RawChunk { u32x4 a; };
template <> struct RawChunk<MO_F32> { u32x4 a, b; };

template <int DT>
__device__ __forceinline__ void load_raw(const void* p, int64_t i, RawChunk<DT>& r) {
    if constexpr (DT == MO_F32) {
        const u32x4* q = (const u32x4*)((const float*)p + i);
        r.a = __builtin_nontemporal_load(q);
        r.b = __builtin_nontemporal_load(q + 1);
    } else {
        r.a = __builtin_nontemporal_load((const u32x4*)((const uint16_t*)p + i));
    }
}

template <int DT>
__device__ __forceinline__ void zero_raw(RawChunk<DT>& r) {
    const u32x4 z = {0, 0, 0, 0};
    r.a = z;
    if constexpr (DT == MO_F32) r.b = z;
}

template <int DT>
__device__ __forceinline__ void unpack_raw(const RawChunk<DT>& r, float (&v)[8]) {
    if constexpr (DT == MO_F32) {
        v[0] = u2f(r.a.x); v[1] = u2f(r.a.y); v[2] = u2f(r.a.z); v[3] = u2f(r.a.w);
        v[4] = u2f(r.b.x); v[5] = u2f(r.b.y); v[6] = u2f(r.b.z); v[7] = u2f(r.b.w);
    } else {
        const uint32_t w[4] = {r.a.x, r.a.y, r.a.z, r.a.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if constexpr (DT == MO_BF16) {
                v[2 * j] = u2f(w[j] << 16);
                v[2 * j + 1] = u2f(w[j] & 0xFFFF0000u);
            } else {
                v[2 * j] = f16_bits_to_f32(w[j] & 0xFFFFu);
                v[2 * j + 1] = f16_bits_to_f32(w[j] >> 16);
            }
        }
    }
}

template <int DT>
__device__ __forceinline__ void store_chunk(void* p, int64_t i, const float (&v)[8]) {
    if constexpr (DT == MO_F32) {
        f32x4* q = (f32x4*)((float*)p + i);
        f32x4 a = {v[0], v[1], v[2], v[3]}, b = {v[4], v[5], v[6], v[7]};
        __builtin_nontemporal_store(a, q);
        __builtin_nontemporal_store(b, q + 1);
    } else {
        uint32_t r[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if constexpr (DT == MO_BF16)
                r[j] = f32x2_to_bf16x2(v[2 * j], v[2 * j + 1]);
            else
                r[j] = f32_to_f16_bits(v[2 * j]) | (f32_to_f16_bits(v[2 * j + 1]) << 16);
        }
        u32x4 w = {r[0], r[1], r[2], r[3]};
        __builtin_nontemporal_store(w, (u32x4*)((uint16_t*)p + i));
    }
}

// Guarded chunk: elements [i, i + 8) of a row of which only indices < limit exist; the rest
// read as +0 and are not written.
template <int DT>
__device__ __forceinline__ void load_chunk_guarded(const void* p, int64_t base, int64_t col,
                                                   int64_t limit, float (&v)[8]) {
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = (col + j < limit) ? load_elem<DT>(p, base + col + j) : 0.0f;
}

template <int DT>
__device__ __forceinline__ void store_chunk_guarded(void* p, int64_t base, int64_t col,
                                                    int64_t limit, const float (&v)[8]) {
#pragma unroll
    for (int j = 0; j < 8; ++j)
        if (col + j < limit) store_elem<DT>(p, base + col + j, v[j]);
}

// Scalar read of an amax / scale operand given in any of the three float dtypes.
__device__ __forceinline__ float load_scalar(const void* p, int dtype, int64_t i) {
    if (dtype == MO_F32) return ((const float*)p)[i];
    if (dtype == MO_F16) return f16_bits_to_f32(((const uint16_t*)p)[i]);
    return bf16_bits_to_f32(((const uint16_t*)p)[i]);
}

// ---------------------------------------------------------------- E4M3 (OCP e4m3fn)

// gfx950's FP8 converts implement OCP E4M3: v_cvt_pk_fp8_f32 rounds to nearest even, keeps
// subnormals and returns the NaN pattern 0x7F | sign for magnitudes that round above 448
// (i.e. > 464; the tie at 464 goes to 448), for infinities and for NaN -- on every non-NaN fp32 input the same byte as
// torch's CPU cast (a NaN input gives a NaN byte of unspecified sign).  v_cvt_f32_fp8 decodes
// every byte exactly (both NaN bytes to a quiet NaN).
typedef float f32pair __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float clamp448(float f) {
    f = f > 448.0f ? 448.0f : f;  // NaN fails both comparisons and stays NaN
    return f < -448.0f ? -448.0f : f;
}

// fp32 -> E4M3 byte.  With SAT the result saturates at +-448 instead of overflowing to NaN.
template <bool SAT = false>
__device__ __forceinline__ uint32_t f32_to_e4m3(float f) {
    if constexpr (SAT) f = clamp448(f);
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f, f, 0, false) & 0xFFu;
}

// two fp32 -> two E4M3 bytes in bits 0..15
template <bool SAT = false>
__device__ __forceinline__ uint32_t f32x2_to_e4m3x2(float a, float b) {
    if constexpr (SAT) { a = clamp448(a); b = clamp448(b); }
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false) & 0xFFFFu;
}

__device__ __forceinline__ float e4m3_to_f32(uint32_t b) {
    return __builtin_amdgcn_cvt_f32_fp8((int)b, 0);
}

// fp32 rounded to the E4M3 grid, returned as fp32
template <bool SAT = false>
__device__ __forceinline__ float round_e4m3(float f) {
    if constexpr (SAT) f = clamp448(f);
    return __builtin_amdgcn_cvt_f32_fp8(__builtin_amdgcn_cvt_pk_fp8_f32(f, f, 0, false), 0);
}

template <bool SAT = false>
__device__ __forceinline__ void round_e4m3_pair(float& a, float& b) {
    if constexpr (SAT) { a = clamp448(a); b = clamp448(b); }
    const f32pair p =
        __builtin_amdgcn_cvt_pk_f32_fp8(__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false), false);
    a = p.x;
    b = p.y;
}

// ---------------------------------------------------------------- E2M1 (FP4)

// fp32 -> 4-bit code = sign << 3 | ordinal, ties to the even code.  NaN and +-inf give
// ordinal 7; the sign bit is (v < 0), so -0.0 and NaN are unsigned.
__device__ __forceinline__ uint32_t f32_to_e2m1(float v) {
    float a = __builtin_fabsf(v);
    uint32_t c = (uint32_t)!(a <= 0.25f) + (uint32_t)!(a < 0.75f) + (uint32_t)!(a <= 1.25f) +
                 (uint32_t)!(a < 1.75f) + (uint32_t)!(a <= 2.5f) + (uint32_t)!(a < 3.5f) +
                 (uint32_t)!(a <= 5.0f);
    return c | ((v < 0.0f) ? 8u : 0u);
}

// 4-bit code -> fp32 value; code 8 decodes to +0.
__device__ __forceinline__ float e2m1_to_f32(uint32_t c) {
    uint32_t m = c & 7u;
    // 0, .5, 1, 1.5, 2, 3, 4, 6: ordinal m >= 2 is a normal number with exponent (m >> 1) - 1
    float mag = (m < 2u) ? 0.5f * (float)m
                         : u2f(((126u + (m >> 1)) << 23) | ((m & 1u) << 22));
    return (c & 8u) && m ? -mag : mag;
}

// ---------------------------------------------------------------- exact division by a shared divisor
// RN(x / s) from r = RN(1 / s) (one IEEE division shared by many x) and four FMAs:
//   q0 = RN(x * r)                        within 1.5 ulp of x / s
//   q1 = RN(q0 + RN(x - s * q0) * r)      faithful (the residual is exact in an FMA)
//   q  = RN(q1 + RN(x - s * q1) * r)      correctly rounded: a faithful quotient and a correctly
//                                         rounded reciprocal need one FMA correction (Markstein)
// Valid when nothing over- or underflows (callers check the range of s and of the quotient).
// A zero x gives +0 for either sign of x.
__device__ __forceinline__ float exact_quotient(float x, float s, float r) {
    const float q0 = x * r;
    const float q1 = __builtin_fmaf(__builtin_fmaf(-s, q0, x), r, q0);
    return __builtin_fmaf(__builtin_fmaf(-s, q1, x), r, q1);
}

// Placed at the top of a rarely taken block: an empty statement the optimiser may not move or
// run speculatively, so the block stays behind a branch (without it a cheap-looking block -- one
// fp32 division is ten instructions -- is evaluated on every pass and its result selected).
__device__ __forceinline__ void keep_branch() { asm volatile(""); }

// true when 2^-64 <= s <= 2^64 (normal, and far from the ends of the exponent range)
__device__ __forceinline__ bool mid_range(float s) {
    const uint32_t b = f2u(s);
    return b >= 0x1F800000u && b <= 0x5F800000u;
}

// Two fp32 values -> two E2M1 codes (hardware conversion: round to nearest even, saturating,
// sign from the sign bit) written to byte `sel` of `old`, first value in the low nibble.
__device__ __forceinline__ uint32_t fp4_pair(uint32_t old, float a, float b, int sel) {
    // v_cvt_scalef32_pk_fp4_f32: two fp32 -> two E2M1 codes written to byte `sel` of `old`
    switch (sel) {
        case 0: return __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(old, a, b, 1.0f, 0);
        case 1: return __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(old, a, b, 1.0f, 1);
        case 2: return __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(old, a, b, 1.0f, 2);
        default: return __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(old, a, b, 1.0f, 3);
    }
}

// ---------------------------------------------------------------- reductions

typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));

// max of two pairs of unsigned 16-bit values packed in a word (v_pk_max_u16)
__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
    u16x2 x, y;
    __builtin_memcpy(&x, &a, 4);
    __builtin_memcpy(&y, &b, 4);
    u16x2 r = __builtin_elementwise_max(x, y);
    uint32_t o;
    __builtin_memcpy(&o, &r, 4);
    return o;
}

// Max over aligned groups of 1 << lg adjacent lanes (lg <= 6), every lane of a group getting
// the result.  The steps up to 16 lanes are DPP moves (adjacent-lane swap, pair swap, mirror
// within 8, mirror within 16); wider groups finish with cross-row shuffles.
__device__ __forceinline__ uint32_t group_max_u32(uint32_t m, int lg) {
#define MO_DPP_MAX(CTRL)                                                              \
    {                                                                                 \
        const uint32_t t = (uint32_t)__builtin_amdgcn_mov_dpp((int)m, CTRL, 0xF, 0xF, true); \
        m = t > m ? t : m;                                                            \
    }
    if (lg >= 1) MO_DPP_MAX(0xB1)   // quad_perm [1, 0, 3, 2]
    if (lg >= 2) MO_DPP_MAX(0x4E)   // quad_perm [2, 3, 0, 1]
    if (lg >= 3) MO_DPP_MAX(0x141)  // row_half_mirror
    if (lg >= 4) MO_DPP_MAX(0x140)  // row_mirror
#undef MO_DPP_MAX
    for (int o = 16; o < (1 << lg); o <<= 1) {
        const uint32_t t = (uint32_t)__shfl_xor((int)m, o, kWave);
        m = t > m ? t : m;
    }
    return m;
}

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        uint32_t t = (uint32_t)__shfl_xor((int)v, o, kWave);
        v = t > v ? t : v;
    }
    return v;
}

// Block-wide max; result valid in thread 0.  `smem` holds one word per wave.
__device__ __forceinline__ uint32_t block_max_u32(uint32_t v, uint32_t* smem) {
    v = wave_max_u32(v);
    int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    if (lane == 0) smem[wave] = v;
    __syncthreads();
    if (wave == 0) {
        int nw = (blockDim.x + kWave - 1) / kWave;
        v = lane < nw ? smem[lane] : 0u;
        v = wave_max_u32(v);
    }
    return v;
}


// ---------------------------------------------------------------- one-launch amax -> quantize
// The fused kernels read their share of the tensor into registers, agree on the global abs-max
// and then quantise from the registers: the tensor is read once.  Each workgroup waits here for
// all the others, so the host launches no more workgroups than the device holds at the same time
// (resident_grid_limit).  It is an ordinary launch: hipLaunchCooperativeKernel adds about 15 us
// per call on this device, more than the second launch that the fusion saves.  Workgroups of
// other kernels that occupy the device only delay the exchange, because they end without help
// from this kernel; two of THESE kernels running side by side (or a device on which part of the
// compute units is masked off) could leave workgroups waiting for others that cannot start.  The
// wait is therefore bounded, and a workgroup whose wait expires computes the abs-max of the whole
// tensor by itself (workgroup_absmax_bits) and goes on: the outputs are the same bits either way,
// only later.
//
// ws: MO_FUSED_WS_BYTES of device memory, all zero before the first use; one word per 128-byte
// line, so that the atomics on different words do not queue behind each other:
//   line 0  workgroups that have delivered their maximum (back to 0 when the exchange is over)
//   line 1  running maximum, an abs-max bit pattern (back to 0 likewise)
//   line 2  64-bit {generation, result}: the last workgroup to arrive publishes the maximum
//           together with a generation one higher than the one every workgroup read on entry
//   line 3  set to 1 when a wait expired (information for the host: the call took the slow way;
//           no kernel reads it and the host clears it)
// EVERY workgroup of a launch delivers its maximum and counts itself before it waits, also one
// that gives up later, so the count reaches the grid size when the last workgroup of the launch
// has started, that one cleans lines 0 and 1 and publishes, and the workspace is in order again
// when the kernel ends -- whatever happened to the waits.
// Only these words cross workgroups and every access to them is a device-scope atomic performed
// at the memory side, so relaxed ordering is enough (a release / acquire pair would write back
// and invalidate caches on this multi-die part); program order between two atomics of a thread
// is kept by waiting for the value the first one returns.
// After `spin_limit` polls (one about every half microsecond) a workgroup sets the flag and
// returns false.  Calls that share a workspace must follow each other in one stream.
constexpr int kWsCount = 0, kWsMax = 32, kWsPublished = 64, kWsFail = 96;  // word offsets

__device__ __forceinline__ bool grid_max_exchange(uint32_t* ws, uint32_t local, uint32_t nwg,
                                                  uint32_t spin_limit, uint32_t* smem /* 8 words */,
                                                  uint32_t& global) {
    unsigned long long* published = (unsigned long long*)(ws + kWsPublished);
    unsigned long long entry = 0;
    if (threadIdx.x == 0)  // issued ahead of the reduction: the previous generation
        entry = __hip_atomic_load(published, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint32_t m = block_max_u32(local, smem);
    if (threadIdx.x == 0) {
        asm volatile("s_waitcnt vmcnt(0)" ::"v"(entry) : "memory");
        bool ok = true;
        uint32_t g = 0, old = 0;
        if (m) old = __hip_atomic_fetch_max(ws + kWsMax, m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::"v"(old) : "memory");
        const uint32_t before = __hip_atomic_fetch_add(ws + kWsCount, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (before + 1 == nwg) {
            // last to arrive: every maximum has been applied.  Clean up, then publish.
            g = __hip_atomic_load(ws + kWsMax, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            asm volatile("s_waitcnt vmcnt(0)" ::"v"(g) : "memory");
            const uint32_t c0 = __hip_atomic_exchange(ws + kWsCount, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const uint32_t m0 = __hip_atomic_exchange(ws + kWsMax, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            asm volatile("s_waitcnt vmcnt(0)" ::"v"(c0), "v"(m0) : "memory");
            const unsigned long long next = (((entry >> 32) + 1ull) << 32) | (unsigned long long)g;
            __hip_atomic_store(published, next, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
            uint32_t spins = 0;
            unsigned long long now;
            for (;;) {
                __builtin_amdgcn_s_sleep(16);
                now = __hip_atomic_load(published, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if ((now >> 32) != (entry >> 32)) break;
                if (spins++ >= spin_limit) { ok = false; break; }
            }
            g = (uint32_t)now;
            if (!ok) __hip_atomic_store(ws + kWsFail, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        smem[4] = g;
        smem[5] = ok ? 1u : 0u;
    }
    __syncthreads();
    global = smem[4];
    return smem[5] != 0u;
}

// Abs-max of `nbytes / 16` 16-byte units at x (fp32 words when WORDS32, else pairs of 16-bit
// floats), taken by ONE workgroup of 256 lanes that walks over all of them: the way out for a
// workgroup of a fused kernel whose wait for the others expired.  Returns the masked maximum in
// the packed form of the loads (fp32: the bit pattern; 16-bit: max of both halves in the low 16
// bits), the same in every lane.  `extra`: a lane's share of what the units do not cover, in the
// returned form.  `smem`: 8 words, free to reuse.
template <bool WORDS32>
__device__ __noinline__ uint32_t workgroup_absmax_bits(const void* x, int64_t units, uint32_t extra,
                                                       uint32_t* smem) {
    const uint4* p = (const uint4*)x;
    uint32_t m = 0;
    auto fold = [&](const uint4 v) {
        if constexpr (WORDS32) {
            const uint32_t a = v.x & 0x7FFFFFFFu, b = v.y & 0x7FFFFFFFu, c = v.z & 0x7FFFFFFFu,
                           d = v.w & 0x7FFFFFFFu;
            const uint32_t ab = a > b ? a : b, cd = c > d ? c : d;
            const uint32_t t = ab > cd ? ab : cd;
            m = t > m ? t : m;
        } else {
            m = pk_max_u16(m, pk_max_u16(pk_max_u16(v.x & 0x7FFF7FFFu, v.y & 0x7FFF7FFFu),
                                         pk_max_u16(v.z & 0x7FFF7FFFu, v.w & 0x7FFF7FFFu)));
        }
    };
    int64_t u = threadIdx.x;
    for (; u + 3 * 256 < units; u += 4 * 256) {
        const uint4 v0 = p[u], v1 = p[u + 256], v2 = p[u + 512], v3 = p[u + 768];
        fold(v0); fold(v1); fold(v2); fold(v3);
    }
    for (; u < units; u += 256) fold(p[u]);
    if constexpr (!WORDS32) m = (m & 0xFFFFu) > (m >> 16) ? (m & 0xFFFFu) : (m >> 16);
    m = extra > m ? extra : m;
    __syncthreads();  // smem is still being read by the caller's exchange
    m = block_max_u32(m, smem);
    if (threadIdx.x == 0) smem[6] = m;
    __syncthreads();
    return smem[6];
}

// How many workgroups of `kernel` (of `threads` lanes) the current device holds at the same time;
// cached by the caller; 0 on error.
template <typename K>
static int resident_grid_limit(K kernel, int threads) {
    int dev = 0, cus = 0, per_cu = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, 0) != hipSuccess)
        return 0;
    return cus * per_cu;
}

}  // namespace mo
