// Abs-max reductions (per tensor, per channel, per block) for gfx950.
//
// HBM-bound: 2 bytes (bf16/fp16) or 4 bytes (fp32) read per element, nothing written but the
// accumulator.  All variants fold |x| with integer max on the abs bit pattern so NaN
// propagates, and finish with one atomicMax per (row worker | column | block) into the fp32
// accumulator the caller owns.
#include "common.h"

#include <mutex>

namespace mo {

// Running max state of one lane.  16-bit inputs keep two packed 15-bit magnitudes per word.
// KEEP: plain loads instead of streaming ones, for a caller that reads the tensor again right
// away (the fake quant of a dynamic quantizer: MO_ABSMAX_REREAD).  The streaming hint takes the
// lines out of the memory-side cache under that second reader's feet: with plain loads abs-max
// + FP8 fake quant of a 33 MB tensor goes from 22.7 to 20.6 us and of a 134 MB one from 66 to
// 62 us (inputs that were not in any cache before).  The reduction itself is about 12 % slower
// that way, so passes nobody follows up on (calibration, the multi-tensor pass over a whole
// model's weights) keep the streaming loads.
template <int DT, bool KEEP = false> struct AbsAcc {
    uint32_t m = 0;
    static __device__ __forceinline__ u32x4 load(const u32x4* q) {
        if constexpr (KEEP) return *q;
        else return __builtin_nontemporal_load(q);
    }
    __device__ __forceinline__ void chunk(const void* p, int64_t i) {
        if constexpr (DT == MO_F32) {
            const u32x4* q = (const u32x4*)((const float*)p + i);
            u32x4 a = load(q), b = load(q + 1);
            uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int j = 0; j < 8; ++j) { uint32_t t = w[j] & 0x7FFFFFFFu; m = t > m ? t : m; }
        } else {
            u32x4 a = load((const u32x4*)((const uint16_t*)p + i));
            uint32_t t = pk_max_u16(pk_max_u16(a.x & 0x7FFF7FFFu, a.y & 0x7FFF7FFFu),
                                    pk_max_u16(a.z & 0x7FFF7FFFu, a.w & 0x7FFF7FFFu));
            m = pk_max_u16(m, t);
        }
    }
    // the same for a chunk loaded earlier
    __device__ __forceinline__ void raw(const RawChunk<DT>& r) {
        if constexpr (DT == MO_F32) {
            const uint32_t w[8] = {r.a.x, r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w};
#pragma unroll
            for (int j = 0; j < 8; ++j) { uint32_t t = w[j] & 0x7FFFFFFFu; m = t > m ? t : m; }
        } else {
            uint32_t t = pk_max_u16(pk_max_u16(r.a.x & 0x7FFF7FFFu, r.a.y & 0x7FFF7FFFu),
                                    pk_max_u16(r.a.z & 0x7FFF7FFFu, r.a.w & 0x7FFF7FFFu));
            m = pk_max_u16(m, t);
        }
    }
    __device__ __forceinline__ void elem(const void* p, int64_t i) {
        if constexpr (DT == MO_F32) {
            uint32_t t = ((const uint32_t*)p)[i] & 0x7FFFFFFFu;
            m = t > m ? t : m;
        } else {
            m = pk_max_u16(m, ((const uint16_t*)p)[i] & 0x7FFFu);
        }
    }
    // fp32 bit pattern of the lane's maximum
    __device__ __forceinline__ uint32_t bits() const {
        if constexpr (DT == MO_F32) return m;
        uint32_t h = (m & 0xFFFFu) > (m >> 16) ? (m & 0xFFFFu) : (m >> 16);
        if constexpr (DT == MO_BF16) return h << 16;
        return f2u(f16_bits_to_f32(h));
    }
};

// Fold v into the running maximum.  The accumulator only ever grows, so a plain (possibly stale)
// read that already shows a value >= v proves the atomic is unnecessary; thousands of
// workgroups hitting one address then cost a handful of atomics instead of one each.
__device__ __forceinline__ void fold_max(uint32_t* acc, uint32_t v) {
    if (v && v > __builtin_nontemporal_load(acc)) atomicMax(acc, v);
}

// The same with a device-coherent read, which never returns a value older than the last atomic
// but is itself served one request at a time per address: better when few workgroups share an
// accumulator (the multi-tensor launch), worse when thousands do.
__device__ __forceinline__ void fold_max_coherent(uint32_t* acc, uint32_t v) {
    if (v && v > __hip_atomic_load(acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
        atomicMax(acc, v);
}

// ------------------------------------------------------------------------------ per tensor
// One workgroup per tile of TILE_ELEMS elements, dispatched in order.
template <int DT, int TILE_ELEMS, bool KEEP = false>
__device__ __forceinline__ void absmax_flat_tile(const void* __restrict__ x, int64_t n, int64_t tile,
                                                 uint32_t* __restrict__ acc,
                                                 uint32_t* __restrict__ parts, uint32_t* smem) {
    constexpr int64_t kTileChunks = TILE_ELEMS / 8;
    AbsAcc<DT, KEEP> a;
    const int64_t chunks = n >> 3;
    const int64_t c0 = tile * kTileChunks;
    int64_t c1 = c0 + kTileChunks;
    if (c1 > chunks) c1 = chunks;
    int64_t c = c0 + threadIdx.x;
    for (; c + 768 < c1; c += 1024) {
        a.chunk(x, c << 3);
        a.chunk(x, (c + 256) << 3);
        a.chunk(x, (c + 512) << 3);
        a.chunk(x, (c + 768) << 3);
    }
    for (; c < c1; c += 256) a.chunk(x, c << 3);
    if (c1 == chunks && threadIdx.x < (n & 7)) a.elem(x, (chunks << 3) + threadIdx.x);
    const uint32_t v = block_max_u32(a.bits(), smem);
    if (threadIdx.x == 0) {
        fold_max(acc, v);
        if (parts) parts[tile] = v;   // the tile's own maximum, for callers that share a reduction
    }
}

template <int DT, int TILE_ELEMS, bool KEEP = false>
__global__ __launch_bounds__(256) void absmax_flat_kernel(const void* __restrict__ x, int64_t n,
                                                          uint32_t* __restrict__ acc,
                                                          uint32_t* __restrict__ parts = nullptr) {
    __shared__ uint32_t smem[4];
    absmax_flat_tile<DT, TILE_ELEMS, KEEP>(x, n, blockIdx.x, acc, parts, smem);
}

// Two tensors, each into its own accumulator, in one launch: workgroups [0, tiles0) take the
// tiles of the first, the others those of the second.
template <int DT, int TILE_ELEMS>
__global__ __launch_bounds__(256) void absmax_pair_kernel(const void* __restrict__ x0, int64_t n0,
                                                          uint32_t* __restrict__ acc0,
                                                          const void* __restrict__ x1, int64_t n1,
                                                          uint32_t* __restrict__ acc1, int tiles0) {
    __shared__ uint32_t smem[4];
    if ((int)blockIdx.x < tiles0) absmax_flat_tile<DT, TILE_ELEMS>(x0, n0, blockIdx.x, acc0, nullptr, smem);
    else absmax_flat_tile<DT, TILE_ELEMS>(x1, n1, (int)blockIdx.x - tiles0, acc1, nullptr, smem);
}

// ------------------------------------------------------------------------------ rows
// x viewed as [nrows, inner]; row r feeds acc[r % axis].  A row is handled by `L` adjacent
// lanes (power of two, <= 64) that stride over its chunks; gridDim.y splits long rows.
template <int DT, bool ALIGNED>
__global__ __launch_bounds__(256) void absmax_rows_kernel(const void* __restrict__ x,
                                                          int64_t nrows, int64_t inner,
                                                          int64_t axis, int lg_l, int64_t seg_chunks,
                                                          uint32_t* __restrict__ acc) {
    const int L = 1 << lg_l;
    const int sub = threadIdx.x & (L - 1);
    const int64_t workers = ((int64_t)gridDim.x * blockDim.x) >> lg_l;
    const int64_t row_chunks = (inner + 7) >> 3;
    const int64_t c0 = (int64_t)blockIdx.y * seg_chunks;
    int64_t c1 = c0 + seg_chunks;
    if (c1 > row_chunks) c1 = row_chunks;
    // every lane of a worker iterates the same number of rows, so the shuffles stay convergent
    for (int64_t r = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> lg_l; r < nrows;
         r += workers) {
        AbsAcc<DT> a;
        const int64_t base = r * inner;
        int64_t c = c0 + sub;
        if (ALIGNED && (inner & 7) == 0) {
            // whole chunks only: four loads of the lane in flight at a time
            for (; c + 3 * L < c1; c += 4 * L) {
                a.chunk(x, base + (c << 3));
                a.chunk(x, base + ((c + L) << 3));
                a.chunk(x, base + ((c + 2 * L) << 3));
                a.chunk(x, base + ((c + 3 * L) << 3));
            }
        }
        for (; c < c1; c += L) {
            const int64_t col = c << 3;
            if (ALIGNED && col + 8 <= inner) {
                a.chunk(x, base + col);
            } else {
                for (int j = 0; j < 8; ++j)
                    if (col + j < inner) a.elem(x, base + col + j);
            }
        }
        uint32_t v = a.bits();
        for (int o = L >> 1; o > 0; o >>= 1) {
            uint32_t t = (uint32_t)__shfl_xor((int)v, o, kWave);
            v = t > v ? t : v;
        }
        if (sub == 0) fold_max(acc + (r % axis), v);
    }
}

// Short aligned rows (inner % 8 == 0, inner / 8 a power of two <= 64): a row is exactly one chunk
// per lane of its group, so a wavefront load covers 64 / L whole rows of contiguous memory.
// One workgroup per tile of 1024 chunks, four chunks (of four different rows) per lane.  When
// `exclusive` (every accumulator element is fed by one row only) the fold is a plain
// read-modify-write instead of an atomic.
template <int DT>
__global__ __launch_bounds__(256) void absmax_short_rows_kernel(const void* __restrict__ x,
                                                                int64_t nrows, int64_t axis,
                                                                int lg_l, int exclusive,
                                                                uint32_t* __restrict__ acc) {
    const int64_t chunks = nrows << lg_l;
    const int64_t c0 = (int64_t)blockIdx.x * 1024 + threadIdx.x;
    RawChunk<DT> raw[4];
    uint32_t old[4] = {0, 0, 0, 0};
    // all loads first and in straight-line code (a chunk past the end re-reads the last one and
    // folds nothing): the four chunks, then -- for the plain read-modify-write of an accumulator
    // that one row feeds -- the four accumulator words, one round trip instead of one per round
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        int64_t c = c0 + u * 256;
        c = c < chunks ? c : chunks - 1;
        load_raw<DT>(x, c << 3, raw[u]);
    }
    if (exclusive) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            int64_t c = c0 + u * 256;
            c = c < chunks ? c : chunks - 1;
            old[u] = acc[c >> lg_l];
        }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int64_t c = c0 + u * 256;
        AbsAcc<DT> a;
        a.raw(raw[u]);
        const uint32_t v = group_max_u32(a.bits(), lg_l);
        if (c < chunks && (threadIdx.x & ((1 << lg_l) - 1)) == 0) {
            const int64_t r = c >> lg_l;
            if (exclusive) {
                if (v > old[u]) acc[r] = v;
            } else {
                fold_max(acc + r % axis, v);
            }
        }
    }
}

// ------------------------------------------------------------------------------ columns
// x viewed as [outer, axis] (inner == 1).  Vector path (axis % 8 == 0, aligned): a lane owns 8
// adjacent columns, a wavefront 512; the four wavefronts of a workgroup take interleaved rows of
// a slab, combine through LDS and fold once per column.  Scalar path: one column per lane.
// STAGED: instead of folding into acc[axis] with atomics, the workgroup of row slab blockIdx.y
// stores its maxima to row blockIdx.y of acc[gridDim.y, axis] with plain stores (a second pass
// reduces those rows).  With a fresh accumulator every workgroup of the first wave would
// otherwise issue one atomic per column, millions in total, served a few per cache line at a time.
template <int DT, bool STAGED>
__global__ __launch_bounds__(256) void absmax_cols8_kernel(const void* __restrict__ x,
                                                           int64_t outer, int64_t axis,
                                                           int64_t slab,
                                                           uint32_t* __restrict__ acc) {
    __shared__ uint32_t smem[4][512];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t col = ((int64_t)blockIdx.x * 64 + lane) * 8;
    const int64_t r0 = (int64_t)blockIdx.y * slab;
    int64_t r1 = r0 + slab;
    if (r1 > outer) r1 = outer;
    uint32_t m[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (col < axis) {
        if constexpr (DT == MO_F32) {
            for (int64_t r = r0 + wave; r < r1; r += 4) {
                const u32x4* q = (const u32x4*)((const float*)x + r * axis + col);
                u32x4 a = __builtin_nontemporal_load(q), b = __builtin_nontemporal_load(q + 1);
                uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
                for (int j = 0; j < 8; ++j) { uint32_t t = w[j] & 0x7FFFFFFFu; m[j] = t > m[j] ? t : m[j]; }
            }
        } else {
            uint32_t p[4] = {0, 0, 0, 0};  // packed pairs of columns
            int64_t r = r0 + wave;
            for (; r + 12 < r1; r += 16) {
                u32x4 a[4];
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    a[u] = __builtin_nontemporal_load(
                        (const u32x4*)((const uint16_t*)x + (r + 4 * u) * axis + col));
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    p[0] = pk_max_u16(p[0], a[u].x & 0x7FFF7FFFu);
                    p[1] = pk_max_u16(p[1], a[u].y & 0x7FFF7FFFu);
                    p[2] = pk_max_u16(p[2], a[u].z & 0x7FFF7FFFu);
                    p[3] = pk_max_u16(p[3], a[u].w & 0x7FFF7FFFu);
                }
            }
            for (; r < r1; r += 4) {
                u32x4 a = __builtin_nontemporal_load(
                    (const u32x4*)((const uint16_t*)x + r * axis + col));
                p[0] = pk_max_u16(p[0], a.x & 0x7FFF7FFFu);
                p[1] = pk_max_u16(p[1], a.y & 0x7FFF7FFFu);
                p[2] = pk_max_u16(p[2], a.z & 0x7FFF7FFFu);
                p[3] = pk_max_u16(p[3], a.w & 0x7FFF7FFFu);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                uint32_t lo = p[j] & 0xFFFFu, hi = p[j] >> 16;
                m[2 * j] = DT == MO_BF16 ? lo << 16 : f2u(f16_bits_to_f32(lo));
                m[2 * j + 1] = DT == MO_BF16 ? hi << 16 : f2u(f16_bits_to_f32(hi));
            }
        }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) smem[wave][lane * 8 + j] = m[j];
    __syncthreads();
    for (int t = threadIdx.x; t < 512; t += 256) {
        const int64_t c = (int64_t)blockIdx.x * 512 + t;
        if (c < axis) {
            uint32_t v = smem[0][t];
            v = smem[1][t] > v ? smem[1][t] : v;
            v = smem[2][t] > v ? smem[2][t] : v;
            v = smem[3][t] > v ? smem[3][t] : v;
            if constexpr (STAGED) acc[(int64_t)blockIdx.y * axis + c] = v;
            else fold_max(acc + c, v);
        }
    }
}

// Wide variant for axis >= 2048: a workgroup spans 2048 adjacent columns (4 KiB of a bf16 row per
// load instruction round), every lane keeps its 8 columns for the whole slab of rows -- no LDS.
template <int DT, bool STAGED>
__global__ __launch_bounds__(256) void absmax_cols8_wide_kernel(const void* __restrict__ x,
                                                                int64_t outer, int64_t axis,
                                                                int64_t slab,
                                                                uint32_t* __restrict__ acc) {
    const int64_t col = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
    if (col >= axis) return;
    const int64_t r0 = (int64_t)blockIdx.y * slab;
    int64_t r1 = r0 + slab;
    if (r1 > outer) r1 = outer;
    uint32_t m[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if constexpr (DT == MO_F32) {
        int64_t r = r0;
        for (; r + 1 < r1; r += 2) {
            const u32x4* q0 = (const u32x4*)((const float*)x + r * axis + col);
            const u32x4* q1 = (const u32x4*)((const float*)x + (r + 1) * axis + col);
            const u32x4 a = __builtin_nontemporal_load(q0), b = __builtin_nontemporal_load(q0 + 1);
            const u32x4 c = __builtin_nontemporal_load(q1), d = __builtin_nontemporal_load(q1 + 1);
            const uint32_t w[16] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w,
                                    c.x, c.y, c.z, c.w, d.x, d.y, d.z, d.w};
#pragma unroll
            for (int j = 0; j < 16; ++j) { const uint32_t t = w[j] & 0x7FFFFFFFu; m[j & 7] = t > m[j & 7] ? t : m[j & 7]; }
        }
        for (; r < r1; ++r) {
            const u32x4* q = (const u32x4*)((const float*)x + r * axis + col);
            const u32x4 a = __builtin_nontemporal_load(q), b = __builtin_nontemporal_load(q + 1);
            const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int j = 0; j < 8; ++j) { const uint32_t t = w[j] & 0x7FFFFFFFu; m[j] = t > m[j] ? t : m[j]; }
        }
    } else {
        uint32_t p[4] = {0, 0, 0, 0};  // packed pairs of columns
        int64_t r = r0;
        for (; r + 3 < r1; r += 4) {
            u32x4 a[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                a[u] = __builtin_nontemporal_load(
                    (const u32x4*)((const uint16_t*)x + (r + u) * axis + col));
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                p[0] = pk_max_u16(p[0], a[u].x & 0x7FFF7FFFu);
                p[1] = pk_max_u16(p[1], a[u].y & 0x7FFF7FFFu);
                p[2] = pk_max_u16(p[2], a[u].z & 0x7FFF7FFFu);
                p[3] = pk_max_u16(p[3], a[u].w & 0x7FFF7FFFu);
            }
        }
        for (; r < r1; ++r) {
            const u32x4 a = __builtin_nontemporal_load(
                (const u32x4*)((const uint16_t*)x + r * axis + col));
            p[0] = pk_max_u16(p[0], a.x & 0x7FFF7FFFu);
            p[1] = pk_max_u16(p[1], a.y & 0x7FFF7FFFu);
            p[2] = pk_max_u16(p[2], a.z & 0x7FFF7FFFu);
            p[3] = pk_max_u16(p[3], a.w & 0x7FFF7FFFu);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t lo = p[j] & 0xFFFFu, hi = p[j] >> 16;
            m[2 * j] = DT == MO_BF16 ? lo << 16 : f2u(f16_bits_to_f32(lo));
            m[2 * j + 1] = DT == MO_BF16 ? hi << 16 : f2u(f16_bits_to_f32(hi));
        }
    }
    if constexpr (STAGED) {
        u32x4* dst = (u32x4*)(acc + (int64_t)blockIdx.y * axis + col);
        const u32x4 lo = {m[0], m[1], m[2], m[3]}, hi = {m[4], m[5], m[6], m[7]};
        dst[0] = lo;
        dst[1] = hi;
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) fold_max(acc + col + j, m[j]);
    }
}

template <int DT>
__global__ __launch_bounds__(256) void absmax_cols1_kernel(const void* __restrict__ x,
                                                           int64_t outer, int64_t axis,
                                                           int64_t slab,
                                                           uint32_t* __restrict__ acc) {
    const int64_t col = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (col >= axis) return;
    const int64_t r0 = (int64_t)blockIdx.y * slab;
    int64_t r1 = r0 + slab;
    if (r1 > outer) r1 = outer;
    AbsAcc<DT> a;
    for (int64_t r = r0; r < r1; ++r) a.elem(x, r * axis + col);
    fold_max(acc + col, a.bits());
}

// ------------------------------------------------------------------------------ many tensors
template <int DT>
__global__ __launch_bounds__(256) void absmax_multi_kernel(const mo_absmax_job* __restrict__ jobs,
                                                           int njobs,
                                                           const int32_t* __restrict__ tile_job) {
    __shared__ uint32_t smem[4];
    constexpr int64_t kTileChunks = MO_ABSMAX_TILE_ELEMS / 8;
    const int64_t t = blockIdx.x;  // one workgroup per tile, dispatched in tile order
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
    const mo_absmax_job jb = jobs[lo];
    const int64_t chunks = jb.elems >> 3;
    const int64_t c0 = (t - jb.tile_begin) * kTileChunks;
    int64_t c1 = c0 + kTileChunks;
    if (c1 > chunks) c1 = chunks;
    AbsAcc<DT> a;
    int64_t c = c0 + threadIdx.x;
    for (; c + 768 < c1; c += 1024) {
        a.chunk(jb.x, c << 3);
        a.chunk(jb.x, (c + 256) << 3);
        a.chunk(jb.x, (c + 512) << 3);
        a.chunk(jb.x, (c + 768) << 3);
    }
    for (; c < c1; c += 256) a.chunk(jb.x, c << 3);
    if (c1 == chunks && threadIdx.x < (jb.elems & 7)) a.elem(jb.x, (chunks << 3) + threadIdx.x);
    const uint32_t v = block_max_u32(a.bits(), smem);
    if (threadIdx.x == 0) fold_max_coherent((uint32_t*)jb.acc, v);
}

template <int DT>
static int launch_absmax(const void* x, int64_t outer, int64_t axis, int64_t inner, uint32_t* acc,
                         hipStream_t s, bool keep = false) {
    const bool base_ok = ((uintptr_t)x & 15u) == 0;
    if (axis == 1) {  // per tensor
        const int64_t n = outer * inner;
        if (base_ok) {
            // 32768-element tiles under the occupancy cap.  Smaller tiles without the cap read a
            // 67 MB tensor 6 % faster into a warm accumulator, but with a fresh one (dynamic
            // quantisation, the first batch of a calibration) twice as many workgroups meet at the
            // accumulator's atomic and the launch and its successor lose 10 us.
            const int64_t tile = mo::tuned("absmax_flat_tile", 32768);
            const int64_t tiles = (n + tile - 1) / tile;
            if (tiles > 0x7FFFFFFF) return MO_ERR_UNSUPPORTED;
            const size_t cap = mo::ballast_bytes("absmax_flat_kernel", 36);
            if (keep) absmax_flat_kernel<DT, 32768, true><<<dim3((unsigned)((n + 32767) / 32768)), 256, cap, s>>>(x, n, acc);
            else if (tile == 8192) absmax_flat_kernel<DT, 8192><<<dim3((unsigned)tiles), 256, cap, s>>>(x, n, acc);
            else if (tile == 16384) absmax_flat_kernel<DT, 16384><<<dim3((unsigned)tiles), 256, cap, s>>>(x, n, acc);
            else absmax_flat_kernel<DT, 32768><<<dim3((unsigned)tiles), 256, cap, s>>>(x, n, acc);
            return MO_OK;
        }
        outer = 1; inner = n;  // unaligned base: guarded row path below
    }
    if (inner == 1) {  // per column
        const bool vec = base_ok && (axis % 8 == 0);
        const int64_t gx = vec ? (axis + 511) / 512 : (axis + 255) / 256;
        // enough row slabs to fill the chip, each at least 16 rows (a multiple of 4)
        int64_t gy = (4096 + gx - 1) / gx;
        int64_t slab = (outer + gy - 1) / gy;
        if (slab < 16) slab = 16;
        slab = (slab + 3) / 4 * 4;
        gy = (outer + slab - 1) / slab;
        if (gy > 65535) { gy = 65535; slab = ((outer + gy - 1) / gy + 3) / 4 * 4; gy = (outer + slab - 1) / slab; }
        if (vec && axis >= 2048) {
            const int64_t wx = (axis + 2047) / 2048;
            int64_t wy = (2048 + wx - 1) / wx;
            int64_t ws = (outer + wy - 1) / wy;
            if (ws < 16) ws = 16;
            wy = (outer + ws - 1) / ws;
            if (wy > 65535) { wy = 65535; ws = (outer + wy - 1) / wy; wy = (outer + ws - 1) / ws; }
            absmax_cols8_wide_kernel<DT, false><<<dim3((unsigned)wx, (unsigned)wy), 256, mo::ballast_bytes("absmax_cols8_wide_kernel", 0), s>>>(x, outer, axis, ws, acc);
        } else if (vec)
            absmax_cols8_kernel<DT, false><<<dim3((unsigned)gx, (unsigned)gy), 256, mo::ballast_bytes("absmax_cols8_kernel", 0), s>>>(x, outer, axis, slab, acc);
        else
            absmax_cols1_kernel<DT><<<dim3((unsigned)gx, (unsigned)gy), 256, 0, s>>>(x, outer, axis, slab, acc);
        return MO_OK;
    }
    // rows of length `inner`
    const int64_t nrows = outer * axis;
    const int64_t row_chunks = (inner + 7) >> 3;
    if (base_ok && inner % 8 == 0 && row_chunks <= 64 && (row_chunks & (row_chunks - 1)) == 0) {
        int lg_l = 0;
        while ((int64_t(1) << lg_l) < row_chunks) ++lg_l;
        const int64_t tiles = (nrows * row_chunks + 1023) / 1024;
        if (tiles <= 0x7FFFFFFF) {
            absmax_short_rows_kernel<DT><<<dim3((unsigned)tiles), 256, mo::ballast_bytes("absmax_short_rows_kernel", 0), s>>>(
                x, nrows, axis, lg_l, outer == 1 ? 1 : 0, acc);
            return MO_OK;
        }
    }
    int lg = 0;
    while ((1 << lg) < 64 && (int64_t(1) << lg) < row_chunks) ++lg;
    const int64_t workers_per_block = 256 >> lg;
    int64_t gx = (nrows + workers_per_block - 1) / workers_per_block;
    if (gx > 4096) gx = 4096;
    // split long rows when there are too few rows to fill the chip
    int64_t gy = 1;
    const int64_t per_worker_chunks = row_chunks >> lg;
    if (gx < 1024 && per_worker_chunks > 16) {
        gy = 1024 / gx;
        if (gy > per_worker_chunks / 8) gy = per_worker_chunks / 8;
        if (gy < 1) gy = 1;
        if (gy > 65535) gy = 65535;
    }
    int64_t seg = (row_chunks + gy - 1) / gy;
    seg = ((seg + (1 << lg) - 1) >> lg) << lg;  // whole strides per segment
    gy = (row_chunks + seg - 1) / seg;
    const bool aligned = base_ok && (inner % 8 == 0);
    if (aligned)
        absmax_rows_kernel<DT, true><<<dim3((unsigned)gx, (unsigned)gy), 256, mo::ballast_bytes("absmax_rows_kernel", 0), s>>>(x, nrows, inner, axis, lg, seg, acc);
    else
        absmax_rows_kernel<DT, false><<<dim3((unsigned)gx, (unsigned)gy), 256, mo::ballast_bytes("absmax_rows_kernel", 0), s>>>(x, nrows, inner, axis, lg, seg, acc);
    return MO_OK;
}

// Second pass of the staged per-column reduction: acc[c] = max(acc[c], max over rows of
// partial[r, c]).  A workgroup owns 32 columns (eight lanes-groups take interleaved rows, then
// combine through LDS), so the accumulator is updated by plain stores from its only writer.
__global__ __launch_bounds__(256) void absmax_fold_partials_kernel(
    const uint32_t* __restrict__ partial, int64_t rows, int64_t axis, uint32_t* __restrict__ acc) {
    __shared__ uint32_t smem[8][32];
    const int c = threadIdx.x & 31, g = threadIdx.x >> 5;
    const int64_t col = (int64_t)blockIdx.x * 32 + c;
    uint32_t m = 0;
    if (col < axis) {
        int64_t r = g;
        for (; r + 24 < rows; r += 32) {
            uint32_t v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = partial[(r + 8 * u) * axis + col];
#pragma unroll
            for (int u = 0; u < 4; ++u) m = v[u] > m ? v[u] : m;
        }
        for (; r < rows; r += 8) {
            const uint32_t v = partial[r * axis + col];
            m = v > m ? v : m;
        }
    }
    smem[g][c] = m;
    __syncthreads();
    if (g == 0 && col < axis) {
#pragma unroll
        for (int k = 1; k < 8; ++k) m = smem[k][c] > m ? smem[k][c] : m;
        const uint32_t old = acc[col];
        if (m > old) acc[col] = m;
    }
}

// Per-column abs-max in two passes: row slabs -> partial[slabs, axis] (plain stores), then the
// columns of that small matrix into acc.  No atomics.
template <int DT>
static int launch_absmax_cols_staged(const void* x, int64_t outer, int64_t axis, uint32_t* acc,
                                     uint32_t* partial, int64_t partial_rows, hipStream_t s) {
    if ((((uintptr_t)x | (uintptr_t)partial) & 15u) || (axis % 8)) return MO_ERR_UNSUPPORTED;
    int64_t slabs = partial_rows < 65535 ? partial_rows : 65535;
    int64_t rows = (outer + slabs - 1) / slabs;
    rows = (rows + 3) / 4 * 4;  // the 16-bit paths take rows in groups of four
    slabs = (outer + rows - 1) / rows;
    if (axis >= 2048) {
        const int64_t wx = (axis + 2047) / 2048;
        absmax_cols8_wide_kernel<DT, true><<<dim3((unsigned)wx, (unsigned)slabs), 256, mo::ballast_bytes("absmax_cols8_wide_kernel", 0), s>>>(
            x, outer, axis, rows, partial);
    } else {
        const int64_t gx = (axis + 511) / 512;
        absmax_cols8_kernel<DT, true><<<dim3((unsigned)gx, (unsigned)slabs), 256, mo::ballast_bytes("absmax_cols8_kernel", 0), s>>>(
            x, outer, axis, rows, partial);
    }
    absmax_fold_partials_kernel<<<dim3((unsigned)((axis + 31) / 32)), 256, 0, s>>>(partial, slabs, axis, acc);
    return MO_OK;
}

// Workspace of the entry point that may not allocate: row-slab maxima of the staged per-column
// reduction.  One copy per GPU, held until the process ends.  In host code the array's name is
// only a handle for hipGetSymbolAddress; kernels are given the address that call returns.
static __device__ __align__(256) uint32_t scratch[MO_ABSMAX_COLS_NOALLOC_WORDS];

constexpr int kMaxDevices = 64;
static uint32_t* g_scratch_ptr[kMaxDevices] = {nullptr};
static std::mutex g_scratch_mutex;

// Device address of `scratch` on the current device (looked up once per device).
static int scratch_address(uint32_t** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return MO_ERR_LAUNCH;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        uint32_t* ptr = nullptr;
        if (hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr)
            return MO_ERR_LAUNCH;
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return MO_OK;
}


// ---------------------------------------------------------------- two-dimensional blocks
// acc[b] = max(acc[b], abs-max of tile b) for x viewed as [rows, cols] cut into tiles of
// block_rows x block_cols elements, b = (row / block_rows) * (cols / block_cols) + col /
// block_cols: one workgroup per tile (a 128 x 128 tile is 32 KB of bf16), no atomics.
template <int DT>
__global__ __launch_bounds__(256) void absmax_blocks2d_kernel(const void* __restrict__ x, int64_t cols,
                                                              uint32_t block_rows, uint32_t block_chunks,
                                                              uint32_t blocks_across,
                                                              uint32_t* __restrict__ acc) {
    __shared__ uint32_t smem[8];
    const int64_t tile_row = blockIdx.x / blocks_across;
    const uint32_t across = blockIdx.x - (uint32_t)tile_row * blocks_across;
    const int64_t base = tile_row * block_rows * cols + (int64_t)across * block_chunks * 8;
    const uint32_t total = block_rows * block_chunks;   // 16-byte (fp32: 32-byte) chunks of the tile
    AbsAcc<DT> a;
    uint32_t q = threadIdx.x;
    for (; q + 768 < total; q += 1024) {   // four loads of a lane in flight
        RawChunk<DT> raw[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t qq = q + u * 256, r = qq / block_chunks;
            load_raw<DT>(x, base + (int64_t)r * cols + (int64_t)(qq - r * block_chunks) * 8, raw[u]);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) a.raw(raw[u]);
    }
    for (; q < total; q += 256) {
        const uint32_t r = q / block_chunks;
        a.chunk(x, base + (int64_t)r * cols + (int64_t)(q - r * block_chunks) * 8);
    }
    const uint32_t m = block_max_u32(a.bits(), smem);
    if (threadIdx.x == 0) {
        const uint32_t old = acc[blockIdx.x];
        acc[blockIdx.x] = m > old ? m : old;
    }
}

// ---------------------------------------------------------------- value ranges of small tensors
// The smallest and the largest element of each of up to kRangeJobs tensors, and whether it holds
// a NaN, one launch for all of them: a workgroup per 4096-element chunk of a tensor, three floats
// per chunk for the host to fold.  The tensors are calibrated amax and scale buffers (a scalar
// to a few hundred thousand values each), whose "finite, not negative" checks the host wants
// answered with a single synchronisation.
constexpr int kRangeJobs = 32;
constexpr int kRangeChunk = 4096;
struct RangeJobs {
    const void* ptr[kRangeJobs];
    int64_t count[kRangeJobs];
    int dtype[kRangeJobs];
    int first[kRangeJobs + 1];   // first workgroup of each tensor; first[n] = the grid
};

__global__ __launch_bounds__(256) void value_ranges_kernel(RangeJobs jobs, int n, float* __restrict__ out) {
    int job = 0;
    while (job + 1 < n && (int)blockIdx.x >= jobs.first[job + 1]) ++job;
    const void* p = jobs.ptr[job];
    const int dt = jobs.dtype[job];
    const int64_t begin = (int64_t)((int)blockIdx.x - jobs.first[job]) * kRangeChunk;
    const int64_t left = jobs.count[job] - begin;
    const int here = left < kRangeChunk ? (int)left : kRangeChunk;
    float lo = __builtin_inff(), hi = -__builtin_inff();
    bool nan = false;
#pragma unroll
    for (int u = 0; u < kRangeChunk / 256; ++u) {
        const int i = u * 256 + (int)threadIdx.x;
        if (i < here) {
            const float v = dt == MO_F32 ? load_elem<MO_F32>(p, begin + i)
                            : dt == MO_F16 ? load_elem<MO_F16>(p, begin + i) : load_elem<MO_BF16>(p, begin + i);
            nan |= v != v;
            lo = __builtin_fminf(lo, v);   // a NaN operand is ignored: it is carried by the flag
            hi = __builtin_fmaxf(hi, v);
        }
    }
    __shared__ float slo[4], shi[4];
    __shared__ int snan[4];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        lo = __builtin_fminf(lo, __shfl_xor(lo, o, kWave));
        hi = __builtin_fmaxf(hi, __shfl_xor(hi, o, kWave));
        nan |= (bool)__shfl_xor((int)nan, o, kWave);
    }
    if ((threadIdx.x & 63) == 0) {
        slo[threadIdx.x >> 6] = lo;
        shi[threadIdx.x >> 6] = hi;
        snan[threadIdx.x >> 6] = nan;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 1; w < 4; ++w) {
            lo = __builtin_fminf(lo, slo[w]);
            hi = __builtin_fmaxf(hi, shi[w]);
            nan |= snan[w] != 0;
        }
        out[3 * blockIdx.x] = lo;
        out[3 * blockIdx.x + 1] = hi;
        out[3 * blockIdx.x + 2] = nan ? 1.0f : 0.0f;
    }
}

}  // namespace mo

extern "C" int mo_absmax_hinted(const void* x, int64_t outer, int64_t axis, int64_t inner, int dtype,
                                float* acc, unsigned hints, void* stream) {
    if (outer < 0 || axis < 0 || inner < 0 || (hints & ~(unsigned)MO_ABSMAX_REREAD)) return MO_ERR_ARG;
    if (outer == 0 || axis == 0 || inner == 0) return MO_OK;
    if (!x || !acc) return MO_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    const bool keep = (hints & MO_ABSMAX_REREAD) != 0;
    int rc;
    switch (dtype) {
        case MO_F32: rc = mo::launch_absmax<MO_F32>(x, outer, axis, inner, (uint32_t*)acc, s, keep); break;
        case MO_F16: rc = mo::launch_absmax<MO_F16>(x, outer, axis, inner, (uint32_t*)acc, s, keep); break;
        case MO_BF16: rc = mo::launch_absmax<MO_BF16>(x, outer, axis, inner, (uint32_t*)acc, s, keep); break;
        default: return MO_ERR_DTYPE;
    }
    if (rc != MO_OK) return rc;
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_absmax(const void* x, int64_t outer, int64_t axis, int64_t inner, int dtype,
                         float* acc, void* stream) {
    return mo_absmax_hinted(x, outer, axis, inner, dtype, acc, 0u, stream);
}

extern "C" int mo_absmax_pair(const void* x0, int64_t n0, float* acc0, const void* x1, int64_t n1,
                              float* acc1, int dtype, void* stream) {
    if (n0 < 0 || n1 < 0) return MO_ERR_ARG;
    if (dtype < MO_F32 || dtype > MO_BF16) return MO_ERR_DTYPE;
    if ((n0 && (!x0 || !acc0)) || (n1 && (!x1 || !acc1))) return MO_ERR_ARG;
    if (n0 == 0 && n1 == 0) return MO_OK;
    if ((((uintptr_t)x0 | (uintptr_t)x1) & 15u)) return MO_ERR_UNSUPPORTED;
    // 8192-element tiles: the pair is for small tensors (K and V of one batch), which a larger
    // tile would spread over too few compute units
    constexpr int64_t kTile = 8192;
    const int64_t t0 = (n0 + kTile - 1) / kTile, t1 = (n1 + kTile - 1) / kTile;
    if (t0 + t1 > 0x7FFFFFFF) return MO_ERR_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((unsigned)(t0 + t1));
    switch (dtype) {
        case MO_F32: mo::absmax_pair_kernel<MO_F32, kTile><<<grid, 256, 0, s>>>(x0, n0, (uint32_t*)acc0, x1, n1, (uint32_t*)acc1, (int)t0); break;
        case MO_F16: mo::absmax_pair_kernel<MO_F16, kTile><<<grid, 256, 0, s>>>(x0, n0, (uint32_t*)acc0, x1, n1, (uint32_t*)acc1, (int)t0); break;
        default: mo::absmax_pair_kernel<MO_BF16, kTile><<<grid, 256, 0, s>>>(x0, n0, (uint32_t*)acc0, x1, n1, (uint32_t*)acc1, (int)t0); break;
    }
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_absmax_tensor_parts(const void* x, int64_t n, int dtype, float* acc,
                                      uint32_t* parts, int64_t parts_capacity,
                                      int64_t* parts_written, void* stream) {
    if (n < 0 || parts_capacity < 0 || !parts_written) return MO_ERR_ARG;
    *parts_written = 0;
    if (n == 0) return MO_OK;
    if (!x || !acc || !parts) return MO_ERR_ARG;
    if (((uintptr_t)x & 15u) || ((uintptr_t)parts & 3u)) return MO_ERR_UNSUPPORTED;
    constexpr int64_t kTile = 32768;
    const int64_t tiles = (n + kTile - 1) / kTile;
    if (tiles > parts_capacity) return MO_ERR_TOO_LARGE;
    if (tiles > 0x7FFFFFFF) return MO_ERR_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
    const size_t cap = mo::ballast_bytes("absmax_flat_kernel", 36);
    switch (dtype) {
        case MO_F32: mo::absmax_flat_kernel<MO_F32, kTile><<<dim3((unsigned)tiles), 256, cap, s>>>(x, n, (uint32_t*)acc, parts); break;
        case MO_F16: mo::absmax_flat_kernel<MO_F16, kTile><<<dim3((unsigned)tiles), 256, cap, s>>>(x, n, (uint32_t*)acc, parts); break;
        case MO_BF16: mo::absmax_flat_kernel<MO_BF16, kTile><<<dim3((unsigned)tiles), 256, cap, s>>>(x, n, (uint32_t*)acc, parts); break;
        default: return MO_ERR_DTYPE;
    }
    *parts_written = tiles;
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_absmax_multi(const mo_absmax_job* jobs_dev, int njobs,
                               const int32_t* tile_job_dev, int64_t total_tiles, int dtype,
                               void* stream) {
    if (njobs < 0 || total_tiles < 0 || total_tiles > 0x7FFFFFFF) return MO_ERR_ARG;
    if (njobs == 0 || total_tiles == 0) return MO_OK;
    if (!jobs_dev) return MO_ERR_ARG;
    const unsigned grid = (unsigned)total_tiles;
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case MO_F32: mo::absmax_multi_kernel<MO_F32><<<grid, 256, mo::ballast_bytes("absmax_multi_kernel", 0), s>>>(jobs_dev, njobs, tile_job_dev); break;
        case MO_F16: mo::absmax_multi_kernel<MO_F16><<<grid, 256, mo::ballast_bytes("absmax_multi_kernel", 0), s>>>(jobs_dev, njobs, tile_job_dev); break;
        case MO_BF16: mo::absmax_multi_kernel<MO_BF16><<<grid, 256, mo::ballast_bytes("absmax_multi_kernel", 0), s>>>(jobs_dev, njobs, tile_job_dev); break;
        default: return MO_ERR_DTYPE;
    }
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_absmax_cols_staged(const void* x, int64_t outer, int64_t axis, int dtype,
                                     float* acc, void* partial, int64_t partial_rows,
                                     void* stream) {
    if (outer < 0 || axis < 0 || partial_rows < 1) return MO_ERR_ARG;
    if (outer == 0 || axis == 0) return MO_OK;
    if (!x || !acc || !partial) return MO_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    int rc;
    switch (dtype) {
        case MO_F32: rc = mo::launch_absmax_cols_staged<MO_F32>(x, outer, axis, (uint32_t*)acc, (uint32_t*)partial, partial_rows, s); break;
        case MO_F16: rc = mo::launch_absmax_cols_staged<MO_F16>(x, outer, axis, (uint32_t*)acc, (uint32_t*)partial, partial_rows, s); break;
        case MO_BF16: rc = mo::launch_absmax_cols_staged<MO_BF16>(x, outer, axis, (uint32_t*)acc, (uint32_t*)partial, partial_rows, s); break;
        default: return MO_ERR_DTYPE;
    }
    if (rc != MO_OK) return rc;
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_absmax_cols_noalloc(const void* x, int64_t outer, int64_t axis, int dtype,
                                      float* acc, void* stream) {
    if (outer < 0 || axis < 0) return MO_ERR_ARG;
    if (outer == 0 || axis == 0) return MO_OK;
    if (!x || !acc) return MO_ERR_ARG;
    if (axis > MO_ABSMAX_COLS_NOALLOC_WORDS) return MO_ERR_TOO_LARGE;
    // as many row slabs as fit the fixed workspace, up to what fills the chip
    int64_t slabs = MO_ABSMAX_COLS_NOALLOC_WORDS / axis;
    if (slabs > 256) slabs = 256;
    uint32_t* partial = nullptr;
    int rc = mo::scratch_address(&partial);
    if (rc != MO_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case MO_F32: rc = mo::launch_absmax_cols_staged<MO_F32>(x, outer, axis, (uint32_t*)acc, partial, slabs, s); break;
        case MO_F16: rc = mo::launch_absmax_cols_staged<MO_F16>(x, outer, axis, (uint32_t*)acc, partial, slabs, s); break;
        case MO_BF16: rc = mo::launch_absmax_cols_staged<MO_BF16>(x, outer, axis, (uint32_t*)acc, partial, slabs, s); break;
        default: return MO_ERR_DTYPE;
    }
    if (rc != MO_OK) return rc;
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_absmax_blocks2d(const void* x, int64_t rows, int64_t cols, int64_t block_rows,
                                  int64_t block_cols, int dtype, float* acc, void* stream) {
    if (rows < 0 || cols < 0 || block_rows <= 0 || block_cols <= 0) return MO_ERR_ARG;
    if (dtype < MO_F32 || dtype > MO_BF16) return MO_ERR_DTYPE;
    if (rows == 0 || cols == 0) return MO_OK;
    if (!x || !acc) return MO_ERR_ARG;
    const int64_t tiles = (rows / block_rows) * (cols / block_cols);
    if (rows % block_rows || cols % block_cols || block_cols % 8 || ((uintptr_t)x & 15u) ||
        tiles > 0x7FFFFFFF || block_rows * (block_cols / 8) > 0x7FFFFFFF)
        return MO_ERR_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
#define CALL(DT)                                                                               \
    mo::absmax_blocks2d_kernel<DT><<<dim3((unsigned)tiles), 256, 0, s>>>(                      \
        x, cols, (uint32_t)block_rows, (uint32_t)(block_cols / 8), (uint32_t)(cols / block_cols), \
        (uint32_t*)acc)
    switch (dtype) {
        case MO_F32: CALL(MO_F32); break;
        case MO_F16: CALL(MO_F16); break;
        default: CALL(MO_BF16); break;
    }
#undef CALL
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_value_ranges(const void* const* xs, const int64_t* counts, const int* dtypes, int n,
                               float* out, int64_t out_chunks, void* stream) {
    if (n < 0 || out_chunks < 0) return MO_ERR_ARG;
    if (n == 0) return MO_OK;
    if (!xs || !counts || !dtypes || !out) return MO_ERR_ARG;
    if (n > mo::kRangeJobs) return MO_ERR_TOO_LARGE;
    mo::RangeJobs jobs;
    int64_t grid = 0;
    for (int i = 0; i < mo::kRangeJobs; ++i) {
        if (i < n) {
            if (counts[i] < 0 || (counts[i] && !xs[i])) return MO_ERR_ARG;
            if (dtypes[i] < MO_F32 || dtypes[i] > MO_BF16) return MO_ERR_DTYPE;
            if ((uintptr_t)xs[i] & (dtypes[i] == MO_F32 ? 3u : 1u)) return MO_ERR_UNSUPPORTED;
        }
        jobs.ptr[i] = i < n ? xs[i] : nullptr;
        jobs.count[i] = i < n ? counts[i] : 0;
        jobs.dtype[i] = i < n ? dtypes[i] : MO_F32;
        jobs.first[i] = (int)grid;
        if (i < n) {
            const int64_t chunks = (counts[i] + mo::kRangeChunk - 1) / mo::kRangeChunk;
            grid += chunks > 0 ? chunks : 1;   // an empty tensor still owns one (+inf, -inf, 0) entry
            if (grid > out_chunks || grid > 0x7FFFFFFF) return MO_ERR_TOO_LARGE;
        }
    }
    jobs.first[mo::kRangeJobs] = (int)grid;
    mo::value_ranges_kernel<<<dim3((unsigned)grid), 256, 0, (hipStream_t)stream>>>(jobs, n, out);
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}
