// Elementwise quantize-dequantize kernels (FP8 E4M3 and N-bit integer) for gfx950.
//
// HBM-bound: one read and one write of the tensor (4 bytes per bf16 element).  x and y are
// viewed as [outer, axis, inner] with one amax per index of `axis`.  Addressing modes:
//   TENSOR  one scale for everything (axis == 1);
//   CHUNK   inner % 8 == 0, so the 8 elements a lane holds share a scale;
//   COLS    inner == 1 and axis % 8 == 0 (scales along the innermost dim): a lane keeps the 8
//           scales of its columns in registers and walks down a slab of rows;
//   ELEM    anything else: per-element scale lookup.
// TENSOR / CHUNK / ELEM run one workgroup per tile of 1024 chunks (4 per lane, all loads issued
// before the math), dispatched in tile order.
#include "common.h"
#include "qdq_ops.h"

namespace mo {

enum { TENSOR = 0, CHUNK = 1, ELEM = 2 };

#ifndef MO_QDQ_U
#define MO_QDQ_U 4
#endif
constexpr int kQdqU = MO_QDQ_U;   // 16-byte chunks per lane
constexpr int kTileChunks = 256 * kQdqU;

template <int DT, int KIND, bool FLAG, typename Op>
__global__ __launch_bounds__(256) void qdq_kernel(const void* __restrict__ x, void* __restrict__ y,
                                                  int64_t n, int64_t axis, int64_t inner,
                                                  const void* __restrict__ amax, int amax_dtype,
                                                  Op op) {
    const int64_t chunks = n >> 3;
    const int64_t c0 = (int64_t)blockIdx.x * kTileChunks + threadIdx.x;
    typename Op::Scale s0 = {};
    if (KIND == TENSOR && amax) s0 = op.make(load_scalar(amax, amax_dtype, 0));
    if (chunks > 0) {
        // All loads of the lane (the per-chunk amax too) come first, in straight-line code: a
        // chunk past the end re-reads the last one and is not stored.  Loads inside per-chunk
        // branches, or after a store, would make every round wait for the store before it.
        const int64_t inner_chunks = KIND == CHUNK ? inner >> 3 : 1;
        RawChunk<DT> raw[kQdqU];
        float am[kQdqU];
#pragma unroll
        for (int u = 0; u < kQdqU; ++u) {
            int64_t c = c0 + u * 256;
            c = c < chunks ? c : chunks - 1;
            load_raw<DT>(x, c << 3, raw[u]);
            am[u] = 0.0f;
            if constexpr (KIND == CHUNK) {
                int64_t row;
                if (chunks <= 0xFFFFFFFFll) row = (uint32_t)c / (uint32_t)inner_chunks;
                else row = c / inner_chunks;
                am[u] = load_scalar(amax, amax_dtype, row < axis ? row : row % axis);
            }
        }
        float v[kQdqU][8];
#pragma unroll
        for (int u = 0; u < kQdqU; ++u) {
            const int64_t c = c0 + u * 256;
            unpack_raw<DT>(raw[u], v[u]);
            if constexpr (KIND == TENSOR || KIND == CHUNK) {
                // one decision per chunk between the branch-free arithmetic and the general one
                // (a branch per element would end the basic block after every element)
                typename Op::Scale s = s0;
                if constexpr (KIND == CHUNK) s = op.make(am[u]);
                if (Op::is_fast(s)) {
#pragma unroll
                    for (int j = 0; j < 8; j += 2) op.template apply2_fast<FLAG>(v[u][j], v[u][j + 1], s, s);
                } else {
#pragma unroll
                    for (int j = 0; j < 8; j += 2) op.template apply2<FLAG>(v[u][j], v[u][j + 1], s, s);
                }
            } else {
                if (c >= chunks) continue;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int64_t a = (((c << 3) + j) / inner) % axis;
                    v[u][j] = op.template apply<FLAG>(v[u][j], op.make(load_scalar(amax, amax_dtype, a)));
                }
            }
            if (c < chunks) store_chunk<DT>(y, c << 3, v[u]);
        }
    }
    // tail (n % 8 elements): the first lanes of the last workgroup
    if (blockIdx.x == gridDim.x - 1 && threadIdx.x < (n & 7)) {
        const int64_t i = (chunks << 3) + threadIdx.x;
        const int64_t a = KIND == TENSOR ? 0 : (i / inner) % axis;
        typename Op::Scale s = {};
        if (amax) s = op.make(load_scalar(amax, amax_dtype, a));
        store_elem<DT>(y, i, op.template apply<FLAG>(load_elem<DT>(x, i), s));
    }
}

// Scales along the innermost dim: x viewed as [rows, axis], axis % 8 == 0.
template <int DT, bool FLAG, typename Op>
__global__ __launch_bounds__(256) void qdq_cols_kernel(const void* __restrict__ x,
                                                       void* __restrict__ y, int64_t rows,
                                                       int64_t axis, int64_t slab,
                                                       const void* __restrict__ amax,
                                                       int amax_dtype, Op op) {
    const int64_t col = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) << 3;
    if (col >= axis) return;
    typename Op::Scale s[8];
    bool fast = true;   // whether all 8 columns of the lane take the branch-free arithmetic
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        s[j] = op.make(load_scalar(amax, amax_dtype, col + j));
        fast = fast && Op::is_fast(s[j]);
    }
    const int64_t r0 = (int64_t)blockIdx.y * slab;
    int64_t r1 = r0 + slab;
    if (r1 > rows) r1 = rows;
    int64_t r = r0;
    for (; r + 3 < r1; r += 4) {
        RawChunk<DT> raw[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) load_raw<DT>(x, (r + u) * axis + col, raw[u]);
        float v[4][8];
#pragma unroll
        for (int u = 0; u < 4; ++u) unpack_raw<DT>(raw[u], v[u]);
        if (fast) {
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int j = 0; j < 8; j += 2)
                    op.template apply2_fast<FLAG>(v[u][j], v[u][j + 1], s[j], s[j + 1]);
        } else {
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int j = 0; j < 8; j += 2)
                    op.template apply2<FLAG>(v[u][j], v[u][j + 1], s[j], s[j + 1]);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) store_chunk<DT>(y, (r + u) * axis + col, v[u]);
    }
    for (; r < r1; ++r) {
        float v[8];
        load_chunk<DT>(x, r * axis + col, v);
#pragma unroll
        for (int j = 0; j < 8; j += 2) op.template apply2<FLAG>(v[j], v[j + 1], s[j], s[j + 1]);
        store_chunk<DT>(y, r * axis + col, v);
    }
}

// Scales per two-dimensional block: x viewed as [rows, cols] with one amax per tile of
// block_rows x block_cols elements, amax[(row / block_rows) * (cols / block_cols) + col /
// block_cols] (block_cols % 8 == 0, so the 8 elements of a lane's chunk share a scale).  The same
// tile walk as the CHUNK mode above: all loads first, one decision per chunk.
template <int DT, bool FLAG, typename Op>
__global__ __launch_bounds__(256) void qdq_blocks2d_kernel(const void* __restrict__ x,
                                                           void* __restrict__ y, int64_t chunks,
                                                           uint32_t row_chunks, uint32_t block_rows,
                                                           uint32_t block_chunks,
                                                           const void* __restrict__ amax,
                                                           int amax_dtype, Op op) {
    const int64_t c0 = (int64_t)blockIdx.x * kTileChunks + threadIdx.x;
    const uint32_t blocks_across = row_chunks / block_chunks;
    RawChunk<DT> raw[kQdqU];
    float am[kQdqU];
#pragma unroll
    for (int u = 0; u < kQdqU; ++u) {
        int64_t c = c0 + u * 256;
        c = c < chunks ? c : chunks - 1;
        load_raw<DT>(x, c << 3, raw[u]);
        const int64_t row = c / row_chunks;
        const uint32_t across = (uint32_t)(c - row * row_chunks) / block_chunks;
        am[u] = load_scalar(amax, amax_dtype, (row / block_rows) * blocks_across + across);
    }
#pragma unroll
    for (int u = 0; u < kQdqU; ++u) {
        const int64_t c = c0 + u * 256;
        float v[8];
        unpack_raw<DT>(raw[u], v);
        const typename Op::Scale s = op.make(am[u]);
        if (Op::is_fast(s)) {
#pragma unroll
            for (int j = 0; j < 8; j += 2) op.template apply2_fast<FLAG>(v[j], v[j + 1], s, s);
        } else {
#pragma unroll
            for (int j = 0; j < 8; j += 2) op.template apply2<FLAG>(v[j], v[j + 1], s, s);
        }
        if (c < chunks) store_chunk<DT>(y, c << 3, v);
    }
}

template <int DT, bool FLAG, typename Op>
static int launch_qdq_blocks2d(const void* x, void* y, int64_t rows, int64_t cols, int64_t block_rows,
                               int64_t block_cols, const void* amax, int amax_dtype, Op op,
                               hipStream_t s) {
    const int64_t chunks = rows * (cols >> 3);
    const int64_t tiles = (chunks + kTileChunks - 1) / kTileChunks;
    if (tiles > 0x7FFFFFFF) return MO_ERR_UNSUPPORTED;
    qdq_blocks2d_kernel<DT, FLAG, Op><<<dim3((unsigned)tiles), 256, 0, s>>>(
        x, y, chunks, (uint32_t)(cols >> 3), (uint32_t)block_rows, (uint32_t)(block_cols >> 3), amax,
        amax_dtype, op);
    return MO_OK;
}

// What the two-dimensional entry points accept: whole blocks (the caller pads), chunks of 8 that
// stay inside a block, 16-byte aligned tensors.
static int check_blocks2d(const void* x, const void* y, int64_t rows, int64_t cols, int64_t block_rows,
                          int64_t block_cols, const void* amax, int amax_dtype) {
    if (rows < 0 || cols < 0 || block_rows <= 0 || block_cols <= 0) return MO_ERR_ARG;
    if (amax_dtype < MO_F32 || amax_dtype > MO_BF16) return MO_ERR_DTYPE;
    if (rows == 0 || cols == 0) return MO_OK;
    if (!x || !y || !amax) return MO_ERR_ARG;
    if (rows % block_rows || cols % block_cols || block_cols % 8 || cols > 0x7FFFFFFFll ||
        block_rows > 0x7FFFFFFFll || (((uintptr_t)x | (uintptr_t)y) & 15u))
        return MO_ERR_UNSUPPORTED;
    return MO_OK;
}

// Unaligned base pointers: same math, scalar accesses.
template <int DT, bool FLAG, typename Op>
__global__ __launch_bounds__(256) void qdq_scalar_kernel(const void* __restrict__ x,
                                                         void* __restrict__ y, int64_t n,
                                                         int64_t axis, int64_t inner,
                                                         const void* __restrict__ amax,
                                                         int amax_dtype, Op op) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        typename Op::Scale s = {};
        if (amax) s = op.make(load_scalar(amax, amax_dtype, (i / inner) % axis));
        store_elem<DT>(y, i, op.template apply<FLAG>(load_elem<DT>(x, i), s));
    }
}

template <int DT, bool FLAG, typename Op>
static int launch_qdq(const void* x, void* y, int64_t outer, int64_t axis, int64_t inner,
                      const void* amax, int amax_dtype, Op op, hipStream_t s) {
    const int64_t n = outer * axis * inner;
    const bool aligned = (((uintptr_t)x | (uintptr_t)y) & 15u) == 0;
    if (!aligned) {
        int64_t b = (n + 255) / 256;
        if (b > 16384) b = 16384;
        qdq_scalar_kernel<DT, FLAG, Op><<<(unsigned)b, 256, 0, s>>>(x, y, n, axis, inner, amax, amax_dtype, op);
        return MO_OK;
    }
    if (amax && axis > 1 && inner == 1 && axis % 8 == 0 && axis >= 512) {
        const int64_t gx = (axis / 8 + 255) / 256;
        int64_t gy = (4096 + gx - 1) / gx;
        int64_t slab = (outer + gy - 1) / gy;
        if (slab < 8) slab = 8;
        gy = (outer + slab - 1) / slab;
        if (gy > 65535) { gy = 65535; slab = (outer + gy - 1) / gy; gy = (outer + slab - 1) / slab; }
        qdq_cols_kernel<DT, FLAG, Op><<<dim3((unsigned)gx, (unsigned)gy), 256, mo::ballast_bytes("qdq_cols_kernel", 0), s>>>(
            x, y, outer, axis, slab, amax, amax_dtype, op);
        return MO_OK;
    }
    int64_t tiles = ((n >> 3) + kTileChunks - 1) / kTileChunks;
    if (tiles < 1) tiles = 1;
    if (tiles > 0x7FFFFFFF) return MO_ERR_UNSUPPORTED;
    const unsigned g = (unsigned)tiles;
    // the occupancy cap pays from about 64 MB of input (measured: 4096 x 4096 bf16 runs at 6.4
    // TB/s without and 5.5 with it, 8192 x 8192 at 5.7 without and 6.1 with it)
    if (axis == 1 || !amax)
        qdq_kernel<DT, TENSOR, FLAG, Op><<<g, 256, mo::ballast_bytes("qdq_kernel_tensor", tiles >= 4096 ? 36 : 0), s>>>(x, y, n, axis, inner, amax, amax_dtype, op);
    else if (inner % 8 == 0)
        qdq_kernel<DT, CHUNK, FLAG, Op><<<g, 256, mo::ballast_bytes("qdq_kernel", 0), s>>>(x, y, n, axis, inner, amax, amax_dtype, op);
    else
        qdq_kernel<DT, ELEM, FLAG, Op><<<g, 256, mo::ballast_bytes("qdq_kernel", 0), s>>>(x, y, n, axis, inner, amax, amax_dtype, op);
    return MO_OK;
}

// ------------------------------------------------------------------------------ one launch
// Per-tensor abs-max and quantize-dequantize in ONE launch that reads x once: a lane loads its
// U chunks into registers, the workgroups agree on the abs-max (grid_max_exchange) and every
// lane quantises what it holds.  Chunk (u * gridDim.x + blockIdx.x) * 256 + threadIdx.x belongs
// to round u of a lane, so a round of a workgroup is 4 KiB of contiguous memory.
template <int DT, int U, bool FLAG, typename Op>
__global__ __launch_bounds__(256) void fused_amax_qdq_kernel(
    const void* __restrict__ x, void* __restrict__ y, int64_t n, Op op, uint32_t* __restrict__ ws,
    uint32_t spin_limit, float* __restrict__ amax_out) {
    __shared__ uint32_t smem[8];
    const int64_t chunks = n >> 3;
    RawChunk<DT> raw[U];
    uint32_t m = 0;
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int64_t c = ((int64_t)u * gridDim.x + blockIdx.x) * 256 + threadIdx.x;
        zero_raw<DT>(raw[u]);
        if (c < chunks) load_raw<DT>(x, c << 3, raw[u]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        if constexpr (DT == MO_F32) {
            const uint32_t w[8] = {raw[u].a.x, raw[u].a.y, raw[u].a.z, raw[u].a.w,
                                   raw[u].b.x, raw[u].b.y, raw[u].b.z, raw[u].b.w};
#pragma unroll
            for (int j = 0; j < 8; ++j) { const uint32_t t = w[j] & 0x7FFFFFFFu; m = t > m ? t : m; }
        } else {
            const uint32_t t = pk_max_u16(pk_max_u16(raw[u].a.x & 0x7FFF7FFFu, raw[u].a.y & 0x7FFF7FFFu),
                                          pk_max_u16(raw[u].a.z & 0x7FFF7FFFu, raw[u].a.w & 0x7FFF7FFFu));
            m = pk_max_u16(m, t);
        }
    }
    // the tail (n % 8 elements) is handled by the first lanes of workgroup 0
    float tail = 0.0f;
    const bool has_tail = blockIdx.x == 0 && threadIdx.x < (n & 7);
    if (has_tail) tail = load_elem<DT>(x, (chunks << 3) + threadIdx.x);
    uint32_t bits;
    if constexpr (DT == MO_F32) bits = m;
    else {
        const uint32_t h = (m & 0xFFFFu) > (m >> 16) ? (m & 0xFFFFu) : (m >> 16);
        bits = DT == MO_BF16 ? h << 16 : f2u(f16_bits_to_f32(h));
    }
    const uint32_t tb = f2u(tail) & 0x7FFFFFFFu;
    bits = tb > bits ? tb : bits;
    uint32_t gbits;
    if (!grid_max_exchange(ws, bits, gridDim.x, spin_limit, smem, gbits)) {
        // the wait for the other workgroups expired: take the abs-max of the whole tensor here
        // (x is not written by this launch: the host refuses overlapping x and y)
        keep_branch();
        constexpr int kPerUnit = DT == MO_F32 ? 4 : 8;
        const int64_t units = n / kPerUnit;
        uint32_t extra = 0;
        if ((int64_t)threadIdx.x < n - units * kPerUnit) {
            const int64_t i = units * kPerUnit + threadIdx.x;
            extra = DT == MO_F32 ? (((const uint32_t*)x)[i] & 0x7FFFFFFFu)
                                 : (uint32_t)(((const uint16_t*)x)[i] & 0x7FFFu);
        }
        const uint32_t h = workgroup_absmax_bits<DT == MO_F32>(x, units, extra, smem);
        gbits = DT == MO_F32 ? h : (DT == MO_BF16 ? h << 16 : f2u(f16_bits_to_f32(h)));
    }
    if (amax_out && blockIdx.x == 0 && threadIdx.x == 0) amax_out[0] = u2f(gbits);
    const typename Op::Scale s0 = op.make(u2f(gbits));
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int64_t c = ((int64_t)u * gridDim.x + blockIdx.x) * 256 + threadIdx.x;
        if (c >= chunks) continue;
        float v[8];
        unpack_raw<DT>(raw[u], v);
        if (Op::is_fast(s0)) {
#pragma unroll
            for (int j = 0; j < 8; j += 2) op.template apply2_fast<FLAG>(v[j], v[j + 1], s0, s0);
        } else {
#pragma unroll
            for (int j = 0; j < 8; j += 2) op.template apply2<FLAG>(v[j], v[j + 1], s0, s0);
        }
        store_chunk<DT>(y, c << 3, v);
    }
    if (has_tail) store_elem<DT>(y, (chunks << 3) + threadIdx.x, op.template apply<FLAG>(tail, s0));
}

template <int DT, int U, bool FLAG, typename Op>
static int launch_fused_qdq_u(const void* x, void* y, int64_t n, Op op, uint32_t* ws,
                              uint32_t spin_limit, float* amax_out, int64_t grid, hipStream_t s) {
    static int limit[64] = {0};  // per device: workgroups of this instantiation resident at once
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return MO_ERR_LAUNCH;
    if (!limit[dev]) {
        const int l = resident_grid_limit(fused_amax_qdq_kernel<DT, U, FLAG, Op>, 256);
        limit[dev] = l > 0 ? l : -1;
    }
    if (limit[dev] < 0) return MO_ERR_UNSUPPORTED;
    if (grid > limit[dev]) return MO_ERR_TOO_LARGE;
    fused_amax_qdq_kernel<DT, U, FLAG, Op><<<dim3((unsigned)grid), 256, 0, s>>>(x, y, n, op, ws, spin_limit, amax_out);
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

// chunks per lane: the smallest of 4, 8, 16 that covers the tensor with at most 512 workgroups
// (two per CU: the fewer workgroups meet at the exchange, the cheaper it is)
template <int DT, bool FLAG, typename Op>
static int launch_fused_qdq(const void* x, void* y, int64_t n, Op op, uint32_t* ws,
                            uint32_t spin_limit, float* amax_out, hipStream_t s) {
    if ((((uintptr_t)x | (uintptr_t)y) & 15u)) return MO_ERR_UNSUPPORTED;
    const int64_t chunks = n >> 3;
    const int64_t lanes = 512 * 256;
    const int64_t need = (chunks + lanes - 1) / lanes;
    const int u = need <= 4 ? 4 : (need <= 8 ? 8 : 16);
    if (need > 16) return MO_ERR_TOO_LARGE;
    int64_t grid = (chunks + 256 * u - 1) / (256 * u);
    if (grid < 1) grid = 1;
    if (u == 4) return launch_fused_qdq_u<DT, 4, FLAG, Op>(x, y, n, op, ws, spin_limit, amax_out, grid, s);
    if (u == 8) return launch_fused_qdq_u<DT, 8, FLAG, Op>(x, y, n, op, ws, spin_limit, amax_out, grid, s);
    return launch_fused_qdq_u<DT, 16, FLAG, Op>(x, y, n, op, ws, spin_limit, amax_out, grid, s);
}

}  // namespace mo

static int check_common(const void* x, void* y, int64_t outer, int64_t axis, int64_t inner,
                        int amax_dtype) {
    if (outer < 0 || axis < 0 || inner < 0) return MO_ERR_ARG;
    if (amax_dtype < MO_F32 || amax_dtype > MO_BF16) return MO_ERR_DTYPE;
    if (outer && axis && inner && (!x || !y)) return MO_ERR_ARG;
    return MO_OK;
}

extern "C" int mo_fp8_qdq(const void* x, void* y, int64_t outer, int64_t axis, int64_t inner,
                          int dtype, const void* amax, int amax_dtype, int saturate,
                          void* stream) {
    int rc = check_common(x, y, outer, axis, inner, amax_dtype);
    if (rc != MO_OK) return rc;
    if (outer == 0 || axis == 0 || inner == 0) return MO_OK;
    hipStream_t s = (hipStream_t)stream;
#define CALL2(DT, SAT)                                                                                 \
    rc = amax ? mo::launch_qdq<DT, SAT>(x, y, outer, axis, inner, amax, amax_dtype,                    \
                                        mo::Fp8Op<true>(), s)                                          \
              : mo::launch_qdq<DT, SAT>(x, y, outer, axis, inner, amax, amax_dtype,                    \
                                        mo::Fp8Op<false>(), s)
#define CALL(DT) \
    if (saturate) { CALL2(DT, true); } else { CALL2(DT, false); }
    switch (dtype) {
        case MO_F32: CALL(MO_F32); break;
        case MO_F16: CALL(MO_F16); break;
        case MO_BF16: CALL(MO_BF16); break;
        default: return MO_ERR_DTYPE;
    }
#undef CALL
#undef CALL2
    if (rc != MO_OK) return rc;
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_int_qdq(const void* x, void* y, int64_t outer, int64_t axis, int64_t inner,
                          int dtype, const void* amax, int amax_dtype, int num_bits,
                          int is_unsigned, int narrow_range, void* stream) {
    int rc = check_common(x, y, outer, axis, inner, amax_dtype);
    if (rc != MO_OK) return rc;
    if (!amax || num_bits < 1 || num_bits > 24) return MO_ERR_ARG;
    if (outer == 0 || axis == 0 || inner == 0) return MO_OK;
    hipStream_t s = (hipStream_t)stream;
    mo::IntOp op;
    op.bound = (float)((1 << (num_bits - 1 + (is_unsigned ? 1 : 0))) - 1);
    op.lo = is_unsigned ? 0.0f : (narrow_range ? -op.bound : -op.bound - 1.0f);
    switch (dtype) {
        case MO_F32: rc = mo::launch_qdq<MO_F32, false>(x, y, outer, axis, inner, amax, amax_dtype, op, s); break;
        case MO_F16: rc = mo::launch_qdq<MO_F16, false>(x, y, outer, axis, inner, amax, amax_dtype, op, s); break;
        case MO_BF16: rc = mo::launch_qdq<MO_BF16, false>(x, y, outer, axis, inner, amax, amax_dtype, op, s); break;
        default: return MO_ERR_DTYPE;
    }
    if (rc != MO_OK) return rc;
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_fp8_qdq_blocks2d(const void* x, void* y, int64_t rows, int64_t cols,
                                   int64_t block_rows, int64_t block_cols, int dtype,
                                   const void* amax, int amax_dtype, int saturate, void* stream) {
    int rc = mo::check_blocks2d(x, y, rows, cols, block_rows, block_cols, amax, amax_dtype);
    if (rc != MO_OK || rows == 0 || cols == 0) return rc;
    hipStream_t s = (hipStream_t)stream;
#define CALL(DT)                                                                                  \
    rc = saturate ? mo::launch_qdq_blocks2d<DT, true>(x, y, rows, cols, block_rows, block_cols, amax, \
                                                      amax_dtype, mo::Fp8Op<true>(), s)           \
                  : mo::launch_qdq_blocks2d<DT, false>(x, y, rows, cols, block_rows, block_cols, amax, \
                                                       amax_dtype, mo::Fp8Op<true>(), s)
    switch (dtype) {
        case MO_F32: CALL(MO_F32); break;
        case MO_F16: CALL(MO_F16); break;
        case MO_BF16: CALL(MO_BF16); break;
        default: return MO_ERR_DTYPE;
    }
#undef CALL
    if (rc != MO_OK) return rc;
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_int_qdq_blocks2d(const void* x, void* y, int64_t rows, int64_t cols,
                                   int64_t block_rows, int64_t block_cols, int dtype,
                                   const void* amax, int amax_dtype, int num_bits, int is_unsigned,
                                   int narrow_range, void* stream) {
    int rc = mo::check_blocks2d(x, y, rows, cols, block_rows, block_cols, amax, amax_dtype);
    if (rc != MO_OK) return rc;
    if (num_bits < 1 || num_bits > 24) return MO_ERR_ARG;
    if (rows == 0 || cols == 0) return MO_OK;
    hipStream_t s = (hipStream_t)stream;
    mo::IntOp op;
    op.bound = (float)((1 << (num_bits - 1 + (is_unsigned ? 1 : 0))) - 1);
    op.lo = is_unsigned ? 0.0f : (narrow_range ? -op.bound : -op.bound - 1.0f);
    switch (dtype) {
        case MO_F32: rc = mo::launch_qdq_blocks2d<MO_F32, false>(x, y, rows, cols, block_rows, block_cols, amax, amax_dtype, op, s); break;
        case MO_F16: rc = mo::launch_qdq_blocks2d<MO_F16, false>(x, y, rows, cols, block_rows, block_cols, amax, amax_dtype, op, s); break;
        case MO_BF16: rc = mo::launch_qdq_blocks2d<MO_BF16, false>(x, y, rows, cols, block_rows, block_cols, amax, amax_dtype, op, s); break;
        default: return MO_ERR_DTYPE;
    }
    if (rc != MO_OK) return rc;
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}

extern "C" int mo_fused_amax_qdq(const void* x, void* y, int64_t n, int dtype, int kind,
                                 int num_bits, int is_unsigned, int narrow_range, int saturate,
                                 float* amax_out, void* workspace, int64_t spin_limit,
                                 void* stream) {
    if (n < 0 || (kind != 0 && kind != 1) || spin_limit < 0) return MO_ERR_ARG;
    if (kind == 0 && (num_bits < 1 || num_bits > 24)) return MO_ERR_ARG;
    if (n == 0) return MO_OK;
    if (!x || !y || !workspace || ((uintptr_t)workspace & 127u)) return MO_ERR_ARG;
    {
        // a workgroup whose wait expires reads all of x again while others may be writing y
        const int64_t bytes = n * (dtype == MO_F32 ? 4 : 2);
        const uintptr_t x0 = (uintptr_t)x, y0 = (uintptr_t)y;
        if (x0 < y0 + (uintptr_t)bytes && y0 < x0 + (uintptr_t)bytes) return MO_ERR_UNSUPPORTED;
    }
    hipStream_t s = (hipStream_t)stream;
    uint32_t* ws = (uint32_t*)workspace;
    const uint32_t spins = spin_limit > 0xFFFFFFFFll ? 0xFFFFFFFFu : (uint32_t)spin_limit;
    int rc;
    if (kind == 1) {
#define CALL(DT)                                                                                   \
    rc = saturate ? mo::launch_fused_qdq<DT, true>(x, y, n, mo::Fp8Op<true>(), ws, spins, amax_out, s) \
                  : mo::launch_fused_qdq<DT, false>(x, y, n, mo::Fp8Op<true>(), ws, spins, amax_out, s)
        switch (dtype) {
            case MO_F32: CALL(MO_F32); break;
            case MO_F16: CALL(MO_F16); break;
            case MO_BF16: CALL(MO_BF16); break;
            default: return MO_ERR_DTYPE;
        }
#undef CALL
    } else {
        mo::IntOp op;
        op.bound = (float)((1 << (num_bits - 1 + (is_unsigned ? 1 : 0))) - 1);
        op.lo = is_unsigned ? 0.0f : (narrow_range ? -op.bound : -op.bound - 1.0f);
        switch (dtype) {
            case MO_F32: rc = mo::launch_fused_qdq<MO_F32, false>(x, y, n, op, ws, spins, amax_out, s); break;
            case MO_F16: rc = mo::launch_fused_qdq<MO_F16, false>(x, y, n, op, ws, spins, amax_out, s); break;
            case MO_BF16: rc = mo::launch_fused_qdq<MO_BF16, false>(x, y, n, op, ws, spins, amax_out, s); break;
            default: return MO_ERR_DTYPE;
        }
    }
    return rc;
}
