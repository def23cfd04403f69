// Measurement aid, not part of the quantization library: how fast can the compute units of
// gfx950 pull L2-resident data through their L1 misses?  The AWQ-lite search kernel reads its A
// operand that way (every compute unit of an XCD walks the same 4 MB of activations, 16 bytes a
// lane, a few steps ahead of their use), and this kernel does nothing else: each workgroup of
// 8 wavefronts walks a region with 16-byte loads, DEPTH of them in flight per lane, and folds the
// values into one word so that the loads stay.  Built into its own small library
// (libmodelopt_probe.so) and driven by `bench.py --probe-l2`.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kXcds = 8;
constexpr int kThreads = 512;

// Workgroup L runs on XCD L % 8.  `region_units` 16-byte units per XCD; a workgroup walks
// `span_units` of them per pass, from `slot * span_units` when `distinct` (every workgroup its
// own slice of the XCD's region) and from 0 otherwise (all workgroups of an XCD the same
// addresses at about the same time, as the search kernel's column tiles do).  `zero` is 0: the
// compiler cannot know that, so the passes are not folded into one.
template <int DEPTH>
__global__ __launch_bounds__(kThreads) void l2_read_probe_kernel(
    const u32x4* __restrict__ base, uint32_t region_units, uint32_t span_units, int passes,
    int distinct, int zero, uint32_t* __restrict__ sink) {
    extern __shared__ char ballast[];   // unused: its size sets how many workgroups share a unit
    const uint32_t xcd = blockIdx.x % kXcds, slot = blockIdx.x / kXcds;
    const u32x4* p = base + (size_t)xcd * region_units + (distinct ? (size_t)slot * span_units : 0) +
                     threadIdx.x;
    u32x4 acc = {0u, 0u, 0u, 0u};
    constexpr uint32_t kStep = kThreads * DEPTH;
    for (int pass = 0; pass < passes; ++pass) {
        const u32x4* q = p + (size_t)pass * (size_t)zero;
        u32x4 v[DEPTH];
#pragma unroll
        for (int j = 0; j < DEPTH; ++j) v[j] = q[j * kThreads];
        for (uint32_t i = kStep; i < span_units; i += kStep) {
#pragma unroll
            for (int j = 0; j < DEPTH; ++j) {
                acc ^= v[j];
                v[j] = q[i + j * kThreads];
            }
        }
#pragma unroll
        for (int j = 0; j < DEPTH; ++j) acc ^= v[j];
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9E3779B9u) sink[0] = 1u;   // never true for a zeroed buffer
}

}  // namespace

// Launches `workgroups` (a multiple of 8) workgroups of 512 threads, `ballast_bytes` of unused
// LDS each (more than half of a compute unit's 160 KB keeps one workgroup per unit).  Returns 0,
// or -1 for arguments the kernel's indexing does not cover.  Bytes read through L1 misses:
// workgroups * passes * span_bytes.
extern "C" int mo_probe_l2_read(const void* buf, int64_t buf_bytes, int64_t region_bytes,
                                int64_t span_bytes, int workgroups, int passes, int distinct,
                                int depth, int ballast_bytes, void* sink, void* stream) {
    if (!buf || !sink || ((uintptr_t)buf & 15u) || workgroups <= 0 || workgroups % kXcds || passes <= 0)
        return -1;
    if (depth != 4 && depth != 8 && depth != 16) return -1;
    if (ballast_bytes < 0 || ballast_bytes > 160 * 1024 - 64) return -1;
    const int64_t step_bytes = (int64_t)kThreads * depth * 16;
    if (region_bytes <= 0 || span_bytes <= 0 || span_bytes % step_bytes || region_bytes > (1ll << 31)) return -1;
    const int64_t per_xcd = workgroups / kXcds;
    if ((distinct ? span_bytes * per_xcd : span_bytes) > region_bytes) return -1;
    if (region_bytes * kXcds > buf_bytes) return -1;
    const uint32_t region_units = (uint32_t)(region_bytes / 16), span_units = (uint32_t)(span_bytes / 16);
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)workgroups), block(kThreads);
    const u32x4* b = (const u32x4*)buf;
    uint32_t* s = (uint32_t*)sink;
#define LAUNCH(D)                                                                              \
    {                                                                                          \
        if (ballast_bytes > 64 * 1024 &&                                                       \
            hipFuncSetAttribute((const void*)l2_read_probe_kernel<D>,                         \
                                hipFuncAttributeMaxDynamicSharedMemorySize, ballast_bytes) != hipSuccess) \
            return -2;                                                                         \
        hipLaunchKernelGGL(l2_read_probe_kernel<D>, grid, block, (size_t)ballast_bytes, st, b, \
                           region_units, span_units, passes, distinct, 0, s);                  \
    }
    if (depth == 4) LAUNCH(4)
    else if (depth == 8) LAUNCH(8)
    else LAUNCH(16)
#undef LAUNCH
    return hipGetLastError() == hipSuccess ? 0 : -2;
}
