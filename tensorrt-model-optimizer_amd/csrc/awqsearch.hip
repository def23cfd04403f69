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
// A workgroup owns a column tile of 64 output features for one alpha and all T <= 512 tokens, so
// every weight element is scaled and quantised exactly once per alpha; the quantised tile goes
// to LDS as bf16 and is the B operand of v_mfma_f32_32x32x16_bf16 (the 16 x 16 x 32 form reaches
// 70 % of this form's rate here), the activations are loaded straight into the A operand
// registers from a chunk-major copy, in which the lanes of an operand read adjacent memory.  The output tile never leaves the registers: it is rounded
// to bf16, compared with the reference output and reduced to one double per workgroup.
#include "awq_ops.h"
#include "common.h"

namespace mo {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int kSearchTileN = 64;    // output features per workgroup
constexpr int kSearchBlockK = 128;  // k elements per step: 16 chunks of 8

// MB = 32-row blocks per consumer wavefront; the workgroup covers 128 * MB token rows.
// Eight wavefronts: 0-3 produce (weight tile of the next k block: scale, quantise, to LDS), 4-7
// consume (activation fragments from memory, weight fragments from LDS, MFMA).  A SIMD hosts one
// of each, so the vector ALU work of quantising overlaps the matrix work.  Both roles pass the
// same number of barriers: the producer after each tile it wrote, the consumer before each tile
// it reads; tile kb lives in buffer kb & 1, which the producer rewrites (as tile kb + 2) only
// after the barrier that the consumers reach when they are done with tile kb.
template <int MB>
__global__ __launch_bounds__(512) void awq_search_kernel(
    const uint16_t* __restrict__ xs,   // [A][K / 8][T][8] bf16, activations * (1 / s[a])
    const uint16_t* __restrict__ w,    // [N, K] bf16
    const uint16_t* __restrict__ s,    // [A, K] bf16
    const uint16_t* __restrict__ ref,  // [T, N] bf16
    int T, int N, int K, int lg_g, float bound, float lo, double* __restrict__ loss) {
    // quantised weight tile, two buffers: [64 rows][16 chunk slots] of 16 bytes, the slot of
    // chunk c in row r is c ^ (r & 15) so that both the writers (16 lanes per row) and the
    // readers (lanes along rows) spread over all banks
    __shared__ u32x4 tile[2][kSearchTileN][16];
    __shared__ double red[4];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int a = blockIdx.y;
    const int n0 = blockIdx.x * kSearchTileN;
    const int nkb = K / kSearchBlockK;

    // Wavefront w of a workgroup runs on SIMD w % 4: wavefronts 0-3 produce and 4-7 consume, so
    // that every SIMD hosts one of each (with alternating roles two SIMDs would get both
    // consumers and the matrix work would run at half rate).
    const bool producer = wave < 4;
    const int rw = wave & 3;  // index within the role
    if (producer) {
        // ------------------------------------------------------------------ producer
        const uint16_t* sa = s + (int64_t)a * K;
        const int pid = rw * 64 + lane;
        const int qc = pid & 15, qr = pid >> 4;  // chunk qc of rows qr + 16 u
        // Raw weight chunks and scales of two blocks in flight: block kb lives in buffer kb & 1
        // and, once unpacked, its registers are refilled with block kb + 2 (the last blocks fetch
        // the last block again, which is never used).
        const uint16_t* wp[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) wp[u] = w + (int64_t)(n0 + qr + 16 * u) * K + qc * 8;
        const uint16_t* sp = sa + qc * 8;
        u32x4 w0[4], s0, w1[4], s1;
        {
            const int k1 = nkb > 1 ? kSearchBlockK : 0;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                w0[u] = *(const u32x4*)wp[u];
                w1[u] = *(const u32x4*)(wp[u] + k1);
            }
            s0 = *(const u32x4*)sp;
            s1 = *(const u32x4*)(sp + k1);
        }
        auto produce = [&](int kb, u32x4 (&wb)[4], u32x4& sb) {
            const uint32_t sw[4] = {sb.x, sb.y, sb.z, sb.w};
            float sc[8];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                sc[2 * j] = u2f(sw[j] << 16);
                sc[2 * j + 1] = u2f(sw[j] & 0xFFFF0000u);
            }
            float v[4][8];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const uint32_t ww[4] = {wb[u].x, wb[u].y, wb[u].z, wb[u].w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    v[u][2 * j] = round_to_bf16(u2f(ww[j] << 16) * sc[2 * j]);
                    v[u][2 * j + 1] = round_to_bf16(u2f(ww[j] & 0xFFFF0000u) * sc[2 * j + 1]);
                }
            }
            const int k2 = (kb + 2 < nkb ? kb + 2 : nkb - 1) * kSearchBlockK;
#pragma unroll
            for (int u = 0; u < 4; ++u) wb[u] = *(const u32x4*)(wp[u] + k2);
            sb = *(const u32x4*)(sp + k2);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                block_int_qdq_chunk(v[u], lg_g, bound, lo);
                u32x4 o;
                o.x = f32x2_to_bf16x2(v[u][0], v[u][1]);
                o.y = f32x2_to_bf16x2(v[u][2], v[u][3]);
                o.z = f32x2_to_bf16x2(v[u][4], v[u][5]);
                o.w = f32x2_to_bf16x2(v[u][6], v[u][7]);
                const int r = qr + 16 * u;
                tile[kb & 1][r][qc ^ (r & 15)] = o;
            }
            __syncthreads();
        };
        for (int kb = 0; kb < nkb; kb += 2) {
            produce(kb, w0, s0);
            if (kb + 1 < nkb) produce(kb + 1, w1, s1);
        }
        __syncthreads();  // the consumers' reduction barrier
        return;
    }

    // ---------------------------------------------------------------------- consumer
    // v_mfma_f32_32x32x16_bf16: lane (fr, kg) = (lane & 31, lane >> 5) supplies row fr of the A
    // block and column fr of the B block, elements [8 kg, 8 kg + 8) of the 16 k of a step, and
    // receives rows 8 (i / 4) + 4 kg + i % 4 (i = 0..15) of column fr.
    const int cw = rw;
    const int fr = lane & 31, kg = lane >> 5;
    const int row_base = cw * (MB * 32);
    const uint16_t* xa = xs + (int64_t)a * T * K;

    f32x16_t acc[MB][2];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0.0f;

    // Element offsets of this lane's A fragments.  xs is chunk-major: [K / 8][T][8], i.e. the 16
    // bytes of chunk c of row t sit at ((c * T) + t) * 8, so the 32 lanes fr of a k-group read
    // 512 contiguous bytes.  Rows past T repeat row T - 1 (masked in the epilogue); T * K < 2^31
    // is checked by the launcher.
    uint32_t aoff[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        int t = row_base + mb * 32 + fr;
        t = t < T ? t : T - 1;
        aoff[mb] = ((uint32_t)kg * (uint32_t)T + (uint32_t)t) * 8u;
    }
    const uint32_t step_stride = 2u * (uint32_t)T * 8u;  // one step of 16 k = 2 chunks
    // fragments of one half block (four steps of 16 k); each is reloaded for the next half block
    // as soon as the MFMAs that read it have been issued
    u32x4 af[MB][4];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int j = 0; j < 4; ++j) af[mb][j] = *(const u32x4*)(xa + aoff[mb] + j * step_stride);

    const int halves = nkb * 2;
    for (int kb = 0; kb < nkb; ++kb) {
        const int buf = kb & 1;
        __syncthreads();
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            // the half block to prefetch (the last one fetches itself again: no branch in the loop)
            const int nh = kb * 2 + h + 1 < halves ? kb * 2 + h + 1 : halves - 1;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int c = h * 8 + j * 2 + kg;
                bf16x8_t bfrag[2];
#pragma unroll
                for (int nb = 0; nb < 2; ++nb) {
                    const int r = nb * 32 + fr;
                    const u32x4 t = tile[buf][r][c ^ (r & 15)];
                    __builtin_memcpy(&bfrag[nb], &t, 16);
                }
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    bf16x8_t afrag;
                    __builtin_memcpy(&afrag, &af[mb][j], 16);
#pragma unroll
                    for (int nb = 0; nb < 2; ++nb)
                        acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(afrag, bfrag[nb],
                                                                              acc[mb][nb], 0, 0, 0);
                }
                // keep the reloads behind the MFMAs that read the old fragments: hoisted above
                // them they would need a second set of registers
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
                    af[mb][j] = *(const u32x4*)(xa + aoff[mb] + (uint32_t)(nh * 4 + j) * step_stride);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }

    // ---- epilogue: bf16(out) - ref in bf16, squared in fp32 (rows past T read row T - 1 and are
    // masked out of the sum)
    float part = 0.0f;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            const uint16_t* rcol = ref + n0 + nb * 32 + fr;
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
                const float o = round_to_bf16(acc[mb][nb][i]);
                const float d = round_to_bf16(o - bf16_bits_to_f32(rv[i]));
                part += t < T ? d * d : 0.0f;
            }
        }
    double sum = (double)part;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, kWave);
    if (lane == 0) red[cw] = sum;
    __syncthreads();
    if (cw == 0 && lane == 0) atomicAdd(loss + a, red[0] + red[1] + red[2] + red[3]);
}

}  // namespace mo

extern "C" int mo_awq_search_losses(const void* xs, const void* w, const void* s, const void* ref,
                                    int64_t n_alpha, int64_t tokens, int64_t n, int64_t k,
                                    int dtype, int64_t block_size, int num_bits, int is_unsigned,
                                    int narrow_range, double* loss, void* stream) {
    if (n_alpha < 0 || tokens < 0 || n < 0 || k < 0 || num_bits < 2 || num_bits > 16) return MO_ERR_ARG;
    if (dtype != MO_BF16) return MO_ERR_UNSUPPORTED;
    if (n_alpha == 0 || tokens == 0 || n == 0 || k == 0) return MO_OK;
    if (!xs || !w || !s || !ref || !loss) return MO_ERR_ARG;
    int lg_g = -1;
    if (block_size == 32) lg_g = 2;
    else if (block_size == 64) lg_g = 3;
    else if (block_size == 128) lg_g = 4;
    if (lg_g < 0 || tokens > 512 || n % mo::kSearchTileN || k % mo::kSearchBlockK ||
        n_alpha > 65535 || n > 0x7FFFFFFF || tokens * k > 0x7FFFFFFF)
        return MO_ERR_UNSUPPORTED;
    if ((((uintptr_t)xs | (uintptr_t)w | (uintptr_t)s) & 15u) || ((uintptr_t)ref & 1u))
        return MO_ERR_UNSUPPORTED;
    const float bound = (float)((1 << (num_bits - 1 + (is_unsigned ? 1 : 0))) - 1);
    const float lo = is_unsigned ? 0.0f : (narrow_range ? -bound : -bound - 1.0f);
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)(n / mo::kSearchTileN), (unsigned)n_alpha);
    const int mb = (int)((tokens + 127) / 128);
#define CALL(MB)                                                                           \
    mo::awq_search_kernel<MB><<<grid, 512, 0, st>>>(                                       \
        (const uint16_t*)xs, (const uint16_t*)w, (const uint16_t*)s, (const uint16_t*)ref, \
        (int)tokens, (int)n, (int)k, lg_g, bound, lo, loss)
    switch (mb) {
        case 1: CALL(1); break;
        case 2: CALL(2); break;
        case 3: CALL(3); break;
        default: CALL(4); break;
    }
#undef CALL
    return hipGetLastError() == hipSuccess ? MO_OK : MO_ERR_LAUNCH;
}
