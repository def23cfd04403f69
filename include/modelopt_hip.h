/*
 * modelopt_hip.h -- C ABI of libmodelopt_hip.so: gfx950 (MI355X) kernels for the ModelOpt
 * quantization hot path.
 *
 * Contract shared by every entry point:
 *   - plain C linkage, raw device pointers, sizes and enums only (no torch / C++ types);
 *   - the caller owns every buffer (inputs, outputs, accumulators); nothing is allocated,
 *     freed or synchronised inside the library; work is enqueued on `stream`
 *     (a hipStream_t passed as void*, NULL = the default stream) and is stream ordered;
 *   - return value 0 on success, a negative MO_ERR_* code otherwise (no exceptions cross the
 *     ABI); mo_error_string() names a code;
 *   - tensors are contiguous row-major; `dtype` selects the element type of x / y.
 *
 * Each function cites the reference interface it replaces (paths relative to the reference
 * checkout; TQ = modelopt/torch/quantization).
 */
#ifndef MODELOPT_HIP_H_
#define MODELOPT_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum mo_dtype { MO_F32 = 0, MO_F16 = 1, MO_BF16 = 2 };

enum mo_status {
    MO_OK = 0,
    MO_ERR_ARG = -1,      /* null pointer, negative size, inconsistent shape */
    MO_ERR_DTYPE = -2,    /* unsupported element type */
    MO_ERR_UNSUPPORTED = -3, /* valid request the kernels do not cover (e.g. block size) */
    MO_ERR_LAUNCH = -4,   /* the HIP runtime rejected the launch */
    MO_ERR_TOO_LARGE = -5 /* input beyond the fixed workspace of an entry point that may not allocate */
};

int mo_version(void);
const char* mo_error_string(int status);

/* Per-call flags of the NVFP4 quantize entry points (there is no process-wide state: two
 * callers with different policies can use the library at once).
 * MO_FLAG_FORCE_EXACT makes the kernels divide every element by its block scale (the
 * reference's literal arithmetic) instead of the reciprocal-and-correct fast path; the outputs
 * are identical either way, which is what the flag exists to demonstrate.
 * MO_FLAG_SATURATE_BLOCK_SCALE makes the kernels clamp a block scale at 448 before its E4M3
 * cast.  The reference's cast (TQ/qtensor/nvfp4_tensor.py:84-91) is torch's non-saturating one:
 * a block whose abs-max exceeds the per-tensor amax by more than 448/464 (possible once awq_clip
 * has shrunk that amax, TQ/model_calib.py:869-876) gets the NaN byte and dequantises to NaN.
 * Without the flag that behaviour is kept.  Unknown bits return MO_ERR_ARG. */
enum mo_quantize_flags { MO_FLAG_FORCE_EXACT = 1, MO_FLAG_SATURATE_BLOCK_SCALE = 2 };

/* ------------------------------------------------------------------ abs-max reductions
 * Replaces reduce_amax (TQ/utils.py:156-188) as used by MaxCalibrator.collect
 * (TQ/calib/max.py:53-94) and TensorQuantizer._get_amax (TQ/nn/modules/tensor_quantizer.py
 * :505-514).
 *
 * x is viewed as [outer, axis, inner]; acc[a] = max(acc[a], max over (o, i) of |x[o, a, i]|).
 * acc holds fp32 values that must be non-negative (or NaN) on entry -- zero for a fresh
 * reduction, the running maximum for a calibrator.  NaN inputs make the result NaN, as
 * torch.max does.  Per-tensor: outer = 1, axis = 1, inner = numel.
 */
int mo_absmax(const void* x, int64_t outer, int64_t axis, int64_t inner, int dtype,
              float* acc, void* stream);

/* mo_absmax with hints from the caller.  MO_ABSMAX_REREAD: the caller reads x again right after
 * this call -- a dynamic quantizer takes the abs-max and then fake-quantises the same tensor
 * (TensorQuantizer._get_amax then _fake_quantize, TQ/nn/modules/tensor_quantizer.py:505-514,
 * 604-640) -- so the per-tensor reduction uses plain instead of streaming loads and leaves the
 * tensor in the memory-side cache for that second pass (the pair is 7-9 % faster on tensors up
 * to 134 MB; the reduction alone is slower, so a calibration pass does not ask for it).  The
 * result is that of mo_absmax; the hint only applies to the per-tensor case (axis == 1).
 * Unknown bits return MO_ERR_ARG. */
enum { MO_ABSMAX_REREAD = 1u };
int mo_absmax_hinted(const void* x, int64_t outer, int64_t axis, int64_t inner, int dtype,
                     float* acc, unsigned hints, void* stream);

/* Two per-tensor mo_absmax calls (x0 of n0 elements into acc0, x1 of n1 into acc1, one dtype) in
 * one launch: the key and the value states of an attention layer reach their quantizers
 * together (k_bmm_quantizer / v_bmm_quantizer, TQ/plugins/huggingface.py:52-69, each a
 * MaxCalibrator.collect, TQ/calib/max.py:53-94) and are a few megabytes each, so a launch per
 * tensor is mostly launch latency.  x0 and x1 16-byte aligned (MO_ERR_UNSUPPORTED otherwise). */
int mo_absmax_pair(const void* x0, int64_t n0, float* acc0, const void* x1, int64_t n1,
                   float* acc1, int dtype, void* stream);

/* The smallest and the largest element of each of n <= 32 tensors and whether it holds a NaN, in
 * one launch.  Tensor i owns max(1, ceil(counts[i] / 4096)) consecutive chunks of out, tensors in
 * order; chunk c of the launch writes out[3 c] = min, out[3 c + 1] = max (NaN elements ignored;
 * +inf / -inf for an empty tensor), out[3 c + 2] = 1 if the chunk holds a NaN, else 0, and the
 * caller folds a tensor's chunks.  xs, counts and dtypes are host arrays of n entries (device
 * pointers, element counts, MO_F32 / MO_F16 / MO_BF16); out is a device buffer of 3 * out_chunks
 * floats.  These are the reductions behind the reference's validity checks of calibrated values --
 * torch.all(amax >= 0) and no inf, no NaN (TensorQuantizer.validate_attr,
 * TQ/nn/modules/tensor_quantizer.py:516-536) and torch.all(pre_quant_scale > 0)
 * (TQ/model_calib.py:384) -- which it runs per quantizer with a host synchronisation each; here
 * the host reads all answers of an algorithm at once.  MO_ERR_TOO_LARGE for n > 32 or more
 * chunks than out_chunks. */
int mo_value_ranges(const void* const* xs, const int64_t* counts, const int* dtypes, int n,
                    float* out, int64_t out_chunks, void* stream);

/* Per-tensor mo_absmax (outer = axis = 1, inner = n) that also leaves the abs-max of every
 * 32768-element tile of x in parts[0 .. *parts_written): the maximum of those words is the
 * abs-max of this tensor alone, whatever acc held before.  For calibration loops that show one
 * tensor to several calibrators in a row (the input of q_proj / k_proj / v_proj; MaxCalibrator.
 * collect, TQ/calib/max.py:53-94, reduces it once per quantizer): the first reduction is shared,
 * the others fold parts into their running maximum later instead of reading the tensor again.
 * parts_written is a host pointer (set before the call returns).  MO_ERR_TOO_LARGE when the
 * tiles outnumber parts_capacity, MO_ERR_UNSUPPORTED when x is not 16-byte aligned. */
int mo_absmax_tensor_parts(const void* x, int64_t n, int dtype, float* acc, uint32_t* parts,
                           int64_t parts_capacity, int64_t* parts_written, void* stream);

/* The per-column case of mo_absmax (x viewed as [outer, axis], inner == 1) in two passes through
 * a caller-provided workspace: row slabs are reduced to partial[slabs, axis] with plain stores
 * (slabs <= partial_rows, chosen by the library), then the columns of that matrix are folded
 * into acc.  Same result as mo_absmax; it avoids the atomic traffic of a fresh accumulator
 * (one atomic per column per workgroup), which dominates when outer * axis is large.
 * partial: device buffer of partial_rows * axis 32-bit words, 16-byte aligned, contents
 * ignored on entry.  Returns MO_ERR_UNSUPPORTED when axis % 8 != 0 or x is not 16-byte
 * aligned (use mo_absmax then).  Replaces the same reference code as mo_absmax. */
int mo_absmax_cols_staged(const void* x, int64_t outer, int64_t axis, int dtype, float* acc,
                          void* partial, int64_t partial_rows, void* stream);

/* mo_absmax_cols_staged for callers that cannot allocate or provide a workspace (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in
 * the reference.  Same arguments minus the workspace, same result: the row-slab maxima go to a
 * fixed 4 MiB array in the library's device image (MO_ABSMAX_COLS_NOALLOC_WORDS 32-bit words,
 * one copy per GPU for the life of the process) and the call performs no hipMalloc / hipFree.
 * axis > MO_ABSMAX_COLS_NOALLOC_WORDS returns MO_ERR_TOO_LARGE; axis % 8 != 0 or a misaligned x
 * returns MO_ERR_UNSUPPORTED.  Every call on a GPU uses that GPU's one array (its contents are
 * overwritten, nothing needs clearing), so calls that overlap on one GPU -- different streams or
 * threads -- race and must be ordered by the caller.  The first call on a device looks the
 * array's address up (hipGetSymbolAddress); make that call outside any stream capture. */
#define MO_ABSMAX_COLS_NOALLOC_WORDS (1 << 20)
int mo_absmax_cols_noalloc(const void* x, int64_t outer, int64_t axis, int dtype, float* acc,
                           void* stream);

/* Per-tensor abs-max of many tensors in ONE launch.  jobs_dev is a device-resident table sorted
 * by tile_begin; job j owns tiles [tile_begin_j, tile_begin_j + ceil(elems_j /
 * MO_ABSMAX_TILE_ELEMS)), total_tiles is the sum (< 2^31).  tile_job_dev[t] = index of the job
 * that owns tile t (device int32[total_tiles]); NULL makes every workgroup binary-search the
 * table instead.  acc as for mo_absmax (one fp32 per job).
 * Every x must be 16-byte aligned.  No counterpart in the reference, which loops over modules
 * in Python (MaxCalibrator.collect per weight, TQ/nn/modules/quant_module.py:148-169). */
#define MO_ABSMAX_TILE_ELEMS 32768
typedef struct mo_absmax_job {
    const void* x;
    float* acc;
    int64_t elems;
    int64_t tile_begin;
} mo_absmax_job;
int mo_absmax_multi(const mo_absmax_job* jobs_dev, int njobs, const int32_t* tile_job_dev,
                    int64_t total_tiles, int dtype, void* stream);

/* ------------------------------------------------------------------ fake quantisation
 * x and y are viewed as [outer, axis, inner]; amax has `axis` elements of type amax_dtype
 * (axis = 1: per tensor).  y may alias x.
 */

/* FP8 E4M3 quantize-dequantize.  Replaces fake_e4m3fy / fake_e4m3fy_with_axis
 * (TQ/src/tensor_quant_gpu_fp8.cu:66-108) with the numerics of the CPU path _fp8_eager
 * (TQ/tensor_quant.py:45-59): scale = RN(RN(1 / f32(amax)) * 448) (what torch computes for
 * `448.0 / amax`), inv = RN(1 / scale), y = T(f32(e4m3_rne(f32(x) * scale)) * inv);
 * amax == NULL is a plain cast.
 * saturate = 0: magnitudes that round above 448 become NaN (CPU torch cast);
 * saturate = 1: they clamp to 448 (the reference's CUDA kernel). */
int mo_fp8_qdq(const void* x, void* y, int64_t outer, int64_t axis, int64_t inner, int dtype,
               const void* amax, int amax_dtype, int saturate, void* stream);

/* Integer quantize-dequantize.  Replaces fake_tensor_quant / fake_tensor_quant_with_axis
 * (TQ/src/tensor_quant_gpu.cu:43-143) with the numerics of _tensor_quant
 * (TQ/tensor_quant.py:574-612): bound = 2^(bits-1+unsigned)-1, scale = bound / f32(amax),
 * amax <= 2^-24 gives 0, y = T(clamp(rne(f32(x) * scale), lo, bound) / scale). */
int mo_int_qdq(const void* x, void* y, int64_t outer, int64_t axis, int64_t inner, int dtype,
               const void* amax, int amax_dtype, int num_bits, int is_unsigned,
               int narrow_range, void* stream);

/* FP8 / integer fake quantisation with one amax per two-dimensional block: x viewed as
 * [rows, cols], amax[(row / block_rows) * (cols / block_cols) + col / block_cols] -- the layout a
 * quantizer with block_sizes on the last two dims gives its amax (FP8_2D_BLOCKWISE_WEIGHT_ONLY_CFG,
 * TQ/config.py; the reshape to [rows / br, br, cols / bc, bc] with the amax on dims 0 and 2 of
 * TQ/nn/modules/tensor_quantizer.py:755-782, for which the reference's kernels fall back to the
 * eager expressions, TQ/tensor_quant.py:75).  Same arithmetic as mo_fp8_qdq / mo_int_qdq, no
 * transposed copy.  rows % block_rows == 0, cols % block_cols == 0 (the caller pads),
 * block_cols % 8 == 0 and 16-byte aligned tensors, MO_ERR_UNSUPPORTED otherwise.  y may alias x. */
int mo_fp8_qdq_blocks2d(const void* x, void* y, int64_t rows, int64_t cols, int64_t block_rows,
                        int64_t block_cols, int dtype, const void* amax, int amax_dtype, int saturate,
                        void* stream);
int mo_int_qdq_blocks2d(const void* x, void* y, int64_t rows, int64_t cols, int64_t block_rows,
                        int64_t block_cols, int dtype, const void* amax, int amax_dtype, int num_bits,
                        int is_unsigned, int narrow_range, void* stream);

/* acc[b] = max(acc[b], abs-max of block b) for the same blocks (reduce_amax over dims 1 and 3 of
 * the reshaped tensor, TQ/utils.py:156-188 under TQ/nn/modules/tensor_quantizer.py:505-514): one
 * workgroup per block.  Same preconditions. */
int mo_absmax_blocks2d(const void* x, int64_t rows, int64_t cols, int64_t block_rows,
                       int64_t block_cols, int dtype, float* acc, void* stream);

/* NVFP4 dynamic-block quantize-dequantize of x[rows, k] with blocks of `block_size` (8, 16 or
 * 32) along k (zero padded).  Replaces fp4_fake_quant_block (TQ/triton/fp4_kernel.py:141-208)
 * and fused_amax_convert for (E2M1, E4M3) (TQ/src/tensor_quant_mx.cu:355).
 * amax: 1-element global amax.
 * mode 0: the threshold-ladder formula of TQ/triton/fp4_kernel.py:86-134 (448 clamp of the
 *         block scale, scale < 1e-5 -> 1, sign from x >= 0);
 * mode 1: identical to NVFP4QTensor.quantize followed by dequantize
 *         (TQ/qtensor/nvfp4_tensor.py:143-297), the reference's CPU path. */
int mo_nvfp4_qdq(const void* x, void* y, int64_t rows, int64_t k, int dtype, const void* amax,
                 int amax_dtype, int block_size, int mode, void* stream);

/* ------------------------------------------------------------------ real quantize + pack */

/* Squared fake-quantisation error for n_cand candidate amax values in one pass over x viewed
 * as [outer, axis, inner]:
 *   loss[k * axis + a] += sum over the elements of channel a of (f32(x) - QDQ(f32(x); cand[k * axis + a]))^2
 * with QDQ the fp32 operator of mo_int_qdq (kind 0: num_bits / is_unsigned / narrow_range) or of
 * mo_fp8_qdq (kind 1: saturate).  Replaces the candidate loop of MseCalibrator.collect
 * (TQ/calib/mse.py:83-107: quant_func, F.mse_loss(reduction="none"), reduce_sum per candidate;
 * driven by mse_calibrate, TQ/model_calib.py:189-262).  x 16-byte aligned; per-channel needs
 * inner % 8 == 0; other layouts return MO_ERR_UNSUPPORTED (callers take the per-candidate path).
 * The sums are fp32, accumulated in an order that differs from torch.sum. */
int mo_qdq_sq_err(const void* x, int64_t outer, int64_t axis, int64_t inner, int dtype,
                  const float* cand, int n_cand, int kind, int num_bits, int is_unsigned,
                  int narrow_range, int saturate, float* loss, void* stream);

/* Block floating point quantize-dequantize of x[rows, k]: blocks of `block_size` (8, 16 or 32)
 * along k (zero padded), one shared scale per block, every element
 * sign(x) * format(|x| * scale) * unscale.  Replaces fused_amax_convert(inputs, block_size,
 * format, scale_format, global_amax) (TQ/src/tensor_quant_mx.cu:355-386; arithmetic :35-57,
 * :97-186; element tables TQ/src/tensor_quant_mx.h:38-178), the kernel behind the MXFP8 / MXFP6 /
 * MXFP4 / MXINT8 configs (TQ/tensor_quant.py:158-198).  The enum follows the reference's Types.
 *   scale_format MO_EF_E8M0, global_amax NULL: unscale = 2^ceil(log2(amax / format_max));
 *   other scale_format, global_amax NULL: unscale = scale_format(amax / format_max), in double;
 *   global_amax given (n_global_amax = 1, or = rows for one per row): the two-level scale of
 *   compute_scale_with_global.  All fp32 steps are IEEE (the reference kernel is built with
 *   --use_fast_math); zero and NaN inputs give a non-negative result. */
enum mo_elem_format {
    MO_EF_E4M3 = 0, MO_EF_E5M2 = 1, MO_EF_INT8 = 2, MO_EF_E0M3 = 3, MO_EF_E1M2 = 4,
    MO_EF_E3M0 = 5, MO_EF_E2M1 = 6, MO_EF_E3M2 = 7, MO_EF_E2M3 = 8, MO_EF_E8M0 = 9
};
int mo_block_fp_qdq(const void* x, void* y, int64_t rows, int64_t k, int dtype, int block_size,
                    int format, int scale_format, const float* global_amax,
                    int64_t n_global_amax, void* stream);

/* y[i] = the value of `format` nearest to x[i] (fp32 in, fp32 out, n elements): the element
 * conversion of mo_block_fp_qdq without a block scale.  Replaces convert_to_exmy(x, format), the
 * binding of convert_to_types (TQ/src/tensor_quant_mx.cu:398, TQ/src/tensor_quant_mx.h:163-186):
 * ties to even (E3M0: away from zero), saturating at the format's maximum, infinities and NaN
 * to the maximum for the table formats; MO_EF_E8M0 gives 0 as there. */
int mo_convert_to_format(const float* x, float* y, int64_t n, int format, void* stream);

/* MXFP4 storage format over the n elements of x in flat blocks of block_size (8 << k, n a
 * multiple of it).  Replaces MXFP4QTensor.quantize / dequantize (TQ/qtensor/mxfp4_tensor.py:38-83,
 * :85-144):
 *   scales[b] = uint8(127 + max(ceil(log2(f32(amax_b) / 6)), -127))   (E8M0)
 *   v = f32(x) / 2^(scales[b] - 127); code = 8 * (v is not > 0) + #{E2M1 bounds < |v|}
 *   (ties to the smaller magnitude, zero packs as code 8); packed[i] = code[2i] | code[2i+1] << 4.
 * Dequantize: y = T((-1)^(code >> 3) * e2m1[code & 7] * 2^(scale - 127)).
 * An infinite or NaN block amax has no defined scale byte in the reference; 255 is written. */
int mo_mxfp4_quantize(const void* x, int64_t n, int dtype, int block_size, uint8_t* packed,
                      uint8_t* scales, void* stream);
int mo_mxfp4_dequantize(const uint8_t* packed, const uint8_t* scales, int64_t n, int block_size,
                        void* y, int dtype, void* stream);

/* NVFP4 quantize + pack.  Replaces NVFP4QTensor.quantize and get_weights_scaling_factor
 * (TQ/qtensor/nvfp4_tensor.py:63-92,143-232) as called by to_quantized_weight
 * (modelopt/torch/export/quant_utils.py:822-834) and TensorQuantizer._real_quantize
 * (TQ/nn/modules/tensor_quantizer.py:610-622).
 * x[rows, k]; kp = k rounded up to a multiple of block_size (zero padded).
 * amax: device fp32 scalar, the global abs-max of x (amax_is_wsf2 = 0) or the already divided
 *       global scale wsf2 (amax_is_wsf2 = 1); wsf2 = f32(amax) / (6 * 448).
 * wsf_in: optional [rows, kp / block_size] E4M3 block scales to use instead of computing
 *       them (NULL to compute).
 * Outputs: packed[rows, kp / 2] (byte i = code[2i] | code[2i+1] << 4, code = sign << 3 |
 * ordinal), wsf_out[rows, kp / block_size] E4M3 bytes (may be NULL when wsf_in is given),
 * wsf2_out (fp32 scalar, may be NULL).  flags: bits of mo_quantize_flags, 0 for the reference's
 * behaviour. */
int mo_nvfp4_quantize(const void* x, int64_t rows, int64_t k, int dtype, int block_size,
                      const float* amax, int amax_is_wsf2, const uint8_t* wsf_in,
                      uint8_t* packed, uint8_t* wsf_out, float* wsf2_out, int flags, void* stream);

/* NVFP4 quantize + pack of many tensors in ONE launch (the whole-model export pass of
 * modelopt/torch/export/unified_export_hf.py:233-391, which calls to_quantized_weight once per
 * linear).  jobs_dev: device-resident table sorted by tile_begin; job j owns tiles
 * [tile_begin_j, tile_begin_j + ceil(elems_j / MO_NVFP4_TILE_ELEMS)); tile_job_dev as for
 * mo_absmax_multi (optional tile -> job index map).  Requirements per job:
 * bf16, block size 16, last dim a multiple of 16 (so elems % 16 == 0 and no padding), x 16-byte
 * and packed 8-byte aligned.  Outputs and amax as for mo_nvfp4_quantize. */
#define MO_NVFP4_TILE_ELEMS 16384
typedef struct mo_nvfp4_job {
    const void* x;
    uint8_t* packed;
    uint8_t* wsf;
    const float* amax;
    float* wsf2_out;   /* may be NULL */
    int64_t elems;
    int64_t tile_begin;
    int64_t reserved;
} mo_nvfp4_job;
int mo_nvfp4_quantize_multi(const mo_nvfp4_job* jobs_dev, int njobs, const int32_t* tile_job_dev,
                            int64_t total_tiles, int dtype, int block_size, int amax_is_wsf2,
                            int flags, void* stream);

/* ------------------------------------------------------------------ one-launch amax -> quantize
 * The fused variants compute the per-tensor abs-max and quantise in ONE launch that reads the
 * tensor once (2 + 2 instead of 2 + 2 + 2 bytes per bf16 element for fake quant, 2.56 instead of
 * 4.56 for NVFP4 quantize + pack): every workgroup keeps its share of the tensor in registers
 * while the workgroups agree on the maximum.  All workgroups have to be resident at once, which
 * bounds the tensor size: MO_ERR_TOO_LARGE beyond 32 MiB (what two workgroups per compute unit
 * hold in registers), MO_ERR_UNSUPPORTED when the layout is not covered; the two-launch entry
 * points take over then.  Other kernels may share the device.  Two fused calls that overlap
 * (different streams) or a device that cannot hold the grid at once (masked compute units) do
 * not break anything, they only make the call slow: see spin_limit.
 * workspace: MO_FUSED_WS_BYTES of device memory, 128-byte aligned, all zero before the first
 *   call; it can be reused by calls that follow each other in one stream (calls that overlap
 *   must not share a workspace).  Every call leaves it ready for the next one.
 * spin_limit: polls (about half a microsecond each) a workgroup waits for the others.  A
 *   workgroup whose wait expires computes the abs-max of the whole tensor by itself and goes on,
 *   so the outputs are the same bits in every case; it also sets the 32-bit word at byte
 *   MO_FUSED_WS_FAIL_OFFSET to 1, which tells the host that a call took that slow way (no kernel
 *   reads the word; the host clears it).
 * amax_out (optional): the abs-max that was used, as fp32. */

#define MO_FUSED_WS_BYTES 512
#define MO_FUSED_WS_FAIL_OFFSET 384

/* mo_absmax (per tensor) followed by mo_nvfp4_quantize with that amax: the same outputs.
 * bf16, block_size 16, k % 16 == 0, x 16-byte and packed 8-byte aligned. */
int mo_nvfp4_quantize_fused(const void* x, int64_t rows, int64_t k, int dtype, int block_size,
                            uint8_t* packed, uint8_t* wsf_out, float* wsf2_out, float* amax_out,
                            int flags, void* workspace, int64_t spin_limit, void* stream);

/* mo_absmax (per tensor) followed by mo_int_qdq (kind 0) or mo_fp8_qdq (kind 1) with that amax:
 * dynamic per-tensor fake quantisation, TensorQuantizer._get_amax + _fake_quantize
 * (TQ/nn/modules/tensor_quantizer.py:505-514, 633-686).  x and y 16-byte aligned and not
 * overlapping (MO_ERR_UNSUPPORTED otherwise: a workgroup whose wait expired reads x again). */
int mo_fused_amax_qdq(const void* x, void* y, int64_t n, int dtype, int kind, int num_bits,
                      int is_unsigned, int narrow_range, int saturate, float* amax_out,
                      void* workspace, int64_t spin_limit, void* stream);

/* NVFP4 unpack + rescale.  Replaces NVFP4QTensor.dequantize (TQ/qtensor/nvfp4_tensor.py
 * :234-297) and fp4_dequantize (TQ/triton/fp4_kernel.py:307):
 * y[rows, kp] = T(LUT[code] * (f32(wsf) * wsf2)). */
int mo_nvfp4_dequantize(const uint8_t* packed, const uint8_t* wsf, const float* wsf2,
                        int64_t rows, int64_t kp, int block_size, void* y, int dtype,
                        void* stream);

/* ------------------------------------------------------------------ FP8 / INT8 storage casts
 * x viewed as [outer, axis, inner], one scale per index of `axis` (axis = 1: per tensor).
 * q = fmt( via( f32(x) / f32(scale) ) ): `via_dtype` is the dtype torch's type promotion gives
 * the quotient (bf16 tensor / bf16 or 0-dim fp32 scale -> bf16: the quotient is rounded to bf16
 * before the final cast; a dim >= 1 fp32 scale -> fp32).  format MO_FMT_E4M3: RNE cast, values
 * that round above 448 become NaN (torch CPU); MO_FMT_INT8: rne, clamp [-128, 127].
 * Replaces FP8QTensor.quantize / INT8QTensor.quantize (TQ/qtensor/fp8_tensor.py:41-113,
 * TQ/qtensor/int8_tensor.py:36-95) and the FP8 / INT8 branches of to_quantized_weight
 * (modelopt/torch/export/quant_utils.py:759-774). */
enum mo_format { MO_FMT_E4M3 = 0, MO_FMT_INT8 = 1 };
int mo_real_quantize(const void* x, int64_t outer, int64_t axis, int64_t inner, int dtype,
                     const void* scale, int scale_dtype, int via_dtype, int format,
                     uint8_t* out, void* stream);

/* y = T( f32(T(q)) * f32(T(scale)) ).  Replaces FP8QTensor.dequantize / INT8QTensor.dequantize
 * (TQ/qtensor/fp8_tensor.py:115-151, TQ/qtensor/int8_tensor.py:97-130). */
int mo_real_dequantize(const uint8_t* q, int64_t outer, int64_t axis, int64_t inner, int format,
                       const void* scale, int scale_dtype, void* y, int dtype, void* stream);

/* The two storage casts with one scale per two-dimensional block: x / q / y viewed as [rows, cols],
 * scale[(row / block_rows) * (cols / block_cols) + col / block_cols] -- FP8QTensor.quantize /
 * dequantize with block_sizes on two dims (TQ/qtensor/fp8_tensor.py:64-112 expands the scales with
 * repeat_interleave; :115-151), the weight-compress path of FP8_2D_BLOCKWISE_WEIGHT_ONLY_CFG and its
 * dequantize-on-forward.  rows % block_rows == 0, cols % block_cols == 0 (the caller pads and
 * crops), block_cols % 8 == 0, x / y 16-byte and q / out 8-byte aligned: MO_ERR_UNSUPPORTED
 * otherwise.  Arguments otherwise as in mo_real_quantize / mo_real_dequantize. */
int mo_real_quantize_blocks2d(const void* x, int64_t rows, int64_t cols, int64_t block_rows,
                              int64_t block_cols, int dtype, const void* scale, int scale_dtype,
                              int via_dtype, int format, uint8_t* out, void* stream);
int mo_real_dequantize_blocks2d(const uint8_t* q, int64_t rows, int64_t cols, int64_t block_rows,
                                int64_t block_cols, int format, const void* scale, int scale_dtype,
                                void* y, int dtype, void* stream);

/* ------------------------------------------------------------------ INT4 weight compression
 * Flat blocks of block_size elements over the n elements of x (tail zero padded).
 * scales[b] = T(f32(T(1 / amax_b)) * 7) (what torch computes for `7 / amax` in dtype T),
 * q = clamp(rne(T(x * scale)), -8, 7) + 8, packed[i] = q[2i] << 4 | q[2i + 1].
 * scales has ceil(n / block_size) elements of dtype T; packed has ceil(n / block_size) *
 * block_size / 2 bytes.  scales_given = 1 makes scales an input: the caller's per-block scales
 * (dtype T) are used as they are and not written, which is the contract of INT4_quantize(input,
 * scales, block_size).  Replaces INT4_quantize (TQ/src/tensor_quant_gpu.cu:311) with the CPU
 * numerics of INT4QTensor.quantize (TQ/qtensor/int4_tensor.py:40-88). */
int mo_int4_block_quantize(const void* x, int64_t n, int64_t block_size, int dtype, void* scales,
                           int scales_given, uint8_t* packed, void* stream);

/* y[2i] = T((packed[i] >> 4) - 8) / scale), y[2i + 1] = T(((packed[i] & 15) - 8) / scale).
 * Replaces INT4_dequantize (TQ/src/tensor_quant_gpu.cu:262) / INT4QTensor.dequantize
 * (TQ/qtensor/int4_tensor.py:90-130). */
int mo_int4_block_dequantize(const uint8_t* packed, int64_t nbytes, int64_t block_size,
                             const void* scales, void* y, int dtype, void* stream);

/* ------------------------------------------------------------------ NF4 weight compression
 * Flat blocks of block_size elements over the n elements of x (tail zero padded).
 * scales[b] = max |x| over block b (dtype T); v = T(f32(x) / f32(scales[b]));
 * code = index of the entry of the bf16-rounded NF4 table nearest to v, distances T(|v - e|)
 * compared after rounding to T, lowest index among equal distances, 0 for NaN;
 * packed[i] = code[2i] << 4 | code[2i + 1].  scales has ceil(n / block_size) elements, packed
 * ceil(n / block_size) * block_size / 2 bytes.  Replaces NF4_quantize
 * (TQ/src/tensor_quant_gpu.cu:211-258) with the CPU numerics of NF4QTensor.quantize
 * (TQ/qtensor/nf4_tensor.py:76-126); the block abs-max is computed here instead of by a
 * separate reduce_amax pass. */
int mo_nf4_quantize(const void* x, int64_t n, int64_t block_size, int dtype, void* scales,
                    uint8_t* packed, void* stream);

/* y[2i] = T(table[packed[i] >> 4] * f32(scales[2i / block_size])), y[2i + 1] likewise for the
 * low nibble; scales and y have dtype T.  Replaces NF4_dequantize
 * (TQ/src/tensor_quant_gpu.cu:146-197) / NF4QTensor.dequantize (TQ/qtensor/nf4_tensor.py:157-201). */
int mo_nf4_dequantize(const uint8_t* packed, int64_t nbytes, int64_t block_size,
                      const void* scales, void* y, int dtype, void* stream);

/* codes[i] = (x[i] < 0) << 3 | ordinal of the E2M1 magnitude nearest to |x[i]| (0, .5, 1, 1.5, 2,
 * 3, 4, 6; ties to the even code, NaN and infinity give ordinal 7, -0.0 gives code 0): one byte
 * per element, unpacked.  Replaces NVFP4QTensor._cast_fp4 (TQ/qtensor/nvfp4_tensor.py:120-140);
 * x is left as it is (the reference takes its absolute value in place). */
int mo_cast_fp4(const void* x, int64_t n, int dtype, uint8_t* codes, void* stream);

/* INT4-AWQ export pack of w[batch, n_rows, k] with fp32 scales ws[batch, n_rows, k/block_size]:
 * q = int8(clamp(rne(f32(w) / ws), -8, 7)); out[b, j, c] = (q[b, 2j, c] & 0xF) |
 * (q[b, 2j+1, c] << 4), out is uint8 [batch, n_rows / 2, k].  Replaces pack_int4_in_uint8
 * (modelopt/torch/export/quant_utils.py:697-738). */
int mo_int4_pack_rows(const void* w, int64_t batch, int64_t n_rows, int64_t k, int64_t block_size,
                      int dtype, const float* ws, uint8_t* out, void* stream);

/* The same with the type the quotient of the reference's tensor division has
 * (modelopt/torch/export/quant_utils.py:704-706: weight / scales follows type promotion): MO_F32
 * for fp32 scales -- what get_scaling_factor (export/quant_utils.py:228) hands the exporter, and
 * what mo_int4_pack_rows computes -- or `dtype` itself when the caller's scales had the weight's
 * own 16-bit type: the quotient is then rounded to that type before it is rounded to an integer
 * (about 1 % of the codes differ).  ws holds the scales widened to fp32 either way.  Any other
 * via_dtype returns MO_ERR_UNSUPPORTED. */
int mo_int4_pack_rows_via(const void* w, int64_t batch, int64_t n_rows, int64_t k, int64_t block_size,
                          int dtype, const float* ws, int via_dtype, uint8_t* out, void* stream);

/* ------------------------------------------------------------------ AWQ-lite / SmoothQuant
 * y[r, c] = T(f32(x[r, c]) * f32(s[c])): the pre_quant_scale multiply of
 * TensorQuantizer.forward (TQ/nn/modules/tensor_quantizer.py:881-882) and the weight folding of
 * _apply_weight_pre_quant_scale (TQ/model_calib.py:346-353).  y may alias x. */
int mo_mul_cols(const void* x, int64_t rows, int64_t k, int dtype, const void* s, int s_dtype,
                void* y, void* stream);

/* Fused weight path of one AWQ-lite search step (TQ/model_calib.py:671-685 through
 * TensorQuantizer.forward and _tensor_quant): xs = T(x * s[c]) (s may be NULL), per-block amax
 * over `block_size` (8..512, power of two) columns, INT-N quantize-dequantize with that amax.
 * y may alias x. */
int mo_scale_block_int_qdq(const void* x, int64_t rows, int64_t k, int dtype, const void* s,
                           int s_dtype, int64_t block_size, int num_bits, int is_unsigned,
                           int narrow_range, void* y, void* stream);

/* acc[c] += sum over rows of |x[r, c]| (blk_amax == NULL: get_act_scale numerator,
 * TQ/model_calib.py:605-606) or of T(|x[r, c]| / T(blk_amax[r, c / block_size] + tiny))
 * (get_weight_scale numerator, TQ/model_calib.py:588-603).  fp32 accumulation; the caller
 * divides by the row count and rounds through T as the reference's `.mean(0)` does. */
int mo_abs_colsum(const void* x, int64_t rows, int64_t k, int dtype, const float* blk_amax,
                  int64_t block_size, float* acc, void* stream);

/* mo_abs_colsum in two passes without atomics: row slabs sum into `partial` (a caller-provided
 * workspace of partial_rows x k floats, 16-byte aligned), then the rows of that matrix are added
 * to acc in a fixed order -- the result does not depend on scheduling.  Returns
 * MO_ERR_UNSUPPORTED unless k % 8 == 0, x is 16-byte aligned and, with blk_amax, block_size is a
 * multiple of 8 that divides k.  Same reference call sites as mo_abs_colsum. */
int mo_abs_colsum_staged(const void* x, int64_t rows, int64_t k, int dtype, const float* blk_amax,
                         int64_t block_size, float* acc, float* partial, int64_t partial_rows,
                         void* stream);

/* acc[c] += sum over rows of T(|x[r, c]| / T(amax(r, c / block_size) + tiny)), amax being the
 * abs-max of the row's block of `block_size` columns taken in the same pass: the whole numerator
 * of get_weight_scale (TQ/model_calib.py:588-603) in one read of the weight, no block-amax
 * array.  Two passes without atomics like mo_abs_colsum_staged (`partial`: partial_rows x k
 * floats, 16-byte aligned); same bits as mo_abs_colsum_staged fed the block abs-max.  Returns
 * MO_ERR_UNSUPPORTED unless block_size is 8, 16, ... 512, divides k, and x is 16-byte aligned. */
int mo_weight_scale_colsum(const void* x, int64_t rows, int64_t k, int dtype, int64_t block_size,
                           float* acc, float* partial, int64_t partial_rows, void* stream);

/* xs[a][c][t][0..8) = bf16(x[t][8 c ..] * inv_s[a][8 c ..]) for n_alpha rows of inv_s: the
 * activations under every candidate scale, in the chunk-major layout mo_awq_search_losses reads
 * ([n_alpha][k / 8][tokens][8] bf16).  This is the `inputs * pre_quant_scale` of the input
 * quantizer in the search forward (TQ/nn/modules/tensor_quantizer.py:881-882, set per alpha at
 * TQ/model_calib.py:671-675) for all alphas at once.  bf16 only, k % 8 == 0, 16-byte aligned
 * buffers; MO_ERR_UNSUPPORTED otherwise. */
int mo_awq_scale_activations(const void* x, const void* inv_s, int64_t n_alpha, int64_t tokens,
                             int64_t k, int dtype, void* xs, void* stream);

/* The candidate scales of a whole AWQ-lite alpha grid in one launch: get_scale
 * (TQ/model_calib.py:608-621) for every alpha a of the grid,
 *   s[a][c] = clamp(x_max[c]^alpha_a / (w_max[c]^(1 - alpha_a) + FLT_MIN), 1e-4, 1e4)
 *   s[a]   /= sqrt(max_c s[a][c] * min_c s[a][c])
 * in fp32 (IEEE division, correctly rounded square root; a NaN anywhere in a row makes the row NaN,
 * as torch's amax / amin do).  exponents: device fp32 [4][n_alpha] -- alpha, 1 - alpha, and for
 * each of the two how the power is evaluated: 0 powf, 1 the constant 1 (exponent 0), 2 the base
 * (exponent 1), 3 the correctly rounded square root (exponent 0.5) -- the cases torch's scalar
 * pow evaluates without calling pow.  Outputs: scales fp32 [n_alpha, k]; w_scales and x_scales
 * (each optional) [n_alpha, k] in dtype: T(s), the weight quantizer's pre-quant scale of the
 * search step, and T(1 / s), the input quantizer's (TQ/model_calib.py:661-664). */
int mo_awq_scale_grid(const float* x_max, const float* w_max, const float* exponents,
                      int64_t n_alpha, int64_t k, float* scales, void* w_scales, void* x_scales,
                      int dtype, void* stream);

/* The end of an AWQ-lite search for one linear, in one launch: best = the index of the first
 * smallest of the n_alpha losses -- what min(loss, key=loss.get) picks (TQ/model_calib.py:633): a
 * NaN is never smaller than anything and a NaN in front is never replaced -- and, from row best
 * of the fp32 candidate grid scales [n_alpha, k] (mo_awq_scale_grid), the tensors the folding
 * makes of it (TQ/model_calib.py:764 and 384-393): best_scale[c] = scales[best][c],
 * pre_quant_scale[c] = 1 / best_scale[c] (fp32, IEEE division), pre_quant_scale_t[c] the same
 * rounded to dtype (the input quantizer's buffer), fold[c] = 1 / pre_quant_scale[c] (what the
 * weight is multiplied by).  loss is a device array of doubles; best (one int64) and every output
 * row are optional device buffers. */
int mo_awq_pick_scale(const double* loss, int64_t n_alpha, const float* scales, int64_t k,
                      int64_t* best, float* best_scale, float* pre_quant_scale,
                      void* pre_quant_scale_t, float* fold, int dtype, void* stream);

/* SmoothQuant's per-channel scale for one linear and what the smoothing makes of it, in one
 * launch (postprocess of smoothquant, TQ/model_calib.py:447-473, and
 * apply_pre_quant_scale_and_smooth, :384-407).  With T the weight dtype, act_amax the fp32
 * per-channel input amax and weight_col_amax the fp32 per-column abs-max of the weight (k each):
 *   ws = T(weight_col_amax[c]);  s[c] = f32(T(ws ^ exp_w)) / act_amax[c] ^ exp_a
 *   if min_c s[c] <= 2^-31: s[c] = 1 where act_amax[c] <= 2^-31;  s[c] = clamp(s[c], 1e-4, 1e4)
 * (exp_w = 1 - alpha, exp_a = alpha; mode_w / mode_a say how each power is evaluated: 0 powf,
 * 1 the constant 1, 2 the base, 3 the correctly rounded square root -- the cases torch's scalar
 * pow evaluates without calling pow; for a 16-bit T and mode_w 0 the caller passes exp_w rounded
 * to T, which is what the tensor expression raises a 16-bit tensor to).  Outputs:
 * pre_quant_scale[c] = s[c] (fp32),
 * pre_quant_scale_t[c] = T(s[c]), fold[c] = 1 / s[c] (what the weight is multiplied by),
 * act_amax_max = T(max_c act_amax[c]) (the per-tensor input amax), smoothed_amax =
 * T(max_c f32(T(act_amax[c])) * s[c]) (the input amax after smoothing); all but pre_quant_scale
 * optional.  NaNs behave as in the tensor expressions: a NaN scale makes the minimum NaN (no
 * channel is reset) and passes the clamp, a NaN operand makes a maximum NaN. */
int mo_smooth_scales(const float* act_amax, const float* weight_col_amax, int64_t k,
                     float exp_w, int mode_w, float exp_a, int mode_a, int dtype,
                     float* pre_quant_scale, void* pre_quant_scale_t, float* fold,
                     void* act_amax_max, void* smoothed_amax, void* stream);

/* AWQ-lite search step for a whole grid of alphas in one launch (bf16 only):
 *   q_a = block INT-N quantise-dequantise (blocks of block_size along k, dynamic abs-max) of
 *         bf16(w * s[a]);   out_a = bf16(xs[a] @ q_a^T)   (fp32 accumulation on the matrix cores)
 *   loss[a] += sum over (t, n) of f32(bf16(out_a[t, n] - ref[t, n]))^2
 * xs holds the activations already multiplied by 1 / s[a], chunk-major: [n_alpha][k / 8][tokens][8]
 * (element (t, c) of alpha a at ((a * (k / 8) + c / 8) * tokens + t) * 8 + c % 8), so that the
 * lanes of a matrix-core operand read adjacent memory; w [n, k]; s [n_alpha, k]; ref [tokens, n];
 * loss: n_alpha doubles, accumulated into (one atomic add per column tile, so the last bits depend
 * on the order the tiles finish in).  The quantised weights and the outputs never reach memory.  Returns MO_ERR_UNSUPPORTED unless dtype is bf16,
 * tokens <= 512, n % 128 == 0, k % 128 == 0, block_size is 32, 64 or 128 and the buffers are
 * 16-byte aligned, or the grid is unsigned (use mo_scale_block_int_qdq + a GEMM + mo_sq_diff_sum
 * per alpha then).  The integer codes are the reference's; the dequantised weight is
 * code * (amax / bound) instead of code / (bound / amax), which can differ in the last bf16 bit
 * for about one weight in 10^4 (per-alpha losses agree to ~1e-6 relative).
 * Replaces the per-alpha loop of the search forward, TQ/model_calib.py:645-690 (weight
 * pre-quant scale, TQ/nn/modules/tensor_quantizer.py:881-882; dynamic block amax :505-514;
 * _tensor_quant TQ/tensor_quant.py:574-612; update_loss TQ/model_calib.py:623-627). */
int mo_awq_search_losses(const void* xs, const void* w, const void* s, const void* ref,
                         int64_t n_alpha, int64_t tokens, int64_t n, int64_t k, int dtype,
                         int64_t block_size, int num_bits, int is_unsigned, int narrow_range,
                         double* loss, void* stream);

/* The same for a linear layer with a bias (the F.linear of nn.Linear.forward under
 * QuantLinearConvBase.forward, TQ/nn/modules/quant_module.py:148-169, which the search forward
 * TQ/model_calib.py:645-690 runs once per alpha): bias[n] (dtype of w, or
 * null for none) is added to the fp32 sums before they are rounded, out_a = bf16(sum + bias). */
int mo_awq_search_losses_biased(const void* xs, const void* w, const void* s, const void* ref,
                                const void* bias, int64_t n_alpha, int64_t tokens, int64_t n,
                                int64_t k, int dtype, int64_t block_size, int num_bits,
                                int is_unsigned, int narrow_range, double* loss, void* stream);

/* AWQ clip search, all ratios and all weight blocks of one [n, k] weight on one batch of
 * `tokens` activations in one launch.  For block (row, b) of `block_size` input channels and
 * ratio r, with T the weight dtype and every step rounded as the tensor expression rounds it:
 *   org[t] = T(sum_j T(x[t, j] * w[row, j])),  cur[t] = T(sum_j T(x[t, j] * wq[row, j])),
 *   wq = T(int_qdq(w, amax = A(f32(w_amax[row, b]) * ratios[r])))   (A: the dtype of w_amax)
 *   loss[r, row, b] += sum_t f32(T(cur[t] - org[t]))^2 / tokens      (fp32, accumulated in place)
 * x: [tokens, k] contiguous, same dtype as w; ratios: host array, at most 32; loss: fp32
 * [n_ratios, n, k / block_size].  Returns MO_ERR_UNSUPPORTED unless block_size is 16, 32, 64 or
 * 128 and divides k.  Replaces the (ratio x row batch) loop of the clip search,
 * TQ/model_calib.py:898-930 (broadcast products :901 and :916, fake quant of the clipped weight
 * :903-905, loss :919). */
int mo_awq_clip_losses(const void* x, int64_t tokens, const void* w, int64_t n, int64_t k,
                       int dtype, int64_t block_size, const void* w_amax, int amax_dtype,
                       const float* ratios, int n_ratios, int num_bits, int is_unsigned,
                       int narrow_range, float* loss, void* stream);

/* acc[0] += sum of f32(T(a[i] - b[i]))^2 in double: the numerator of update_loss
 * (TQ/model_calib.py:623-627). */
int mo_sq_diff_sum(const void* a, const void* b, int64_t n, int dtype, double* acc, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* MODELOPT_HIP_H_ */
