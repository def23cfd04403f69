"""CPU oracle for the quantization hot path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``oracle/`` is part of the shipped product: it may be
imported by ``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py`` as the checker / the timed CPU baseline, and by nothing else.  The product path
(``modelopt_amd``) never imports it and raises when its HIP library is missing.

Every function restates, op for op and dtype for dtype, what the reference's CPU torch path
computes (reference file:line is cited in each docstring; paths are relative to the reference
checkout, ``modelopt/torch/quantization`` abbreviated ``TQ``).  The arithmetic primitives the
reference itself calls on CPU (``Tensor.to(torch.float8_e4m3fn)``, ``torch.round``,
``torch.searchsorted``, IEEE fp32 ``/``) are called here too, so rounding behaviour is the
library's, not a re-derivation.  ``oracle/c/quant_ref.c`` (loaded through ``oracle/cref.py``) is
an independent bit-level C restatement -- software E4M3 / E2M1 / bf16 / fp16 rounding, the NVFP4
quantize+pack and dequantize chain, FP8 and integer fake quantisation, the INT4 block compress
and the FP8 / INT8 storage casts -- that ``tests/test_oracle_c.py`` cross-checks bit for bit
against the torch restatement; it is also the timed CPU baseline of ``bench.py``.

What pins each function (checked by ``tests/test_oracle_golden.py`` against the fixtures in
``tests/golden/`` that were transcribed from the reference's own tests; the search oracles by
``tests/test_oracle_search.py``, the MX formats by ``tests/test_mx_oracle.py``):

=====================================  =========================================================
function                               pinned by
=====================================  =========================================================
reduce.reduce_amax / reduce_block_*    reference vectors tests/unit/torch/quantization/
                                       test_utils.py:25-56, test_calibrator.py:28-90; textbook max
reduce.MaxCalibrator                   test_calibrator.py:28-90 (exact running max, shape error)
fake_quant.fp8_eager                   torch's own float8_e4m3fn cast (library routine) +
                                       golden test_qtensor_cuda.py:191-241; brute force over all
                                       bf16 bit patterns against a bit-level software E4M3 rounder
fake_quant.tensor_quant (INT)          closed form tests/_test_utils/torch/quantization/
                                       quant_utils.py:19-30; tensor_quant_common.py:37-124
fake_quant.nvfp4_fake_quant            boundary vectors test_tensor_quant_cuda.py:198-223
qtensor.nvfp4_*                        test_qtensor_cuda.py:287-375 (values/pack/LUT), :400-440
                                       (brute-force twin of the FP4 cast); oracle/c cross-check
qtensor.int4_* / int8_* / fp8_*        golden bf16 vectors test_qtensor_cuda.py:133-241
export.get_scaling_factor_from_weight  exact vectors tests/gpu/torch/export/test_export.py:163-197
export.pack_int4_in_uint8 /            no reference test holds a vector for these, so
export.fp8_export_cast /               tests/golden/export_vectors.json records what the reference's
export.int8_export_cast                own pack_int4_in_uint8 and to_quantized_weight
                                       (export/quant_utils.py:697-774) return on seeded inputs (2-D and
                                       3-D weights, ties, clamped values, asymmetric nibbles that tell the
                                       two nibble orders apart, bf16 / 0-dim fp32 promotion); written by
                                       tests/golden/make_export_vectors.py in the build container
export.nvfp4_export                    composition of the pinned qtensor.nvfp4_* functions
fake_quant.static_block_fake_quant     float64 closed form (tests/test_oracle_search.py)
nf4.nf4_quantize / double_quantization golden round trips test_qtensor_cuda.py:111-131 (with and
/ nf4_dequantize                       without padding), :30-68; per-element Python brute force
awq.awq_lite_search / awq_get_scale /  tests/test_oracle_search.py: numpy float64 formulations written from
awq_weight_scale / awq_act_scale       the mathematics (no shared code), on the case of the reference's
                                       own test (16-32-16-16 MLP, seed 0, one randn(2, 64, 16) batch, INT4
                                       blocks of 8: tests/unit/torch/quantization/test_calib.py:33-52,
                                       :170-186, which that test checks against its own independent
                                       implementation :72-116 with allclose) + closed forms (alpha 0 / 1,
                                       max * min = 1)
awq.awq_clip_search                    the same case against a float64 formulation of the per-block
                                       clip error (reference's independent implementation
                                       test_calib.py:120-167); token subsampling and batch accumulation
awq.smoothquant_linear /               float64 formulation + the invariant (x * s) @ (w / s)^T == x @ w^T
awq.fold_pre_quant_scale
mse.mse_search / candidates            known-answer cases of tests/unit/torch/quantization/
                                       test_mse_calibrator.py:40-186, :187-232, :321-479 (outlier tensors,
                                       accumulation, independent channels) with the whole loss curve
                                       equal to a float64 closed form
mx.*                                   the reference's golden tables tests/gpu/torch/quantization/
                                       test_quantize_mxformats_cuda.py (tests/golden/mx_vectors.json),
                                       an independent C restatement, fixed points and tie rules
                                       (tests/test_mx_oracle.py)
=====================================  =========================================================
"""

from . import awq, export, fake_quant, nf4, qtensor, reduce  # noqa: F401
