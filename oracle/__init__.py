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
``tests/golden/`` that were transcribed from the reference's own tests):

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
export.pack_int4_in_uint8              PARITY UNPINNED by reference tests (no golden vector
                                       exists); pinned only by brute force on tiny inputs and
                                       the unpack(pack(q)) == q invariant
export.fp8_export_cast                 PARITY UNPINNED by reference tests; pinned by the torch
                                       type-promotion rule probed in tests (bf16 / 0-dim fp32)
nf4.nf4_quantize / double_quantization golden round trips test_qtensor_cuda.py:111-131 (with and
/ nf4_dequantize                       without padding), :30-68; per-element Python brute force
awq.awq_lite / smoothquant             the reference's own independent oracle ``awq_lite_manual``
                                       tests/unit/torch/quantization/test_calib.py:53-118
                                       (restated in tests) + closed forms
=====================================  =========================================================
"""

from . import awq, export, fake_quant, nf4, qtensor, reduce  # noqa: F401
