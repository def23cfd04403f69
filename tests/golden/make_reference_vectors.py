"""Writes tests/golden/reference_vectors.json.

Every entry is DATA (inputs and expected outputs) transcribed from the inline literals of the
reference's own tests; the source test is cited per entry.  Nothing of the reference is imported
or executed.  Run from the repo root: ``python tests/golden/make_reference_vectors.py``.
"""

import json
import os

V = {}

# tests/gpu/torch/quantization/test_qtensor_cuda.py:133-241 (test_qtensor_accuracy): real quantize
# through TensorQuantizer then dequantize; bf16 inputs, expected bf16 outputs (torch.allclose).
V["qtensor_roundtrip"] = [
    {"name": "int4_block4", "num_bits": 4, "block_sizes": {"-1": 4}, "axis": None,
     "input": [[0, 1, 2, 3, 4, 5, 6, 7]],
     "output": [[0.0000, 0.8516, 2.1406, 2.9844, 4.0000, 5.0000, 6.0000, 7.0000]]},
    {"name": "int4_block4_padding", "num_bits": 4, "block_sizes": {"-1": 4}, "axis": None,
     "input": [[0, 1, 2, 3, 4, 5, 6, 7, 3, 3]],
     "output": [[0.0000, 0.8516, 2.1406, 2.9844, 4.0000, 5.0000, 6.0000, 7.0000, 2.9844, 2.9844]]},
    {"name": "int8_per_channel", "num_bits": 8, "block_sizes": None, "axis": 0,
     "input": [[0, 1, 2, 3, 4, 5, 6, 7]],
     "output": [[0.0000, 0.9922, 1.9844, 2.9844, 3.9688, 4.9688, 5.9688, 7.0000]]},
    {"name": "int8_2d_block", "num_bits": 8, "block_sizes": {"-1": 2, "-2": 2}, "axis": None,
     "input": [[0, 1, 2, 3], [4, 5, 6, 7]],
     "output": [[0.0000, 1.0234, 1.9844, 2.9844], [4.0000, 5.0000, 5.9688, 7.0000]]},
    {"name": "fp8_2d_block", "num_bits": [4, 3], "block_sizes": {"-1": 2, "-2": 2}, "axis": None,
     "input": [[0, 1, 2, 3], [4, 5, 6, 7]],
     "output": [[0.0000, 0.9844, 2.0000, 3.0000], [3.9375, 5.0000, 6.0000, 7.0000]]},
    {"name": "fp8_2d_block_padding", "num_bits": [4, 3], "block_sizes": {"-1": 2, "-2": 2},
     "axis": None, "input": [[0, 1, 3], [4, 5, 7]],
     "output": [[0.0000, 0.9844, 3.0000], [3.9375, 5.0000, 7.0000]]},
    {"name": "fp8_1d_block", "num_bits": [4, 3], "block_sizes": {"-1": 2}, "axis": None,
     "input": [[0, 1, 2, 3], [4, 5, 6, 7]],
     "output": [[0.0000, 1.0000, 1.9219, 3.0000], [3.9375, 5.0000, 6.0000, 7.0000]]},
    {"name": "fp8_per_channel", "num_bits": [4, 3], "block_sizes": None, "axis": 0,
     "input": [[0, 1, 2, 3], [4, 5, 6, 7]],
     "output": [[0.0000, 0.9609, 1.9219, 3.0000], [4.0000, 5.0000, 6.0000, 7.0000]]},
    {"name": "fp8_per_tensor", "num_bits": [4, 3], "block_sizes": None, "axis": None,
     "input": [[0, 1, 2, 3], [4, 5, 6, 7]],
     "output": [[0, 1, 2, 3], [4, 5, 6, 7]]},
]

# tests/gpu/torch/quantization/test_qtensor_cuda.py:111-131 (test_qtensor_accuracy, NF4 rows): real
# quantize through TensorQuantizer (4-bit table codes, int8 double-quantised scales) then
# dequantize; bf16 in, expected bf16 out (torch.allclose), cpu and cuda.
V["nf4_roundtrip"] = [
    {"name": "nf4_block2", "block_size": 2, "scale_block_size": 4, "scale_bits": 8,
     "input": [[0, 1, 2, 3, 4, 5, 6, 7]],
     "output": [[0.0000, 1.0156, 2.1719, 3.0156, 3.6094, 5.0000, 5.0625, 7.0000]]},
    {"name": "nf4_block2_padding", "block_size": 2, "scale_block_size": 4, "scale_bits": 8,
     "input": [[0, 1, 2, 3, 4, 5, 7]],
     "output": [[0.0000, 1.0156, 2.1719, 3.0156, 3.6094, 5.0000, 7.0000]]},
]

# tests/gpu/torch/quantization/test_qtensor_cuda.py:254-375 (test_nvfp4_quantize): block size 8,
# dtypes fp32/fp16/bf16, cpu and cuda; dequantised values allclose(x, rtol=2e-1, atol=2e-1).
V["nvfp4_quantize_inputs"] = [
    [0, 0.5, 1, 1.5, 2, 3, 4, 6, 0, -0.5, -1, -1.5, -2, -3, -4, -6],
    [-0.25, 0.25, 0.75, 1.25, 1.75, 2.75, 3.75, 5.75, -0.25, -0.75, -1.25, -1.75, -2.25, -3.25,
     -4.25, -6.25],
    [0.25, 0.75, 1.25, 1.75, 2.25, 3.25, 4.25, 6.25, 0.25, -0.25, -0.75, -1.25, -1.75, -2.75,
     -3.75, -5.75],
    [0.5, 1.0, 1.5, 2.0, 2.5, 3.5, 4.5, 6.5, 0.5, 0.0, -0.5, -1.0, -1.5, -2.5, -3.5, -5.5],
]

# tests/gpu/torch/quantization/test_qtensor_cuda.py:377-440 (test_cast_fp4_equivalence): fp32
# inputs for which _cast_fp4 must equal the brute-force count-of-bounds twin.
V["cast_fp4_inputs"] = [
    [[0.25, 0.75, 1.25], [1.75, 2.5, 3.5]],
    [[0.1, 2.5, 1.0, 4.8], [1.5, 1.25, 3.25, 5.0]],
    [[0, 0.75, 1.25], [1.75, 2.5, 5.5]],
    [[-0.25, -0.75, -1.25], [-1.75, -2.5, -3.5]],
    [[-0.1, -2.5, -1.0, -4.8], [-1.5, -1.25, -3.25, -5.0]],
    [[0, -0.75, -1.25], [-1.75, -2.5, -5.5]],
]

# tests/gpu/torch/quantization/test_tensor_quant_cuda.py:166-223 (Testfp4.test_cuda_ext_fp4):
# NVFP4 fake quant of [values * sign] repeated to the block size, global amax = max |input|.
# "delta" is added in fp32 to every element but the last before the sign is applied, as the
# test does; "ladder_checked" is False where the reference skips its threshold-ladder kernel.
V["nvfp4_fake_quant_boundaries"] = [
    {"base": [0, 0.5, 1, 1.5, 2, 3, 4, 6], "delta": 0.0, "output": [0, 0.5, 1, 1.5, 2, 3, 4, 6],
     "ladder_checked": True},
    {"base": [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5, 6], "delta": 0.0,
     "output": [0.0, 1, 1, 2, 2, 4, 4, 6], "ladder_checked": False},
    {"base": [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5, 6], "delta": -0.1,
     "output": [0.0, 0.5, 1, 1.5, 2, 3, 4, 6], "ladder_checked": True},
    {"base": [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5, 6], "delta": 0.1,
     "output": [0.5, 1, 1.5, 2, 3, 4, 6, 6], "ladder_checked": True},
]

# tests/unit/torch/quantization/test_utils.py:25-56 (test_reduce_block_amax), bf16.
V["reduce_block_amax"] = [
    {"block_sizes": {"-1": 2, "-2": 2}, "input": [[0, 1, 2, 3], [4, 5, 6, 7]],
     "output": [[5.0, 7.0]]},
    {"block_sizes": {"-1": 4, "-2": 2},
     "input": [[0, 1, 2, 3], [4, 5, 6, 7], [8, 9, 10, 11], [12, 13, 14, 15]],
     "output": [[7.0], [15.0]]},
    {"block_sizes": {"-2": 4},
     "input": [[0, 1, 2, 3], [4, 5, 6, 7], [8, 9, 10, 11], [12, 13, 14, 15]],
     "output": [[12.0, 13.0, 14.0, 15.0]]},
]

# tests/gpu/torch/export/test_export.py:163-197 (test_get_scaling_factor_from_weight): fp32,
# compared with rtol=0, atol=0.
V["scaling_factor_from_weight"] = [
    {"weight": [[0.0, 0.35, 0.28, 7.0], [0.49, 0.84, -0.77, 0.07]], "group_size": 2,
     "expected": [[0.05, 1.0], [0.12, 0.11]]},
    {"weight": [[0.127, 0.0, 1.27, -12.7], [0.0, 127.0, 0.254, 2.54]], "group_size": 0,
     "expected": [0.1, 1.0]},
    {"weight": [[0.0, 0.0, 0.0, 0.0], [0.0, -0.127, 0.254, 2.54]], "group_size": 0,
     "expected": [1.0, 0.02]},
    {"weight": [[0.0, 0.84, -0.77, 0.07], [0.0, 0.0, 0.0, 0.0]], "group_size": 2,
     "expected": [[0.12, 0.11], [1.0, 1.0]]},
]

# tests/gpu/torch/quantization/test_tensor_quant_cuda.py:103-107 (test_cuda_ext_tiny_amax):
# per-channel INT8 fake quant, channel with amax 1e-26 must come out all zero.
V["int_tiny_amax"] = {"shape": [2, 3, 4], "amax": [1.0, 1.0e-26, 1.0], "axis": 1}

# tests/gpu/torch/quantization/test_tensor_quant_cuda.py:43-56: parameter grid the CUDA kernels are
# compared over with atol=0 against the closed-form torch helper
# (tests/_test_utils/torch/quantization/quant_utils.py:19-30).
V["int_qdq_grid"] = {"num_bits": [3, 4, 5, 7, 8, 11], "unsigned": [True, False]}

if __name__ == "__main__":
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.json")
    with open(out, "w") as f:
        json.dump(V, f, indent=1)
    print("wrote", out)
