"""Quantization functionals: autograd Functions over the HIP kernels.

Names, argument order and semantics follow the reference's operator boundary
(modelopt/torch/quantization/tensor_quant.py:62-113 dispatchers, :322-402
``FakeTensorQuantFunction``, :405-463 ``ScaledE4M3Function``, :500-571
``DynamicBlockQuantizationFunction``): forward = fake quantisation, backward = straight-through
estimator that zeroes gradients where ``|x| > amax`` unless ``pass_through_bwd``.
"""

import torch
from torch.autograd import Function

from ... import _hip
from . import kernels
from .config import QuantizerAttributeConfig

__all__ = [
    "FakeTensorQuantFunction", "ScaledE4M3Function", "DynamicBlockQuantizationFunction",
    "fake_tensor_quant", "scaled_e4m3", "dynamic_block_quant", "scaled_e4m3_impl",
    "fake_quant_impl", "fp8_eager", "quantize_op", "dynamic_block_quantize_op",
]

mx_format_map = {(4, 3): "E4M3", (5, 2): "E5M2", (3, 2): "E3M2", (2, 3): "E2M3", 8: "INT8",
                 (8, 0): "E8M0", (2, 1): "E2M1", (1, 2): "E1M2", (0, 3): "E0M3", (3, 0): "E3M0"}

# 0: threshold-ladder NVFP4 fake quant (what the reference's GPU kernels compute);
# 1: identical to NVFP4QTensor.quantize -> dequantize (the reference's CPU path).
NVFP4_FAKE_QUANT_MODE = 0


# What FP8 fake quantisation does with a scaled value beyond the E4M3 range (|x| * 448 / amax
# > 464, i.e. data above the calibrated amax).  The reference has both behaviours: its eager
# torch path -- the only one that runs on a CPU -- casts with ``Tensor.to(float8_e4m3fn)``, which
# gives NaN (tensor_quant.py:45-59), its CUDA kernel clamps to +-448 first
# (src/tensor_quant_gpu_fp8.cu:43).  "nan" is the default here because results are held to the
# CPU path bit for bit; "saturate" is what a deployment wants (a KV-cache value a hair above the
# calibration maximum becomes the maximum instead of poisoning the attention output).
_FP8_OVERFLOW = "nan"


def set_fp8_overflow_behavior(mode: str) -> str:
    """``"nan"`` (eager / CPU semantics, default) or ``"saturate"`` (the CUDA kernel's).  Returns
    the previous mode.

    The mode also governs the E4M3 cast of NVFP4 block scales in *real* quantisation (compress,
    export): the reference casts with torch's non-saturating conversion
    (qtensor/nvfp4_tensor.py:84-91), so a block whose abs-max lies above the per-tensor amax --
    which ``awq_clip`` shrinks for NVFP4 (model_calib.py:869-876) -- stores the NaN byte;
    ``"saturate"`` stores 448 instead, which is what the fake-quant kernel the clip search
    itself ran on computes with."""
    global _FP8_OVERFLOW
    if mode not in ("nan", "saturate"):
        raise ValueError(f"mode must be 'nan' or 'saturate', got {mode!r}")
    previous, _FP8_OVERFLOW = _FP8_OVERFLOW, mode
    _hip.set_option(_hip.MO_OPT_SATURATE_BLOCK_SCALE, int(mode == "saturate"))
    return previous


def get_fp8_overflow_behavior() -> str:
    return _FP8_OVERFLOW


def scaled_e4m3_impl(inputs: torch.Tensor, amax: torch.Tensor | None = None) -> torch.Tensor:
    """FP8 E4M3 fake quantisation with the numerics of the reference's eager path (or, after
    ``set_fp8_overflow_behavior("saturate")``, of its CUDA kernel for out-of-range values)."""
    return kernels.fake_quant_fp8(inputs, amax, saturate=_FP8_OVERFLOW == "saturate")


fp8_eager = scaled_e4m3_impl


def fake_quant_impl(inputs, amax, num_bits=8, unsigned=False, narrow_range=True):
    """Integer fake quantisation; ``amax`` per tensor or with one non-unit run of dims."""
    return kernels.fake_quant_int(inputs, amax, num_bits, unsigned, narrow_range)


def _quantize_impl(inputs, amax, num_bits=8, exponent_bits=0, unsigned=False, narrow_range=True):
    if inputs.dtype == torch.float64:
        # the reference's kernels read a double and compute in float as well
        # (src/tensor_quant_gpu.cu:43-71), so the arithmetic is the fp32 kernel's
        return _quantize_impl(inputs.float(), amax.float(), num_bits, exponent_bits, unsigned,
                              narrow_range).double()
    if num_bits == 8 and exponent_bits == 4:
        return scaled_e4m3_impl(inputs, amax)
    if isinstance(num_bits, int):
        return fake_quant_impl(inputs, amax, num_bits, unsigned, narrow_range)
    raise ValueError(f"Invalid combination of (num_bits, exponent_bits): ({num_bits}, {exponent_bits}).")


def _dynamic_block_quantize_impl(inputs, block_size, amax, num_bits, exponent_bits,
                                 scale_num_bits, scale_exponent_bits):
    scale_bits = (scale_exponent_bits, scale_num_bits - scale_exponent_bits - 1)
    if exponent_bits != 0:
        num_bits = (exponent_bits, num_bits - exponent_bits - 1)
    if num_bits not in mx_format_map:
        raise NotImplementedError(f"Unsupported num_bits: {num_bits}, scale_bits: {scale_bits} "
                                  "for dynamic block quantization.")
    assert scale_bits in mx_format_map, f"Scale bits should be in {mx_format_map.keys()}"
    if scale_bits != (8, 0):
        assert amax is not None and amax.is_cuda, "amax must be a GPU tensor for dynamic block quantization."
        if amax.numel() != 1:
            amax = amax.amax()
        if num_bits == (2, 1) and scale_bits == (4, 3):
            return kernels.fake_quant_nvfp4(inputs, amax, block_size, NVFP4_FAKE_QUANT_MODE)
    else:
        amax = None      # a power-of-two block scale has no global level
    return kernels.fake_quant_block_fp(inputs, block_size, mx_format_map[num_bits],
                                       mx_format_map[scale_bits], amax)


quantize_op = _quantize_impl
dynamic_block_quantize_op = _dynamic_block_quantize_impl

QUANT_DESC_8BIT_PER_TENSOR = QuantizerAttributeConfig(num_bits=8)
QUANT_DESC_UNSIGNED_8BIT_PER_TENSOR = QuantizerAttributeConfig(num_bits=8, unsigned=True)
QUANT_DESC_8BIT_LINEAR_WEIGHT_PER_ROW = QuantizerAttributeConfig(num_bits=8, axis=(0))


def _fake_tensor_quant_backward(inputs, amax, grad_outputs):
    if amax is None:
        return grad_outputs
    zero = grad_outputs.new_zeros(1)
    return torch.where(inputs.abs() <= amax, grad_outputs, zero)


def _backward(ctx, grad_outputs, num_args):
    saved = ctx.saved_tensors
    if len(saved) == 0:
        return (grad_outputs,) + (None,) * (num_args - 1)
    inputs, amax = saved
    return (_fake_tensor_quant_backward(inputs, amax, grad_outputs),) + (None,) * (num_args - 1)


def _save_if_needed(ctx, pass_through_bwd, inputs, amax):
    if not pass_through_bwd and amax is not None:
        if not isinstance(amax, torch.Tensor):
            amax = torch.tensor(amax, device=inputs.device, dtype=inputs.dtype)
        ctx.save_for_backward(inputs, amax)


class FakeTensorQuantFunction(Function):
    """Integer fake quantisation with STE-with-clip backward."""

    @staticmethod
    def forward(ctx, inputs, amax, bias=None, num_bits=8, unsigned=False, narrow_range=True,
                trt_high_precision_dtype=None, pass_through_bwd=False, block_size=None, axis=None):
        if bias is not None:
            inputs = inputs - bias
        _save_if_needed(ctx, pass_through_bwd, inputs, amax)
        outputs = quantize_op(inputs, amax, num_bits=num_bits, exponent_bits=0, unsigned=unsigned,
                              narrow_range=narrow_range)
        if bias is not None:
            outputs = outputs + bias
        return outputs

    @staticmethod
    def backward(ctx, grad_outputs):
        return _backward(ctx, grad_outputs, 10)


class ScaledE4M3Function(Function):
    """FP8 E4M3 fake quantisation with STE-with-clip backward."""

    @staticmethod
    def forward(ctx, inputs, amax, bias, E, M, trt_high_precision_dtype=None,  # noqa: N803
                pass_through_bwd=False):
        if E != 4 or M != 3:
            raise NotImplementedError("Only support E=4 & M=3 for now.")
        if bias is not None:
            inputs = inputs - bias
        _save_if_needed(ctx, pass_through_bwd, inputs, amax)
        outputs = quantize_op(inputs, amax, num_bits=8, exponent_bits=4, unsigned=False,
                              narrow_range=False)
        if bias is not None:
            outputs = outputs + bias
        return outputs

    @staticmethod
    def backward(ctx, grad_outputs):
        return _backward(ctx, grad_outputs, 7)


class DynamicBlockQuantizationFunction(Function):
    """Dynamic block quantisation (NVFP4, MX formats) with pass-through backward by default."""

    @staticmethod
    def forward(ctx, inputs, block_size, amax, bias, num_bits, scale_bits,
                trt_high_precision_dtype=None, onnx_quantizer_type="dynamic", pass_through_bwd=True):
        _save_if_needed(ctx, pass_through_bwd, inputs, amax)
        if isinstance(num_bits, int):
            exponent_bits = 0
        else:
            assert isinstance(num_bits, tuple) and len(num_bits) == 2
            exponent_bits = num_bits[0]
            num_bits = num_bits[0] + num_bits[1] + 1
        assert isinstance(scale_bits, tuple) and len(scale_bits) == 2
        return dynamic_block_quantize_op(inputs, block_size, amax, num_bits, exponent_bits,
                                         scale_bits[0] + scale_bits[1] + 1, scale_bits[0])

    @staticmethod
    def backward(ctx, grad_outputs):
        return _backward(ctx, grad_outputs, 9)


fake_tensor_quant = FakeTensorQuantFunction.apply
scaled_e4m3 = ScaledE4M3Function.apply
dynamic_block_quant = DynamicBlockQuantizationFunction.apply
