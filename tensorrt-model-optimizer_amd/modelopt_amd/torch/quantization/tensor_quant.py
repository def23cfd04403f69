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
from . import kernels, modes
from .config import QuantizerAttributeConfig
from .overflow import fp8_saturates, get_fp8_overflow_behavior, set_fp8_overflow_behavior  # noqa: F401

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


def scaled_e4m3_impl(inputs: torch.Tensor, amax: torch.Tensor | None = None) -> torch.Tensor:
    """FP8 E4M3 fake quantisation.  Out-of-range values follow the reference's dispatch
    (tensor_quant.py:62-90): clamped where its CUDA kernel runs (per-tensor or per-axis amax),
    NaN where it falls back to the eager cast; see ``overflow.set_fp8_overflow_behavior``."""
    return kernels.fake_quant_fp8(inputs, amax, saturate=fp8_saturates(amax))


def fp8_eager(inputs: torch.Tensor, amax: torch.Tensor | None = None) -> torch.Tensor:
    """The reference's eager expression (tensor_quant.py:45-59): the non-saturating cast, NaN
    beyond the E4M3 range, whatever the overflow mode."""
    return kernels.fake_quant_fp8(inputs, amax, saturate=False)


_fp8_eager = fp8_eager   # the reference keeps the body under this name (tensor_quant.py:45)

# the reference's switch between its two NVFP4 fake-quant kernels (tensor_quant.py:42); there is
# one kernel here, so the flag is accepted and changes nothing
DISABLE_TRITON_KERNEL = False


def _tensor_quant(inputs, amax, num_bits=8, unsigned=False, narrow_range=True):
    """The reference's eager body (tensor_quant.py:574-612) by name: its two looks at the data on
    the host happen here whatever the strict mode -- negative inputs with ``unsigned`` raise
    ``TypeError``, a negative amax raises ``ValueError`` -- then the kernel."""
    if unsigned and inputs.numel() and inputs.min() < 0.0:
        raise TypeError("Negative values encountered in unsigned quantization.")
    if amax.numel() and amax.min() < 0:
        raise ValueError("Negative values in amax")
    return kernels.fake_quant_int(inputs, amax, num_bits, unsigned, narrow_range)



def fake_quant_impl(inputs, amax, num_bits=8, unsigned=False, narrow_range=True):
    """Integer fake quantisation; ``amax`` per tensor or with one non-unit run of dims.

    The reference's CPU path first looks at the data on the host (tensor_quant.py:577-587):
    negative inputs with ``unsigned=True`` raise ``TypeError``, a negative amax raises
    ``ValueError``.  Its CUDA kernel clamps instead, and so does this function unless
    ``modes.set_strict_checks(True)`` asks for the CPU path's errors (two host synchronisations
    per call)."""
    if modes.strict_checks():
        if unsigned and inputs.numel() and inputs.min() < 0.0:
            raise TypeError("Negative values encountered in unsigned quantization.")
        if amax.numel() and amax.min() < 0:
            raise ValueError("Negative values in amax")
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


def _like_input(inputs, *_args, **_kwargs):
    """Fake (meta) implementation of both operators: same shape and dtype as the input."""
    return torch.empty_like(inputs)


def _register_operators():
    """``tensorrt::quantize_op`` and ``tensorrt::dynamic_block_quantize_op`` (+ ``.overload`` for
    ``amax=None``) with the reference's schemas (tensor_quant.py:221-273), so that a traced or
    exported graph of a quantised model carries the same operator nodes.  Returns the two
    callables; the plain Python functions if registration is impossible (e.g. the names are
    already taken by the reference package loaded in the same process)."""
    try:
        torch.library.define(
            "tensorrt::quantize_op",
            "(Tensor input, Tensor amax, int num_bits, int exponent_bits, "
            "bool unsigned, bool narrow_range) -> Tensor")
        torch.library.define(
            "tensorrt::dynamic_block_quantize_op",
            "(Tensor input, int block_size, Tensor amax, int num_bits, int exponent_bits, "
            "int scale_num_bits, int scale_exponent_bits) -> Tensor")
        torch.library.define(
            "tensorrt::dynamic_block_quantize_op.overload",
            "(Tensor input, int block_size, None amax, int num_bits, int exponent_bits, "
            "int scale_num_bits, int scale_exponent_bits) -> Tensor")
        torch.library.impl("tensorrt::quantize_op", ["cpu", "cuda"])(_quantize_impl)
        torch.library.impl("tensorrt::dynamic_block_quantize_op", ["cpu", "cuda"])(
            _dynamic_block_quantize_impl)
        # the reference's implementation of the amax=None overload returns an uninitialised
        # tensor (tensor_quant.py:241-251); here it quantises (MX formats need no global amax)
        torch.library.impl("tensorrt::dynamic_block_quantize_op.overload", ["cpu", "cuda"])(
            _dynamic_block_quantize_impl)
        for name in ("quantize_op", "dynamic_block_quantize_op", "dynamic_block_quantize_op.overload"):
            torch.library.register_fake("tensorrt::" + name)(_like_input)
        return torch.ops.tensorrt.quantize_op, torch.ops.tensorrt.dynamic_block_quantize_op
    except (AttributeError, RuntimeError) as e:
        import warnings

        warnings.warn("Unable to register operators with torch.library. Exporting quantized models "
                      f"with torch.export will not be supported.\n{e}")
        return _quantize_impl, _dynamic_block_quantize_impl


_quantize_operator, dynamic_block_quantize_op = _register_operators()


def quantize_op(inputs, amax, num_bits=8, exponent_bits=0, unsigned=False, narrow_range=True):
    """``tensorrt::quantize_op``; the operator's schema wants a tensor amax and 32-bit floating
    inputs or narrower, so ``amax=None`` (a plain E4M3 cast) and float64 go to the function."""
    if amax is None or inputs.dtype == torch.float64 or not isinstance(amax, torch.Tensor):
        return _quantize_impl(inputs, amax, num_bits, exponent_bits, unsigned, narrow_range)
    return _quantize_operator(inputs, amax, num_bits, exponent_bits, unsigned, narrow_range)


QUANT_DESC_8BIT_PER_TENSOR = QuantizerAttributeConfig(num_bits=8)
QUANT_DESC_UNSIGNED_8BIT_PER_TENSOR = QuantizerAttributeConfig(num_bits=8, unsigned=True)
QUANT_DESC_8BIT_LINEAR_WEIGHT_PER_ROW = QuantizerAttributeConfig(num_bits=8, axis=(0))
# the per-output-channel descriptors of the convolution wrappers (tensor_quant.py:286-292): same content
QUANT_DESC_8BIT_CONV1D_WEIGHT_PER_CHANNEL = QuantizerAttributeConfig(num_bits=8, axis=(0))
QUANT_DESC_8BIT_CONV2D_WEIGHT_PER_CHANNEL = QuantizerAttributeConfig(num_bits=8, axis=(0))
QUANT_DESC_8BIT_CONV3D_WEIGHT_PER_CHANNEL = QuantizerAttributeConfig(num_bits=8, axis=(0))
QUANT_DESC_8BIT_CONVTRANSPOSE1D_WEIGHT_PER_CHANNEL = QuantizerAttributeConfig(num_bits=8, axis=(0))
QUANT_DESC_8BIT_CONVTRANSPOSE2D_WEIGHT_PER_CHANNEL = QuantizerAttributeConfig(num_bits=8, axis=(0))
QUANT_DESC_8BIT_CONVTRANSPOSE3D_WEIGHT_PER_CHANNEL = QuantizerAttributeConfig(num_bits=8, axis=(0))


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


class _NoGraph:
    """Stands in for the autograd context when nothing will be differentiated."""

    @staticmethod
    def save_for_backward(*tensors):
        pass


def _entry(function):
    """``function.apply``, except that a call whose result cannot need a gradient (grad mode off,
    or an input that does not require one) runs the forward directly: Function.apply costs
    several microseconds of host time per quantizer call even then."""
    def run(inputs, *args, **kwargs):
        if torch.is_grad_enabled() and isinstance(inputs, torch.Tensor) and inputs.requires_grad:
            return function.apply(inputs, *args, **kwargs)
        return function.forward(_NoGraph, inputs, *args, **kwargs)
    run.__name__ = function.__name__
    run.__doc__ = function.__doc__
    return run


fake_tensor_quant = _entry(FakeTensorQuantFunction)
scaled_e4m3 = _entry(ScaledE4M3Function)
dynamic_block_quant = _entry(DynamicBlockQuantizationFunction)
