"""The seam where the reference loads its CUDA extensions (modelopt/torch/quantization/
extensions.py:27-70): the same three accessors, returning objects that expose the same function
names, here bound to the HIP library.  There is no JIT build and no eager fallback -- if the
library is missing the accessors raise.
"""

import torch

from ... import _hip
from . import kernels

__all__ = ["get_cuda_ext", "get_cuda_ext_fp8", "get_cuda_ext_mx"]


class _IntExt:
    """Counterpart of ``modelopt_cuda_ext`` (TQ/src/tensor_quant.cpp:63-77)."""

    @staticmethod
    def fake_tensor_quant(inputs, amax, num_bits=8, unsigned=False, narrow_range=True):
        return kernels.fake_quant_int(inputs, amax.reshape(()), num_bits, unsigned, narrow_range)

    @staticmethod
    def fake_tensor_quant_(inputs, amax, num_bits=8, unsigned=False, narrow_range=True):
        assert inputs.is_contiguous(), "in-place fake quant needs a contiguous tensor"
        _hip.int_qdq(inputs, amax.reshape(1), 1, 1, inputs.numel(), num_bits, unsigned,
                     narrow_range, out=inputs)

    @staticmethod
    def fake_tensor_quant_with_axis(inputs, amax, axis, num_bits=8, unsigned=False,
                                    narrow_range=True):
        x = inputs if inputs.is_contiguous() else inputs.contiguous()
        axis = axis % x.dim()
        outer, n, inner = kernels.amax_layout(tuple(x.shape), [axis])
        assert amax.numel() == x.shape[axis]
        return _hip.int_qdq(x, amax.reshape(-1).contiguous(), outer, x.shape[axis], inner, num_bits,
                            unsigned, narrow_range)

    @staticmethod
    def INT4_quantize(input_flat, scales, block_size):  # noqa: N802
        """``clamp(round(input * scales[block]), -8, 7) + 8`` packed two per byte with the
        caller's per-block scales (rounding follows the reference's tensor expression,
        qtensor/int4_tensor.py:69-83: product in the input dtype, ties to even)."""
        scales = scales.to(input_flat.dtype).contiguous()
        packed, _ = _hip.int4_block_quantize(input_flat.contiguous(), block_size, scales)
        return packed

    @staticmethod
    def INT4_dequantize(q_flat, scales, block_size):  # noqa: N802
        return _hip.int4_block_dequantize(q_flat.contiguous(), scales.contiguous(), block_size)


class _Fp8Ext:
    """Counterpart of ``modelopt_cuda_ext_fp8`` (TQ/src/tensor_quant_gpu_fp8.cu:103-108)."""

    @staticmethod
    def fake_e4m3fy(inputs, amax):
        # the CUDA kernel this stands in for clamps to +-448 before the cast
        return kernels.fake_quant_fp8(inputs, amax.reshape(()), saturate=True)

    @staticmethod
    def fake_e4m3fy_with_axis(inputs, amax, axis):
        x = inputs if inputs.is_contiguous() else inputs.contiguous()
        axis = axis % x.dim()
        outer, n, inner = kernels.amax_layout(tuple(x.shape), [axis])
        return _hip.fp8_qdq(x, amax.reshape(-1).contiguous(), outer, x.shape[axis], inner, True)


class _MxTypes:
    E4M3, E5M2, INT8, E0M3, E1M2, E3M0, E2M1, E3M2, E2M3, E8M0 = range(10)


class _MxExt:
    """Counterpart of ``modelopt_cuda_ext_mx`` (TQ/src/tensor_quant_mx.cu:393-411)."""

    Types = _MxTypes
    _names = ["E4M3", "E5M2", "INT8", "E0M3", "E1M2", "E3M0", "E2M1", "E3M2", "E2M3", "E8M0"]

    @staticmethod
    def fused_amax_convert(inputs, block_size, format, scale_format, global_amax=None):
        if block_size not in (8, 16, 32):
            raise ValueError("Blocksize for fused call must be one of {8, 16, 32}")
        return kernels.fake_quant_block_fp(inputs, block_size, _MxExt._names[int(format)],
                                           _MxExt._names[int(scale_format)], global_amax)

    @staticmethod
    def convert_to_exmy(x, format):
        """One Python float to the nearest value of ``format`` (the reference's host helper,
        TQ/src/tensor_quant_mx.cu:398); computed by the device code that the kernels use."""
        t = torch.tensor([float(x)], dtype=torch.float32, device="cuda")
        return float(_hip.convert_to_format(t, int(format)).item())


def _loaded(raise_if_failed):
    try:
        _hip.load()
        return True
    except RuntimeError:
        if raise_if_failed:
            raise
        return False


def get_cuda_ext(raise_if_failed: bool = False):
    return _IntExt if _loaded(raise_if_failed) else None


def get_cuda_ext_fp8(raise_if_failed: bool = False):
    return _Fp8Ext if _loaded(raise_if_failed) else None


def get_cuda_ext_mx(raise_if_failed: bool = False):
    return _MxExt if _loaded(raise_if_failed) else None
