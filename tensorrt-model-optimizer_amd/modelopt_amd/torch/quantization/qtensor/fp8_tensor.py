"""FP8 E4M3 real quantisation (reference: qtensor/fp8_tensor.py:33-151)."""

import torch

from .... import _hip
from .. import kernels
from ..utils import (convert_quantization_axis_to_reduce_axis, reduce_amax, reduce_block_amax,
                     true_divide)
from .base_qtensor import BaseQuantizedTensor

__all__ = ["FP8QTensor"]


def _block_layout(x, scales, block_sizes):
    """[outer, axis, inner] of a 1-D block layout along the last dim, or raise."""
    dims = {d % x.dim() for d in block_sizes}
    if dims != {x.dim() - 1}:
        raise NotImplementedError("only block scales along the last dim are covered by the kernels")
    blk = block_sizes[-1] if -1 in block_sizes else block_sizes[x.dim() - 1]
    if x.shape[-1] % blk:
        raise NotImplementedError("block scales with padding are not covered by the kernels")
    return 1, x.numel() // blk, blk


class FP8QTensor(BaseQuantizedTensor):
    """One ``float8_e4m3fn`` per element plus per-tensor / per-channel / per-block scales."""

    @classmethod
    def quantize(cls, input, scales=None, axis=None, block_sizes=None) -> tuple:
        x = input.contiguous()
        if scales is None:
            if block_sizes:
                amax = reduce_block_amax(x, block_sizes)
            else:
                amax = reduce_amax(x, axis=convert_quantization_axis_to_reduce_axis(x, axis))
            scales = true_divide(amax, 448.0)
        if block_sizes:
            layout = _block_layout(x, scales, block_sizes)
        else:
            layout = kernels.layout_from_amax_shape(tuple(x.shape), tuple(scales.shape))
            if layout is None:
                raise NotImplementedError("scale shape not covered by the kernels")
        via = torch.result_type(x, scales)
        q = _hip.real_quantize(x, scales.reshape(-1).contiguous(), *layout, via, _hip.MO_FMT_E4M3)
        return cls(input.shape, input.dtype, q), scales

    def dequantize(self, dtype: torch.dtype = None, **kwarg):
        if dtype is None:
            dtype = self.metadata["dtype"]
        assert "scale" in kwarg, "Require scale for FP8 dequantization."
        scales, block_sizes = kwarg["scale"], kwarg.get("block_sizes")
        q = self._quantized_data.contiguous()
        scales = scales.to(q.device)
        if block_sizes:
            layout = _block_layout(q, scales, block_sizes)
        else:
            layout = kernels.layout_from_amax_shape(tuple(q.shape), tuple(scales.shape))
        return _hip.real_dequantize(q, scales.reshape(-1).contiguous(), *layout, _hip.MO_FMT_E4M3, dtype)
