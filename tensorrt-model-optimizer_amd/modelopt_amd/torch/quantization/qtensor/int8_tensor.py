"""INT8 real quantisation (reference: qtensor/int8_tensor.py:30-130)."""

import torch

from .... import _hip
from .. import kernels
from ..utils import convert_quantization_axis_to_reduce_axis, reduce_amax, true_divide
from .base_qtensor import BaseQuantizedTensor
from .fp8_tensor import _block_dequantize, _block_quantize

__all__ = ["INT8QTensor"]


class INT8QTensor(BaseQuantizedTensor):
    """One int8 per element plus scales ``amax / 127``."""

    @classmethod
    def quantize(cls, input, scales=None, axis=None, block_sizes=None) -> tuple:
        if block_sizes:
            return _block_quantize(cls, input, scales, block_sizes, 127.0, _hip.MO_FMT_INT8, crop=False)
        x = input.contiguous()
        if scales is None:
            amax = reduce_amax(x, axis=convert_quantization_axis_to_reduce_axis(x, axis))
            scales = true_divide(amax, 127.0)
        via = torch.result_type(x, scales)
        # scales on two separated runs of dims go through a transposing copy, like fake quant
        q = kernels.with_scale_layout(x, scales, lambda x2, s, outer, axis, inner: _hip.real_quantize(
            x2, s, outer, axis, inner, via, _hip.MO_FMT_INT8))
        return cls(input.shape, input.dtype, q), scales

    def dequantize(self, dtype: torch.dtype = None, **kwarg):
        if dtype is None:
            dtype = self.metadata["dtype"]
        assert "scale" in kwarg, "Require scale for INT8 dequantization."
        scales, block_sizes = kwarg["scale"], kwarg.get("block_sizes")
        q = self._quantized_data.contiguous()
        scales = scales.to(q.device)
        if block_sizes:
            return _block_dequantize(q, self.metadata["shape"], scales, block_sizes,
                                     _hip.MO_FMT_INT8, dtype)
        return kernels.with_scale_layout(q, scales, lambda q2, s, outer, axis, inner: _hip.real_dequantize(
            q2.view(torch.uint8), s, outer, axis, inner, _hip.MO_FMT_INT8, dtype))
