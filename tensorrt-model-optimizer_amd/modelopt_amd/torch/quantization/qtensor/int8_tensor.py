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
        layout = kernels.layout_from_amax_shape(tuple(x.shape), tuple(scales.shape))
        if layout is None:
            raise NotImplementedError("scale shape not covered by the kernels")
        via = torch.result_type(x, scales)
        q = _hip.real_quantize(x, scales.reshape(-1).contiguous(), *layout, via, _hip.MO_FMT_INT8)
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
        layout = kernels.layout_from_amax_shape(tuple(q.shape), tuple(scales.shape))
        return _hip.real_dequantize(q.view(torch.uint8), scales.reshape(-1).contiguous(), *layout,
                                    _hip.MO_FMT_INT8, dtype)
