"""MXFP4 real-quantised tensor (reference: qtensor/mxfp4_tensor.py:25-144)."""

import torch

from .... import _hip
from .base_qtensor import BaseQuantizedTensor

__all__ = ["MXFP4QTensor"]


class MXFP4QTensor(BaseQuantizedTensor):
    """E2M1 codes, two per byte, with one E8M0 scale byte per block of the flattened tensor."""

    E2M1_max = 6.0
    E2M1_values = [0, 0.5, 1, 1.5, 2, 3, 4, 6]

    @classmethod
    def quantize(cls, input: torch.Tensor, block_size: int | None) -> tuple:
        """-> (MXFP4QTensor, e8m0 scale bytes ``uint8 [numel / block_size, 1]``)."""
        if block_size is None:
            block_size = 32
        x = input if input.is_contiguous() else input.contiguous()
        packed, scales = _hip.mxfp4_quantize(x, block_size)
        return cls(input.shape, input.dtype, packed), scales

    def dequantize(self, dtype: torch.dtype = None, **kwarg):
        scale = kwarg["scale"]
        block_size = kwarg["block_sizes"][-1]
        if dtype is None:
            dtype = self.metadata["dtype"]
        out = _hip.mxfp4_dequantize(self._quantized_data.contiguous(), scale.contiguous(),
                                    block_size, dtype)
        return out.reshape(self.metadata["shape"])
