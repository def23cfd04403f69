"""INT4 block real quantisation (reference: qtensor/int4_tensor.py:28-130), CPU-branch numerics."""

import math

import torch

from .... import _hip
from .base_qtensor import BaseQuantizedTensor

__all__ = ["INT4QTensor"]


class INT4QTensor(BaseQuantizedTensor):
    """Two 4-bit values per byte (high nibble first), flat blocks, inverse scales ``7 / amax``."""

    @staticmethod
    def _get_quant_maxbound(num_bits):
        return 2 ** (num_bits - 1) - 1

    @classmethod
    def quantize(cls, input: torch.Tensor, block_size: int) -> tuple:
        assert input.shape[-1] % 2 == 0, "Input tensor must have even number on last dimension."
        packed, scales = _hip.int4_block_quantize(input.contiguous().view(-1), block_size)
        packed = packed.reshape(*input.shape[:-1], -1)
        return cls(input.shape, input.dtype, packed), scales

    def dequantize(self, dtype: torch.dtype = None, **kwarg):
        if dtype is None:
            dtype = self.metadata["dtype"]
        scales, block = kwarg["scale"], kwarg["block_sizes"][-1]
        flat = _hip.int4_block_dequantize(self._quantized_data.contiguous().view(-1),
                                          scales.to(self._quantized_data.device).contiguous(), block)
        n = math.prod(self.metadata["shape"])
        return flat[:n].view(self.metadata["shape"]).to(dtype)
