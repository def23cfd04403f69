"""NF4 real quantisation with double-quantised scales (reference: qtensor/nf4_tensor.py:25-201),
CPU-branch numerics: the table is the bf16 rounding of the NF4 constants, the nearest entry is
found on differences rounded to the input dtype, lowest index among equal differences."""

import math

import torch

from .... import _hip
from ..utils import reduce_amax, reduce_block_padding
from .base_qtensor import BaseQuantizedTensor

__all__ = ["NF4QTensor"]

nf4_table = torch.tensor(
    [-1.0000, -0.6962, -0.5251, -0.3949, -0.2844, -0.1848, -0.0911, 0.0000,
     0.0796, 0.1609, 0.2461, 0.3379, 0.4407, 0.5626, 0.7230, 1.0000], dtype=torch.bfloat16)


def _dequantize_scalers(scales, double_scale, scale_zeros, dtype):
    """int8 scales -> ``dtype``: every scale block divided by its own factor, plus the mean.

    The reference divides the flattened scales by ``double_scale.unsqueeze(-1)`` (nf4_tensor.py:
    50-51), which is this expression when there is one scale block -- the only case its tests
    exercise -- and a shape error on its CPU path otherwise."""
    rows = double_scale.numel()
    return ((scales.reshape(rows, -1) / double_scale.reshape(rows, 1)).to(dtype) + scale_zeros).flatten()


class NF4QTensor(BaseQuantizedTensor):
    """Two 4-bit table indices per byte (high nibble first) over flat blocks."""

    @classmethod
    def quantize(cls, input: torch.Tensor, block_size: int, scale_block_size: int | None = None) -> tuple:
        """-> (NF4QTensor, per-block abs-max scales zero padded to whole scale blocks)."""
        packed, scales = _hip.nf4_quantize(input.contiguous().view(-1), block_size)
        if scale_block_size:
            scales = reduce_block_padding(scales, block_sizes={-1: scale_block_size})
        return cls(input.shape, input.dtype, packed), scales

    @classmethod
    def double_quantization(cls, scales: torch.Tensor, scale_block_size: int, num_scale_bits: int):
        """Scales -> int8 per scale block: (int8 [n / sbs, sbs], ``bound / amax`` [n / sbs], mean)."""
        assert scales.numel() % scale_block_size == 0, (
            "Number of scales elements is not divisible by the scale block size.")
        bound = 2 ** (num_scale_bits - 1) - 1
        block_scales = scales.view(-1, scale_block_size)
        zero_point = block_scales.mean()
        block_scales = block_scales - zero_point
        factor = bound / reduce_amax(block_scales, -1)
        q = block_scales * factor.expand(block_scales.shape[0], scale_block_size)
        q = q.round().clamp(-bound, bound).to(torch.int8)
        return q, factor.flatten(), zero_point

    def dequantize(self, dtype: torch.dtype = None, **kwarg):
        if dtype is None:
            dtype = self.metadata["dtype"]
        block = kwarg["block_sizes"][-1]
        data = self._quantized_data.contiguous().view(-1)
        dev = data.device
        n_blocks = data.numel() * 2 // block
        scales = _dequantize_scalers(kwarg["scale"].to(dev), kwarg["double_scale"].to(dev),
                                     kwarg["scale_zeros"].to(dev), dtype)[:n_blocks].contiguous()
        flat = _hip.nf4_dequantize(data, scales, block)
        n = math.prod(self.metadata["shape"])
        return flat[:n].reshape(self.metadata["shape"]).to(dtype)
