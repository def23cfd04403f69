"""Oracle: NF4 real quantisation with double-quantised scales (test infrastructure).

Restates the CPU branch of the reference's ``NF4QTensor``, TQ/qtensor/nf4_tensor.py:25-46 (table),
:54-62 (nearest table entry), :76-126 (quantize), :128-155 (double quantisation of the scales),
:157-201 (dequantize), in the same torch CPU ops and dtypes.  Pinned by the reference's golden
vectors tests/gpu/torch/quantization/test_qtensor_cuda.py:111-131 (values after a quantize /
dequantize round trip, with and without input padding) and :30-68 (round trip within 0.1).
"""

import math

import torch

from .reduce import reduce_amax, reduce_block_padding

# TQ/qtensor/nf4_tensor.py:25-46: the table is *stored in bf16*, so every use sees the
# bf16-rounded constants
NF4_TABLE = torch.tensor(
    [-1.0000, -0.6962, -0.5251, -0.3949, -0.2844, -0.1848, -0.0911, 0.0000,
     0.0796, 0.1609, 0.2461, 0.3379, 0.4407, 0.5626, 0.7230, 1.0000], dtype=torch.bfloat16)


def nearest_table_index(flat: torch.Tensor, lut: torch.Tensor) -> torch.Tensor:
    """Index of the table entry with the smallest ``|x - entry|``, the difference and its
    absolute value taken in the dtype of ``flat``; first index among equal differences, index
    of the first NaN when there is one (torch.argmin).  TQ/qtensor/nf4_tensor.py:54-62."""
    assert flat.dim() == 1
    return (flat[:, None] - lut).abs().argmin(dim=-1)


def nf4_quantize(x: torch.Tensor, block_size: int, scale_block_size: int):
    """-> (packed uint8 [padded_numel / 2], scales [padded number of blocks], input dtype).
    ``byte = index[2i] << 4 | index[2i + 1]``.  TQ/qtensor/nf4_tensor.py:93-126 (CPU branch)."""
    flat = reduce_block_padding(x.reshape(-1), {-1: block_size})
    blocks = flat.view(-1, block_size)
    scales = reduce_amax(blocks, -1)
    scaled = blocks / scales.view(blocks.shape[0], -1)
    idx = nearest_table_index(scaled.flatten(), NF4_TABLE.to(dtype=x.dtype)).to(torch.uint8)
    packed = idx[::2] << 4 | idx[1::2]
    scales = reduce_block_padding(scales.view(-1), {-1: scale_block_size})
    return packed, scales


def double_quantization(scales: torch.Tensor, scale_block_size: int, num_scale_bits: int):
    """Scales -> (int8 [n / sbs, sbs], per-scale-block factor ``127 / amax`` [n / sbs], mean).
    TQ/qtensor/nf4_tensor.py:128-155."""
    assert scales.numel() % scale_block_size == 0
    bound = 2 ** (num_scale_bits - 1) - 1
    block_scales = scales.view(-1, scale_block_size)
    zero_point = block_scales.mean()
    block_scales = block_scales - zero_point
    factor = bound / reduce_amax(block_scales, -1)
    q = block_scales * factor.expand(block_scales.shape[0], scale_block_size)
    q = q.round().clamp(-bound, bound).to(torch.int8)
    return q, factor.flatten(), zero_point


def dequantize_scales(scales, double_scale, scale_zeros, dtype):
    """TQ/qtensor/nf4_tensor.py:50-51, applied per scale block.  The reference divides the
    *flattened* int8 scales by ``double_scale.unsqueeze(-1)``, which only has the intended
    meaning (and only runs) when there is a single scale block -- the case all of its tests
    use; with one block the two forms are the same expression."""
    rows = double_scale.numel()
    return ((scales.view(rows, -1) / double_scale.view(rows, 1)).to(dtype) + scale_zeros).flatten()


def nf4_dequantize(packed, scales_int8, double_scale, scale_zeros, block_size, shape, dtype):
    """TQ/qtensor/nf4_tensor.py:157-201 (CPU branch): ``table[index] * scale`` in the promoted
    dtype of (bf16 table, ``dtype`` scales), then cast to ``dtype``."""
    n_blocks = packed.numel() * 2 // block_size
    scales = dequantize_scales(scales_int8, double_scale, scale_zeros, dtype)[:n_blocks]
    hi = NF4_TABLE[(packed >> 4).long()].view(-1, block_size // 2) * scales.view(-1, 1)
    lo = NF4_TABLE[(packed & 0x0F).long()].view(-1, block_size // 2) * scales.view(-1, 1)
    out = torch.stack([hi.flatten(), lo.flatten()], dim=-1).view(-1)
    return out[:math.prod(shape)].reshape(shape).to(dtype)
