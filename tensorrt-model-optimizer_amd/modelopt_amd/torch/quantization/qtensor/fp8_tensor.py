"""FP8 E4M3 real quantisation (reference: qtensor/fp8_tensor.py:33-151)."""

import math

import torch

from .... import _hip
from .. import kernels
from ..utils import convert_quantization_axis_to_reduce_axis, reduce_amax, true_divide
from ._blocks import BlockRows
from .base_qtensor import BaseQuantizedTensor

__all__ = ["FP8QTensor"]


def _last_two_dims_blocks(br):
    """``(rows, cols, block_rows, block_cols)`` of the padded tensor when the blocks of ``br`` are on
    its last two dims (a stack of matrices cut into tiles) and the kernels for that layout take
    them: the casts then run in place instead of on a copy with every block gathered into a row."""
    nd = len(br.padded)
    if nd < 2 or len(br.split) != nd + 2 or br.perm[-2:] != [len(br.split) - 3, len(br.split) - 1]:
        return None
    block_rows, block_cols = br.split[-3], br.split[-1]
    if block_cols % 8:
        return None
    return math.prod(br.padded[:-1]), br.padded[-1], block_rows, block_cols


def _block_quantize(cls, input, scales, block_sizes, bound, fmt, crop=True):
    """Shared by the FP8 and INT8 containers: block scales on any dims, zero padding.  The FP8
    container stores the codes cropped to the input shape, the INT8 container stores them
    padded (reference: fp8_tensor.py:108-112 against int8_tensor.py:86-88)."""
    br = BlockRows(input.shape, block_sizes)
    tiles = _last_two_dims_blocks(br) if input.is_cuda else None
    if tiles is not None:
        x = br.pad(input).contiguous()
        if x.data_ptr() % 16 == 0:
            if scales is None:
                amax = reduce_amax(x.reshape(br.split), axis=[len(br.split) - 3, len(br.split) - 1],
                                   keepdims=False, squeeze_scalar=False)
                scales = true_divide(amax, bound).reshape(br.scale_shape)
            elif tuple(scales.shape) != br.scale_shape:
                assert scales.numel() == br.rows, (
                    f"Mismatch in expected scale shape: {tuple(scales.shape)} vs {br.scale_shape}")
                scales = scales.reshape(br.scale_shape)
            q = _hip.real_quantize_blocks2d(x, scales.reshape(-1).contiguous(), *tiles,
                                            torch.result_type(input, scales), fmt)
            if crop and br.padded != br.shape:
                q = q[tuple(slice(0, s) for s in br.shape)].contiguous()
            return cls(input.shape, input.dtype, q), scales
    rows = br.to_rows(input)
    if scales is None:
        amax = reduce_amax(rows, axis=1, keepdims=False, squeeze_scalar=False)
        scales = true_divide(amax, bound).reshape(br.scale_shape)
    elif tuple(scales.shape) != br.scale_shape:
        assert scales.numel() == br.rows, (
            f"Mismatch in expected scale shape: {tuple(scales.shape)} vs {br.scale_shape}")
        scales = scales.reshape(br.scale_shape)
    via = torch.result_type(input, scales)
    q = _hip.real_quantize(rows, scales.reshape(-1).contiguous(), 1, br.rows, br.block, via, fmt)
    return cls(input.shape, input.dtype, br.from_rows(q, crop)), scales


def _block_dequantize(q, shape, scales, block_sizes, fmt, dtype):
    br = BlockRows(shape, block_sizes)
    assert tuple(scales.shape) == br.scale_shape, (
        f"Scales shape {tuple(scales.shape)} must match expected {br.scale_shape}.")
    tiles = _last_two_dims_blocks(br) if q.is_cuda else None
    if tiles is not None:
        codes = br.pad(q.view(torch.uint8)).contiguous()
        if codes.data_ptr() % 8 == 0:
            y = _hip.real_dequantize_blocks2d(codes, scales.reshape(-1).contiguous(), *tiles, fmt, dtype)
            if br.padded != br.shape:
                y = y[tuple(slice(0, s) for s in br.shape)].contiguous()
            return y
    rows = br.to_rows(q.view(torch.uint8))
    y = _hip.real_dequantize(rows, scales.reshape(-1).contiguous(), 1, br.rows, br.block, fmt, dtype)
    return br.from_rows(y)


class FP8QTensor(BaseQuantizedTensor):
    """One ``float8_e4m3fn`` per element plus per-tensor / per-channel / per-block scales."""

    @classmethod
    def quantize(cls, input, scales=None, axis=None, block_sizes=None) -> tuple:
        if block_sizes:
            return _block_quantize(cls, input, scales, block_sizes, 448.0, _hip.MO_FMT_E4M3)
        x = input.contiguous()
        if scales is None:
            amax = reduce_amax(x, axis=convert_quantization_axis_to_reduce_axis(x, axis))
            scales = true_divide(amax, 448.0)
        via = torch.result_type(x, scales)
        # scales on two separated runs of dims go through a transposing copy, like fake quant
        q = kernels.with_scale_layout(x, scales, lambda x2, s, outer, axis, inner: _hip.real_quantize(
            x2, s, outer, axis, inner, via, _hip.MO_FMT_E4M3))
        return cls(input.shape, input.dtype, q), scales

    def dequantize(self, dtype: torch.dtype = None, **kwarg):
        if dtype is None:
            dtype = self.metadata["dtype"]
        assert "scale" in kwarg, "Require scale for FP8 dequantization."
        scales, block_sizes = kwarg["scale"], kwarg.get("block_sizes")
        q = self._quantized_data.contiguous()
        scales = scales.to(q.device)
        if block_sizes:
            return _block_dequantize(q, self.metadata["shape"], scales, block_sizes,
                                     _hip.MO_FMT_E4M3, dtype)
        return kernels.with_scale_layout(q, scales, lambda q2, s, outer, axis, inner: _hip.real_dequantize(
            q2, s, outer, axis, inner, _hip.MO_FMT_E4M3, dtype))
