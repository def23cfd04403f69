"""Oracle: real quantize + pack and dequantize (test infrastructure, CPU torch)."""

import math

import torch

from .reduce import (
    quant_axis_to_reduce_dims,
    reduce_amax,
    reduce_block_amax,
    reduce_block_padding,
)

E2M1_BOUNDS = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5])
E2M1_LUT = torch.tensor([0, 0.5, 1, 1.5, 2, 3, 4, 6, 0, -0.5, -1, -1.5, -2, -3, -4, -6])


# ----------------------------------------------------------------------------- NVFP4


def nvfp4_global_scale(x: torch.Tensor):
    """wsf2 = f32(amax(x)) / (6*448).  Follows TQ/qtensor/nvfp4_tensor.py:94-97."""
    return reduce_amax(x).float() / (6.0 * 448.0)


def nvfp4_block_scales(x: torch.Tensor, block_size: int, wsf2: torch.Tensor | None = None,
                       keep_high_precision: bool = False):
    """E4M3 per-block scales.  Follows TQ/qtensor/nvfp4_tensor.py:63-92.

    ``bs = f32(block_amax) / (6.0 * wsf2)``; exact zeros become 1.0; cast to float8_e4m3fn with
    no clamp (values that round above 448 become NaN).
    """
    if wsf2 is None:
        wsf2 = nvfp4_global_scale(x)
    assert block_size != 0
    assert x.shape[-1] % block_size == 0
    bamax = reduce_block_amax(x, {-1: block_size}).float()
    bs = bamax / (6.0 * wsf2)
    bs[bs == 0] = 1.0
    if not keep_high_precision:
        bs = bs.to(torch.float8_e4m3fn)
    return bs, wsf2


def cast_fp4(v: torch.Tensor):
    """fp32 -> 4-bit E2M1 code (sign<<3 | ordinal), ties to even.

    Follows TQ/qtensor/nvfp4_tensor.py:120-140: sign is ``v < 0`` (so -0.0 and NaN are
    unsigned), ordinal = number of bounds strictly below |v| (NaN and inf give 7), plus one
    when |v| is exactly 0.75, 1.75 or 3.5.
    """
    sign = (v < 0).to(torch.uint8)
    mag = v.abs()
    ordinal = torch.searchsorted(E2M1_BOUNDS, mag, out_int32=True).to(torch.uint8)
    bump = torch.any(mag.unsqueeze(-1) == E2M1_BOUNDS[[1, 3, 5]], dim=-1).to(torch.uint8)
    return (sign << 3) + ordinal + bump


def nvfp4_quantize(x: torch.Tensor, block_size: int = 16, wsf: torch.Tensor | None = None,
                   wsf2: torch.Tensor | None = None):
    """NVFP4 quantize + pack.  Follows TQ/qtensor/nvfp4_tensor.py:143-232.

    Returns (packed uint8 [..., Kp/2], wsf float8_e4m3fn [..., Kp/bs], wsf2 f32 scalar) where Kp
    is K zero-padded to a multiple of the block.  ``v = f32(x) / (f32(wsf) * wsf2)`` is one fp32
    multiply then an IEEE divide; ``byte[i] = code[2i] | code[2i+1] << 4``.
    """
    x = reduce_block_padding(x, {-1: block_size})
    if wsf2 is None:
        wsf2 = nvfp4_global_scale(x)
    if wsf is None:
        wsf, _ = nvfp4_block_scales(x, block_size, wsf2)
    shape = x.shape
    blk = x.view(*shape[:-1], -1, block_size)
    v = (blk / (wsf.to(torch.float32) * wsf2).unsqueeze(-1)).view(shape)
    codes = cast_fp4(v)
    packed = (codes[..., 1::2] << 4) | codes[..., 0::2]
    return packed, wsf, wsf2


def nvfp4_dequantize(packed: torch.Tensor, wsf: torch.Tensor, wsf2: torch.Tensor,
                     block_size: int, shape, dtype: torch.dtype):
    """Unpack + LUT + rescale.  Follows TQ/qtensor/nvfp4_tensor.py:234-297 (non-fast branch).

    ``y = dtype( LUT[code] * (f32(wsf) * wsf2) )`` with LUT[8] = +0; result reshaped to
    ``shape`` (the reference reshapes, so ``shape`` must hold the padded element count).
    """
    out_shape = list(packed.shape)
    out_shape[-1] *= 2
    codes = torch.empty(out_shape, dtype=torch.long)
    codes[..., 1::2] = (packed >> 4).long()
    codes[..., 0::2] = (packed & 0x0F).long()
    vals = E2M1_LUT[codes.reshape(-1)].reshape(out_shape)
    scale = (wsf.to(torch.float32) if wsf.dtype == torch.float8_e4m3fn else wsf) * wsf2
    vals = vals.view(*out_shape[:-1], -1, block_size) * scale.unsqueeze(-1)
    return vals.reshape(shape).to(dtype)


# ----------------------------------------------------------------------------- INT4 (compress)


def int4_quantize(x: torch.Tensor, block_size: int):
    """INT4 block quantize + pack, CPU branch.  Follows TQ/qtensor/int4_tensor.py:40-88.

    Flat blocks over the whole tensor (zero padded); ``scales = 7 / amax`` in the input dtype;
    product in the input dtype; RNE round; clamp [-8, 7]; +8; ``byte = q[2i] << 4 | q[2i+1]``.
    Returns (packed uint8 [..., last/2], scales [nblocks, 1]) -- the *inverse* step size.
    """
    assert x.shape[-1] % 2 == 0
    flat = reduce_block_padding(x.reshape(-1), {-1: block_size})
    blk = flat.view(-1, block_size)
    scales = 7 / reduce_amax(blk, -1)
    scales = scales.view(blk.shape[0], -1)
    q = (blk * scales).flatten().round().clamp(-8, 7) + 8
    q = q.to(torch.uint8)
    packed = q[::2] << 4 | q[1::2]
    return packed.reshape(*x.shape[:-1], -1), scales


def int4_dequantize(packed: torch.Tensor, scales: torch.Tensor, block_size: int, shape,
                    dtype: torch.dtype):
    """Follows TQ/qtensor/int4_tensor.py:90-130 (CPU branch): ``(nibble - 8) / scale``."""
    hi = (packed >> 4).to(torch.long) - 8
    lo = (packed & 0x0F).to(torch.long) - 8
    hi = hi.view(-1, block_size // 2) / scales.view(-1, 1)
    lo = lo.view(-1, block_size // 2) / scales.view(-1, 1)
    both = torch.stack([hi.flatten(), lo.flatten()], dim=-1)
    return both.view(-1)[: math.prod(shape)].reshape(shape).to(dtype)


# ----------------------------------------------------------------------------- FP8 / INT8


def _expand_block_scales(scales: torch.Tensor, block_sizes: dict):
    for dim, blk in block_sizes.items():
        scales = scales.repeat_interleave(blk, dim=dim)
    return scales


def fp8_quantize(x: torch.Tensor, scales: torch.Tensor | None = None, axis=None,
                 block_sizes: dict | None = None):
    """FP8 real quantize.  Follows TQ/qtensor/fp8_tensor.py:41-113.

    ``scales = amax / 448.0`` stays in the amax dtype; the division ``x / scales`` follows
    torch type promotion (bf16 / bf16 -> bf16); cast with float8_e4m3fn RNE.
    """
    orig_shape = x.shape
    if block_sizes:
        x = reduce_block_padding(x, block_sizes)
    if scales is None:
        if block_sizes:
            amax = reduce_block_amax(x, block_sizes)
        else:
            amax = reduce_amax(x, axis=quant_axis_to_reduce_dims(x, axis))
        scales = amax / 448.0
    wide = scales.clone()
    if block_sizes:
        expect = list(x.shape)
        for dim, blk in block_sizes.items():
            d = dim if dim >= 0 else x.dim() + dim
            expect[d] = x.shape[d] // blk
        if scales.shape != tuple(expect) and scales.numel() == math.prod(expect):
            scales = scales.reshape(expect)
            wide = wide.reshape(expect)
        assert scales.shape == tuple(expect)
        wide = _expand_block_scales(wide, block_sizes)
    q = (x / wide).to(torch.float8_e4m3fn)
    return q[tuple(slice(0, d) for d in orig_shape)], scales


def fp8_dequantize(q: torch.Tensor, scales: torch.Tensor, shape, dtype: torch.dtype,
                   block_sizes: dict | None = None):
    """Follows TQ/qtensor/fp8_tensor.py:115-151: ``dtype(q) * dtype(scale)``."""
    if block_sizes:
        q = reduce_block_padding(q, block_sizes)
        scales = _expand_block_scales(scales, block_sizes)
    return (q.to(dtype) * scales.to(dtype))[tuple(slice(0, d) for d in shape)]


def int8_quantize(x: torch.Tensor, scales: torch.Tensor | None = None, axis=None,
                  block_sizes: dict | None = None):
    """INT8 real quantize.  Follows TQ/qtensor/int8_tensor.py:36-95."""
    if scales is None:
        if block_sizes:
            x = reduce_block_padding(x, block_sizes)
            amax = reduce_block_amax(x, block_sizes)
        else:
            amax = reduce_amax(x, axis=quant_axis_to_reduce_dims(x, axis))
        scales = amax / 127.0
    wide = scales.clone()
    if block_sizes:
        wide = _expand_block_scales(wide, block_sizes)
    return (x / wide).round().clamp(-128, 127).to(torch.int8), scales


def int8_dequantize(q: torch.Tensor, scales: torch.Tensor, shape, dtype: torch.dtype,
                    block_sizes: dict | None = None):
    """Follows TQ/qtensor/int8_tensor.py:97-130."""
    if block_sizes:
        scales = _expand_block_scales(scales, block_sizes)
    return (q.view(torch.int8).to(dtype) * scales.to(dtype))[tuple(slice(0, d) for d in shape)]
