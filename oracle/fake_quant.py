"""Oracle: quantize-dequantize ("fake quant") functions (test infrastructure, CPU torch)."""

import torch
import torch.nn.functional as F

from .reduce import reduce_amax

E2M1_MAX = 6.0
E4M3_MAX = 448.0


def fp8_eager(x: torch.Tensor, amax: torch.Tensor | None = None):
    """FP8 E4M3 QDQ.  Follows TQ/tensor_quant.py:45-59.

    ``scale = 448.0 / f32(amax)`` is ``float / tensor``, which torch evaluates as
    ``reciprocal(amax) * 448.0`` (two roundings, not a true division); ``inv = 1 / scale`` is
    ``reciprocal(scale)``.  The cast is torch's ``float8_e4m3fn`` (RNE, subnormals kept, magnitudes
    that round above 448 become NaN on CPU).  ``amax`` may be any shape broadcastable to ``x``.
    """
    dt = x.dtype
    if amax is not None:
        scale = 448.0 / amax.to(torch.float32)
        inv = 1 / scale
        x = x.to(torch.float32) * scale
    x = x.to(torch.float8_e4m3fn)
    if amax is not None:
        x = x.to(torch.float32) * inv
    return x.to(dt)


def tensor_quant(x: torch.Tensor, amax: torch.Tensor, num_bits=8, unsigned=False, narrow_range=True):
    """Integer QDQ in fp32.  Follows TQ/tensor_quant.py:574-612.

    ``scale = bound / f32(amax)``; ``amax <= 2**-24`` quantises to exactly 0 (scale forced to 0
    for the multiply, to 1 for the divide); round is half-to-even; result cast back to x.dtype.
    """
    if unsigned and x.min() < 0.0:
        raise TypeError("Negative values encountered in unsigned quantization.")
    dt = x.dtype
    xf, af = x.float(), amax.float()
    lowest = af.min()
    if lowest < 0:
        raise ValueError("Negative values in amax")
    hi = torch.tensor(2.0 ** (num_bits - 1 + int(unsigned)) - 1.0)
    lo = 0 if unsigned else (-hi if narrow_range else -hi - 1)
    scale = hi / af
    eps = 1.0 / (1 << 24)
    dead = None
    if lowest <= eps:
        dead = af <= eps
        scale[dead] = 0
    q = torch.clamp((xf * scale).round_(), lo, hi)
    if dead is not None:
        scale[dead] = 1.0
    return (q / scale).to(dt)


def nvfp4_fake_quant(x: torch.Tensor, global_amax: torch.Tensor, block_size: int = 16):
    """NVFP4 dynamic-block QDQ with the threshold-ladder formula, all in fp32.

    Restates the arithmetic of TQ/triton/fp4_kernel.py:86-134 (launcher :141-208) with IEEE fp32
    division; the reference has no CPU implementation of this function (TQ/tensor_quant.py:173).
    gs = f32(amax)/(6*448); per block of ``block_size`` along the last dim (zero padded):
    sc = min(bmax/(6*gs_safe), 448); q = f32(e4m3(sc))*gs; q < 1e-5 -> 1; r = |x|/q; ladder;
    sign taken from ``x >= 0`` (so NaN and tiny negatives come out negative).
    """
    shape, dt = x.shape, x.dtype
    k = shape[-1]
    x2 = x.reshape(-1, k).float()
    pad = (-k) % block_size
    if pad:
        x2 = F.pad(x2, (0, pad))
    gs = global_amax.float().reshape(()) / (6.0 * 448.0)
    gs_safe = torch.where(gs > 0.0, gs, torch.tensor(1e-12))
    blk = x2.reshape(x2.shape[0], -1, block_size)
    mag = blk.abs()
    bmax = mag.amax(dim=-1, keepdim=True)
    sc = torch.minimum(bmax / (6.0 * gs_safe), torch.tensor(448.0))
    q = sc.to(torch.float8_e4m3fn).to(torch.float32) * gs
    q = torch.where(q >= 1e-5, q, torch.tensor(1.0))
    r = mag / q
    lvl = torch.full_like(r, 6.0)
    lvl = torch.where(r <= 5.0, torch.tensor(4.0), lvl)
    lvl = torch.where(r < 3.5, torch.tensor(3.0), lvl)
    lvl = torch.where(r <= 2.5, torch.tensor(2.0), lvl)
    lvl = torch.where(r < 1.75, torch.tensor(1.5), lvl)
    lvl = torch.where(r <= 1.25, torch.tensor(1.0), lvl)
    lvl = torch.where(r < 0.75, torch.tensor(0.5), lvl)
    lvl = torch.where(r <= 0.25, torch.tensor(0.0), lvl)
    y = lvl * q
    y = torch.where(blk >= 0, y, -y)
    y = y.reshape(x2.shape)[:, :k]
    return y.to(dt).reshape(shape)


def static_block_fake_quant(x: torch.Tensor, block_size: int, fn):
    """Last-axis static block quantisation wrapper.  Follows TQ/nn/modules/tensor_quantizer.py
    :712-800 (fast path :752-761): pad the last dim on the right with zeros to a multiple of the
    block, flatten to ``(-1, block)``, per-row amax ``[rows, 1]`` computed on the fly
    (:505-514), apply ``fn(x2d, amax)``, reshape back and drop the padding.
    """
    k = x.shape[-1]
    pad = (-k) % block_size
    xp = F.pad(x, (0, pad)) if pad else x
    x2 = xp.reshape(-1, block_size)
    amax = reduce_amax(x2, axis=[1], keepdims=True)
    y = fn(x2, amax).reshape(xp.shape)
    return y[..., :k] if pad else y
