"""Oracle: absolute-max reductions and the max calibrator (test infrastructure, CPU torch)."""

import torch
import torch.nn.functional as F


def quant_axis_to_reduce_dims(x: torch.Tensor, axis):
    """Dims to reduce so that ``axis`` survives.  Follows TQ/utils.py:137-152.

    ``None`` means per-tensor (reduce everything).  Negative and positive spellings of the kept
    axes are both honoured.
    """
    if axis is None:
        return None
    kept = list(axis) if isinstance(axis, (list, tuple)) else [axis]
    nd = x.dim()
    return [d for d in range(nd) if d not in kept and (d - nd) not in kept]


@torch.no_grad()
def reduce_amax(x: torch.Tensor, axis=None, keepdims=True, squeeze_scalar=True):
    """max(|max(x)|, |min(x)|) in the input dtype.  Follows TQ/utils.py:156-188.

    NaN propagates (torch.max/min/amax/amin/maximum all propagate NaN).
    """
    if axis is None:
        hi, lo = torch.max(x), torch.min(x)
        return torch.maximum(hi.abs(), lo.abs())
    dims = (axis,) if isinstance(axis, int) else tuple(axis)
    hi = torch.amax(x, dim=dims, keepdim=keepdims)
    lo = torch.amin(x, dim=dims, keepdim=keepdims)
    out = torch.maximum(hi.abs(), lo.abs())
    if squeeze_scalar and out.numel() == 1:
        out.squeeze_()
    return out


@torch.no_grad()
def reduce_block_padding(x: torch.Tensor, block_sizes: dict, pad_value: float = 0):
    """Right-pad each listed dim up to a multiple of its block.  Follows TQ/utils.py:101-134."""
    nd = x.dim()
    for dim, blk in block_sizes.items():
        d = dim if dim >= 0 else nd + dim
        rem = x.size(d) % blk
        if rem:
            spec = [0] * (2 * nd)
            spec[(nd - 1 - d) * 2 + 1] = blk - rem
            x = F.pad(x, spec, value=pad_value)
    return x


@torch.no_grad()
def reduce_block_amax(x: torch.Tensor, block_sizes: dict):
    """Blockwise amax, one listed dim at a time.  Follows TQ/utils.py:52-98."""
    out = x.clone()
    for dim, blk in block_sizes.items():
        d = dim if dim >= 0 else out.dim() + dim
        assert out.shape[d] % blk == 0, "dimension not divisible by block size"
        shape = list(out.shape)
        shape[d:d + 1] = [shape[d] // blk, blk]
        out = reduce_amax(out.reshape(shape), d + 1, keepdims=False, squeeze_scalar=False)
    return out


class MaxCalibrator:
    """Running abs-max over collected tensors.  Follows TQ/calib/max.py:26-94."""

    def __init__(self, num_bits=8, axis=None, unsigned=False):
        self._num_bits, self._axis, self._unsigned = num_bits, axis, unsigned
        self._calib_amax = None

    @torch.no_grad()
    def collect(self, x):
        local = reduce_amax(x, axis=quant_axis_to_reduce_dims(x, self._axis)).detach()
        assert torch.all(local >= 0), "detected negative values after abs"
        assert not torch.any(torch.isinf(local)), "detected inf values in amax"
        assert not torch.any(torch.isnan(local)), "detected nan values in amax"
        if self._calib_amax is None:
            self._calib_amax = local
        else:
            if local.shape != self._calib_amax.shape:
                raise RuntimeError("amax shape changed!")
            self._calib_amax = torch.max(self._calib_amax, local)

    def reset(self):
        self._calib_amax = None

    def compute_amax(self):
        return self._calib_amax
