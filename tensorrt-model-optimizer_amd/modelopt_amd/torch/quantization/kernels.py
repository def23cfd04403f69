"""Shape logic between torch tensors and the HIP C ABI (``modelopt_amd._hip``).

Everything here runs on the GPU through ``libmodelopt_hip.so``; CPU tensors are rejected.  The
functions take and return torch tensors and never synchronise with the host.
"""

import math

import torch

from ... import _hip

__all__ = [
    "amax_layout", "kept_dims_first", "dense_flat_view", "absmax_accumulate", "reduce_amax_gpu", "fake_quant_int", "fake_quant_fp8",
    "fake_quant_nvfp4", "fake_quant_block_fp", "mul_last_dim",
]


def _prod(xs):
    return int(math.prod(xs))


def amax_layout(shape, keep_dims):
    """View a tensor of ``shape`` as [outer, axis, inner] such that the dims in ``keep_dims``
    (a contiguous run of dims, or none) form ``axis``.  Returns (outer, axis, inner) or None
    when the kept dims are not one contiguous run."""
    nd = len(shape)
    keep = sorted(d % nd for d in keep_dims if shape[d % nd] != 1)
    if not keep:
        return 1, 1, _prod(shape)
    if keep != list(range(keep[0], keep[-1] + 1)):
        # unit dims between kept dims do not break contiguity
        for d in range(keep[0], keep[-1] + 1):
            if d not in keep and shape[d] != 1:
                return None
    lo, hi = keep[0], keep[-1]
    return _prod(shape[:lo]), _prod(shape[lo:hi + 1]), _prod(shape[hi + 1:])


def kept_dims_first(x, keep_dims):
    """For kept dims that are not one contiguous run (2-D blocks: dims 0 and 2 of
    ``[N/b0, b0, K/b1, b1]``): a contiguous copy with the kept dims moved to the front, viewed by
    the kernels as [1, prod(kept), prod(rest)], and the permutation that was applied.  Costs one
    transposing copy each way; the common layouts never take this route."""
    nd = x.dim()
    keep = sorted({d % nd for d in keep_dims})
    perm = keep + [d for d in range(nd) if d not in keep]
    xp = x.permute(perm).contiguous()
    return xp, perm, (1, _prod(x.shape[d] for d in keep), _prod(xp.shape[len(keep):]))


def _undo_permutation(y, perm):
    inverse = [0] * len(perm)
    for i, d in enumerate(perm):
        inverse[d] = i
    return y.permute(inverse).contiguous()


def layout_from_amax_shape(x_shape, amax_shape):
    """[outer, axis, inner] for an amax whose shape broadcasts against ``x_shape`` (per-tensor,
    or equal to x on a contiguous run of dims and 1 elsewhere)."""
    n = _prod(amax_shape)
    if n == 1:
        return 1, 1, _prod(x_shape)
    a = list(amax_shape)
    if len(a) == 1 and len(x_shape) >= 1:
        # squeezed per-channel amax: the reference matches it to the dim of equal length
        if a[0] in list(x_shape):
            d = list(x_shape).index(a[0])
            return amax_layout(x_shape, [d])
        return None
    if len(a) != len(x_shape):
        return None
    keep = [d for d in range(len(a)) if a[d] != 1]
    if any(a[d] != x_shape[d] for d in keep):
        return None
    return amax_layout(x_shape, keep)


def dense_flat_view(x: torch.Tensor):
    """A 1-D view over the memory of ``x`` when ``x`` is a permutation of a contiguous block (a
    transposed K / V view, a channels-last tensor): every element appears exactly once, in memory
    order.  None when ``x`` has gaps or overlaps."""
    dims = sorted((d for d in range(x.dim()) if x.shape[d] != 1), key=lambda d: -x.stride(d))
    expect = 1
    for d in reversed(dims):
        if x.stride(d) != expect:
            return None
        expect *= x.shape[d]
    return x.as_strided((x.numel(),), (1,))


def absmax_accumulate(x: torch.Tensor, acc: torch.Tensor, layout, reread: bool = False):
    """acc (fp32, ``axis`` elements) = max(acc, abs-max of x over the reduced dims).  ``reread``:
    the caller reads ``x`` again right away (see ``_hip.absmax_into``)."""
    outer, axis, inner = layout
    if not x.is_contiguous():
        # a per-tensor maximum does not care about element order: a permuted dense tensor (the
        # [B, H, S, D] view of K / V) is reduced where it lies instead of through a copy
        flat = dense_flat_view(x) if axis == 1 else None
        x = flat if flat is not None else x.contiguous()
    return _hip.absmax_into(x, acc, outer, axis, inner, reread=reread)


def reduce_amax_gpu(x: torch.Tensor, reduce_dims, keepdims=True, reread: bool = False):
    """``reduce_amax`` on the device: abs-max over ``reduce_dims`` (None = all) in x.dtype."""
    nd = x.dim()
    if reduce_dims is None:
        keep, out_shape = [], ()
    else:
        red = {d % nd for d in ([reduce_dims] if isinstance(reduce_dims, int) else reduce_dims)}
        keep = [d for d in range(nd) if d not in red]
        out_shape = tuple(1 if d in red else x.shape[d] for d in range(nd)) if keepdims else tuple(
            x.shape[d] for d in keep)
    layout = amax_layout(tuple(x.shape), keep)
    src = x
    if layout is None and x.is_cuda and x.is_contiguous():
        # one abs-max per two-dimensional block of a matrix: a workgroup per block, no transposed copy
        blocks = blocks2d_of(tuple(x.shape), keep)
        if blocks is not None and _hip.blocks2d_covered(x, *blocks):
            rows, cols, block_rows, block_cols = blocks
            acc = torch.zeros((rows // block_rows) * (cols // block_cols), dtype=torch.float32, device=x.device)
            _hip.absmax_blocks2d_into(x, acc, rows, cols, block_rows, block_cols)
            return acc.to(x.dtype).reshape(out_shape)
    if layout is None:
        src, _, layout = kept_dims_first(x, keep)
    acc = torch.zeros(layout[1], dtype=torch.float32, device=x.device)
    absmax_accumulate(src, acc, layout, reread=reread)
    return acc.to(x.dtype).reshape(out_shape)


def _qdq_layout(x, amax):
    return layout_from_amax_shape(tuple(x.shape), tuple(amax.shape))


def blocks2d_of(shape, kept) -> tuple | None:
    """``(rows, cols, block_rows, block_cols)`` when a contiguous tensor of ``shape`` whose scale
    dims are ``kept`` (a sorted list) is a matrix cut into two-dimensional blocks: the reshape
    ``[..., R, block_rows, C, block_cols]`` of ``[..., R * block_rows, C * block_cols]`` with a
    scale for every index of all dims but the two block dims (what a quantizer with block sizes
    on the last two dims sets up).  None otherwise."""
    nd = len(shape)
    if nd < 4 or list(kept) != [d for d in range(nd) if d not in (nd - 3, nd - 1)]:
        return None
    block_rows, block_cols = shape[nd - 3], shape[nd - 1]
    rows = math.prod(shape[:nd - 3]) * block_rows
    return rows, shape[nd - 2] * block_cols, block_rows, block_cols


def _qdq(x, amax, run, run2d=None):
    """``run(x2, amax_flat, outer, axis, inner)`` on ``x`` as it is when the amax spans one run
    of dims; ``run2d(x, amax_flat, rows, cols, block_rows, block_cols)`` when the amax is per
    two-dimensional block of a matrix; else ``run`` on a copy with the amax dims moved to the
    front (and moved back afterwards)."""
    x = x if x.is_contiguous() else x.contiguous()
    layout = _qdq_layout(x, amax)
    if layout is not None:
        return run(x, amax.reshape(-1).contiguous(), *layout)
    if amax.dim() != x.dim() or any(a not in (1, s) for a, s in zip(amax.shape, x.shape)):
        raise NotImplementedError(
            f"amax of shape {tuple(amax.shape)} does not broadcast against input {tuple(x.shape)}")
    if run2d is not None and x.is_cuda:
        blocks = blocks2d_of(tuple(x.shape), [d for d in range(x.dim()) if amax.shape[d] != 1])
        if blocks is not None and _hip.blocks2d_covered(x, *blocks):
            return run2d(x, amax.reshape(-1).contiguous(), *blocks)
    keep = [d for d in range(x.dim()) if amax.shape[d] != 1]
    xp, perm, layout = kept_dims_first(x, keep)
    y = run(xp, amax.reshape(-1).contiguous(), *layout)
    return _undo_permutation(y.view(xp.shape), perm)


with_scale_layout = _qdq   # the storage casts place their scales the same way


def fake_quant_int(x, amax, num_bits=8, unsigned=False, narrow_range=True):
    return _qdq(x, amax, lambda x2, a, outer, axis, inner: _hip.int_qdq(
        x2, a, outer, axis, inner, num_bits, unsigned, narrow_range),
        lambda x2, a, rows, cols, br, bc: _hip.int_qdq_blocks2d(
            x2, a, rows, cols, br, bc, num_bits, unsigned, narrow_range))


def fake_quant_fp8(x, amax=None, saturate=False):
    if amax is None:
        x = x if x.is_contiguous() else x.contiguous()
        return _hip.fp8_qdq(x, None, 1, 1, x.numel(), saturate)
    return _qdq(x, amax, lambda x2, a, outer, axis, inner: _hip.fp8_qdq(
        x2, a, outer, axis, inner, saturate),
        lambda x2, a, rows, cols, br, bc: _hip.fp8_qdq_blocks2d(x2, a, rows, cols, br, bc, saturate))


def fake_quant_nvfp4(x, global_amax, block_size=16, mode=0):
    x = x if x.is_contiguous() else x.contiguous()
    if global_amax.numel() != 1:
        global_amax = global_amax.amax()
    return _hip.nvfp4_qdq(x, global_amax.reshape(1), block_size, mode)


def fake_quant_block_fp(x, block_size, fmt, scale_fmt="E8M0", global_amax=None):
    """Block floating point fake quantisation along the last dim (``fused_amax_convert``):
    ``fmt`` / ``scale_fmt`` are format names (``"E4M3"``, ``"E2M1"``, ``"E8M0"`` ...)."""
    x = x if x.is_contiguous() else x.contiguous()
    if global_amax is not None:
        global_amax = global_amax.to(device=x.device, dtype=torch.float32).reshape(-1).contiguous()
    return _hip.block_fp_qdq(x, block_size, fmt, scale_fmt, global_amax)


def mul_last_dim(x, scale):
    """``x * scale`` for a scale that spans the last dim only."""
    x = x if x.is_contiguous() else x.contiguous()
    return _hip.mul_cols(x, scale.reshape(-1).contiguous())
