"""Block scales on any set of dims, presented to the kernels as one row per block.

The reference pads every blocked dim to a multiple of its block, keeps one scale per block
(``scales.shape[d] = padded.shape[d] // block`` on blocked dims, the full extent elsewhere) and
expands the scales with ``repeat_interleave`` (qtensor/fp8_tensor.py:62-112, int8_tensor.py:
57-104).  Here the padded tensor is split ``[.., d/b, b, ..]``, the block dims are moved to the
back and the result is viewed as ``[number of blocks, elements per block]``: row r then has the
scale ``scales.flatten()[r]``.  For blocks along the last dim without padding this is a plain
view; other layouts cost one transposing copy each way.
"""

import math

import torch.nn.functional as F

__all__ = ["BlockRows"]


class BlockRows:
    def __init__(self, shape, block_sizes: dict):
        nd = len(shape)
        self.shape = tuple(shape)
        blocks = {}
        for d, b in block_sizes.items():
            if isinstance(d, int) and b:
                blocks[d % nd] = int(b)
        self.padded = tuple(-(-s // blocks[d]) * blocks[d] if d in blocks else s
                            for d, s in enumerate(shape))
        split, keep, inner = [], [], []
        for d, s in enumerate(self.padded):
            if d in blocks:
                keep.append(len(split))
                split.append(s // blocks[d])
                inner.append(len(split))
                split.append(blocks[d])
            else:
                keep.append(len(split))
                split.append(s)
        self.split = tuple(split)
        self.perm = keep + inner
        self.scale_shape = tuple(split[i] for i in keep)
        self.rows = math.prod(self.scale_shape)
        self.block = math.prod(split[i] for i in inner)

    def pad(self, x):
        spec = []
        for d in reversed(range(len(self.shape))):
            spec += [0, self.padded[d] - x.shape[d]]
        return F.pad(x, spec) if any(spec) else x

    def to_rows(self, x):
        """[rows, block] contiguous (zero padded)."""
        x = self.pad(x).reshape(self.split).permute(self.perm)
        return x.contiguous().view(self.rows, self.block)

    def from_rows(self, rows, crop=True):
        """Inverse of ``to_rows``, cropped to the original shape unless ``crop`` is False."""
        permuted = [self.split[i] for i in self.perm]
        inverse = [0] * len(self.perm)
        for i, d in enumerate(self.perm):
            inverse[d] = i
        y = rows.view(permuted).permute(inverse).reshape(self.padded)
        if not crop:
            return y.contiguous()
        return y[tuple(slice(0, s) for s in self.shape)].contiguous()
