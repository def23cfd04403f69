"""The module name under which the reference keeps its NVFP4 device kernels
(modelopt/torch/quantization/triton/__init__.py, triton/fp4_kernel.py:141-208,307-350), with the
same three names.  Nothing here uses Triton: both functions call the hand-written HIP kernels
through the C ABI; the tiling and launch arguments of the reference's signatures are accepted and
ignored.
"""

import torch

from .... import _hip
from .. import kernels

__all__ = ["IS_AVAILABLE", "fp4_fake_quant_block", "fp4_dequantize"]

IS_AVAILABLE = _hip.is_available()


def fp4_fake_quant_block(x, global_amax, block_size=16, tile_rows=16, tile_cols=64, num_warps=None,
                         num_stages=None):
    """NVFP4 fake quantisation of ``x`` in blocks of ``block_size`` along the last dim under the
    global abs-max ``global_amax``: the threshold-ladder formula of the reference's kernel
    (triton/fp4_kernel.py:86-134) with IEEE division."""
    return kernels.fake_quant_nvfp4(x, global_amax, block_size, 0)


def fp4_dequantize(packed_tensor, scale_tensor, global_scale, block_size=16, tile_size=128,
                   dtype=None):
    """``dtype(LUT[code] * (f32(scale) * global_scale))``: packed uint8 ``[..., N / 2]`` and E4M3
    block scales ``[..., N / block_size]`` to ``[..., N]``."""
    dtype = torch.get_default_dtype() if dtype is None else dtype
    scale = scale_tensor if scale_tensor.dtype == torch.float8_e4m3fn else scale_tensor.view(
        torch.float8_e4m3fn)
    return _hip.nvfp4_dequantize(packed_tensor.contiguous(), scale.contiguous(),
                                 global_scale.detach().reshape(()).to(torch.float32), block_size, dtype)
