"""NVFP4 real quantisation (reference: qtensor/nvfp4_tensor.py:31-297) on the HIP kernels.

Layout: ``packed`` uint8 [..., K/2] with byte i = code[2i] | code[2i+1] << 4 (code = sign << 3 |
E2M1 ordinal); per-block scales ``float8_e4m3fn`` [..., K/block]; one fp32 global scale
``amax / (6 * 448)``.  The last dim is zero padded to a multiple of the block.
"""

import torch

from .... import _hip
from .. import modes
from ..overflow import nvfp4_quantize_flags
from ..utils import all_positive, reduce_amax, reduce_block_amax, reduce_block_padding, true_divide
from .base_qtensor import BaseQuantizedTensor

__all__ = ["NVFP4QTensor"]

e2m1_bounds = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5])
e2m1_values = torch.tensor([0, 0.5, 1, 1.5, 2, 3, 4, 6, 0, -0.5, -1, -1.5, -2, -3, -4, -6])


def _f32_scalar(t: torch.Tensor):
    return t.detach().reshape(()).to(torch.float32)


def _per_leading_index(scale2, input):
    """The global scales of a stack of matrices -- one per index of the first dim, shaped to
    broadcast (``view(-1, 1, 1)`` for stacked expert weights, export/quant_utils.py:822-829) -- as
    a flat tensor, or None for the usual single scale."""
    if scale2 is None or scale2.numel() == 1:
        return None
    assert input.dim() >= 2 and scale2.numel() == input.shape[0] and (
        scale2.dim() <= 1 or tuple(scale2.shape[1:]) == (1,) * (scale2.dim() - 1)), (
        f"global scale of shape {tuple(scale2.shape)} does not broadcast over the first dim of "
        f"{tuple(input.shape)}")
    return scale2.reshape(-1)


class NVFP4QTensor(BaseQuantizedTensor):
    """Packed NVFP4 tensor."""

    e2m1_values_on_device = {}
    e2m1_bounds_on_device = {}

    @classmethod
    def get_e2m1_values(cls, device):
        """The 16 values a code stands for, on ``device`` (reference: nvfp4_tensor.py:41-46)."""
        if device not in cls.e2m1_values_on_device:
            cls.e2m1_values_on_device[device] = e2m1_values.to(device)
        return cls.e2m1_values_on_device[device]

    @classmethod
    def get_e2m1_bounds(cls, device):
        """The 7 midpoints between adjacent magnitudes, on ``device`` (reference: :48-53)."""
        if device not in cls.e2m1_bounds_on_device:
            cls.e2m1_bounds_on_device[device] = e2m1_bounds.to(device)
        return cls.e2m1_bounds_on_device[device]

    @classmethod
    def _cast_fp4(cls, weight: torch.Tensor):
        """``sign << 3 | ordinal`` per element, uint8, ties to the even code (reference:
        nvfp4_tensor.py:120-140; unlike the reference, ``weight`` is not overwritten with its
        absolute value)."""
        return _hip.cast_fp4(weight.contiguous())

    @classmethod
    def get_weights_scaling_factor_2_from_quantizer(cls, weight_quantizer):
        assert hasattr(weight_quantizer, "_amax"), "Weight quantizer does not have attribute amax"
        return true_divide(weight_quantizer._amax.float(), 6.0 * 448.0)

    @classmethod
    def get_weights_scaling_factor_2(cls, input: torch.Tensor):
        return true_divide(reduce_amax(input).float(), 6.0 * 448.0)

    @classmethod
    def get_weights_scaling_factor(cls, input, block_size, weights_scaling_factor_2=None,
                                   keep_high_precision=False):
        """Per-block scale (E4M3 unless ``keep_high_precision``) and the global scale."""
        if weights_scaling_factor_2 is None:
            weights_scaling_factor_2 = cls.get_weights_scaling_factor_2(input)
        assert block_size != 0, "Block size is zero. Cannot return per_block amax for given input."
        assert input.shape[-1] % block_size == 0, (
            "Weight shape is not divisible for block size for block quantization.")
        wsf2 = weights_scaling_factor_2.to(input.device)
        each = _per_leading_index(wsf2, input)
        if each is not None:
            return torch.stack([cls.get_weights_scaling_factor(input[i], block_size, each[i],
                                                               keep_high_precision)[0]
                                for i in range(input.shape[0])]), weights_scaling_factor_2
        if keep_high_precision:
            bamax = reduce_block_amax(input, {-1: block_size}).float()
            scale = bamax / (6.0 * wsf2)
            scale[scale == 0] = 1.0
            return scale, weights_scaling_factor_2
        _, wsf, _ = _hip.nvfp4_quantize(input.contiguous(), _f32_scalar(wsf2), block_size,
                                        amax_is_wsf2=True, flags=nvfp4_quantize_flags())
        return wsf, weights_scaling_factor_2

    @classmethod
    def get_activation_scaling_factor(cls, quantizer):
        if not quantizer.is_enabled:
            return None
        amax = quantizer.export_amax()
        if amax is None:
            return None
        sf = true_divide(amax.float(), quantizer.maxbound * 448.0)
        # one host synchronisation per layer if checked here: an export defers it to its end
        assert all_positive(sf, lambda: f" activation scaling factor {sf} not positive."), (
            f" activation scaling factor {sf} not positive.")
        return sf

    @classmethod
    def quantize(cls, input, block_size, weights_scaling_factor=None, weights_scaling_factor_2=None,
                 keep_high_precision=False, try_tensorrt=False):
        """Returns (NVFP4QTensor, per-block E4M3 scales, fp32 global scale) in one kernel pass
        (plus one abs-max pass when the global scale is not given)."""
        if keep_high_precision:
            # the reference returns the scaled weight before the FP4 cast, fp32 and still padded
            # (qtensor/nvfp4_tensor.py:208-222); a few tensor ops, no caller on the hot path
            xp = reduce_block_padding(input, {-1: block_size})
            if weights_scaling_factor_2 is None:
                weights_scaling_factor_2 = cls.get_weights_scaling_factor_2(xp)
            if weights_scaling_factor is None:
                weights_scaling_factor, _ = cls.get_weights_scaling_factor(
                    xp, block_size, weights_scaling_factor_2)
            scale = weights_scaling_factor.to(xp.device).to(torch.float32) * \
                weights_scaling_factor_2.to(xp.device)
            blocks = xp.reshape(*xp.shape[:-1], -1, block_size)
            return torch.div(blocks, scale.unsqueeze(-1)).reshape(xp.shape)
        shape, dtype = input.shape, input.dtype
        each = _per_leading_index(weights_scaling_factor_2, input)
        if each is not None:
            parts = [cls.quantize(input[i], block_size,
                                  None if weights_scaling_factor is None else weights_scaling_factor[i],
                                  each[i]) for i in range(shape[0])]
            scales = weights_scaling_factor if weights_scaling_factor is not None else \
                torch.stack([p[1] for p in parts])
            return (cls(shape, dtype, torch.stack([p[0]._quantized_data for p in parts])), scales,
                    weights_scaling_factor_2)
        x = input.contiguous()
        if (weights_scaling_factor_2 is None and weights_scaling_factor is None and block_size == 16
                and modes.one_launch_dynamic_quant()):
            # abs-max, scales and codes in one launch that reads the tensor once (tensors that fit
            # the chip's registers; larger ones take the two launches below); opt-in
            fused = _hip.nvfp4_quantize_fused(x, flags=nvfp4_quantize_flags())
            if fused is not None:
                packed, wsf, wsf2, _ = fused
                return cls(shape, dtype, packed), wsf, wsf2
        if weights_scaling_factor_2 is None:
            acc = torch.zeros(1, dtype=torch.float32, device=x.device)
            _hip.absmax_into(x, acc, 1, 1, x.numel(), reread=True)   # the quantize pass reads x next
            scalar, is_wsf2 = acc.reshape(()), False
        else:
            scalar, is_wsf2 = _f32_scalar(weights_scaling_factor_2.to(x.device)), True
        wsf_in = None
        if weights_scaling_factor is not None:
            wsf_in = weights_scaling_factor.to(x.device).contiguous()
            assert wsf_in.dtype == torch.float8_e4m3fn, "block scales must be float8_e4m3fn"
        packed, wsf, wsf2 = _hip.nvfp4_quantize(x, scalar, block_size, is_wsf2, wsf_in,
                                                flags=nvfp4_quantize_flags())
        if weights_scaling_factor is not None:
            wsf = weights_scaling_factor
        if weights_scaling_factor_2 is not None:
            wsf2 = weights_scaling_factor_2
        return cls(shape, dtype, packed), wsf, wsf2

    def dequantize(self, dtype: torch.dtype = None, fast=False, **kwarg):
        """``dtype(LUT[code] * (f32(scale) * double_scale))`` reshaped to the original shape."""
        if dtype is None:
            dtype = self.metadata["dtype"]
        scale, wsf2 = kwarg["scale"], kwarg["double_scale"]
        block = kwarg["block_sizes"][-1]
        if scale.dtype != torch.float8_e4m3fn:
            raise NotImplementedError("NVFP4 dequantize needs float8_e4m3fn block scales")
        packed = self._quantized_data
        each = _per_leading_index(wsf2, packed)
        if each is not None:
            scale = scale.to(packed.device)
            return torch.stack([_hip.nvfp4_dequantize(
                packed[i].contiguous(), scale[i].contiguous(), _f32_scalar(each[i].to(packed.device)),
                block, dtype) for i in range(packed.shape[0])]).reshape(self.metadata["shape"])
        y = _hip.nvfp4_dequantize(packed.contiguous(), scale.to(packed.device).contiguous(),
                                  _f32_scalar(wsf2.to(packed.device)), block, dtype)
        return y.reshape(self.metadata["shape"])
