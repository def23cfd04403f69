"""Oracle: export-time weight packing (test infrastructure, CPU torch)."""

import torch

from . import qtensor


def get_scaling_factor_from_weight(weight: torch.Tensor, group_size: int):
    """Follows export/quant_utils.py:68-91: ``f32(max|w| per group) / 7`` (``/127`` per row when
    group_size == 0); exact zeros become 1.0."""
    n, k = weight.shape
    if group_size != 0:
        if k % group_size != 0:
            raise NotImplementedError("Weight shape is not divisible for block size")
        weight = weight.reshape(n, k // group_size, group_size)
        bound = 7.0
    else:
        bound = 127.0
    sf = weight.abs().max(dim=-1)[0].float() / bound
    sf[sf == 0] = 1.0
    return sf


def pack_int4_in_uint8(weight: torch.Tensor, wsf: torch.Tensor):
    """INT4-AWQ export pack.  Follows export/quant_utils.py:697-738.

    Pinned by tests/golden/export_vectors.json (outputs of the reference's own function).
    ``q = int8(clamp(round_rne(w / wsf[:, k // bs]), -8, 7))`` (bf16 / fp32 tensor -> fp32
    division); two's-complement nibbles of *adjacent output rows* share a byte:
    ``byte[j, k] = (q[2j, k] & 0xF) | (q[2j+1, k] << 4)``; result uint8 [N/2, K]
    (3-D: [E, N/2, K]).
    """
    out_dim, in_dim = weight.shape[-2], weight.shape[-1]
    assert out_dim % 2 == 0
    bs = in_dim // wsf.shape[-1]
    q = (weight / wsf[..., :, torch.arange(in_dim) // bs]).round().clamp(-8, 7).to(torch.int8)
    if q.dim() == 3:
        t = q.permute(0, 2, 1).reshape(-1, in_dim, out_dim // 2, 2)
        byte = (t[..., 0] & 0x0F) | ((t[..., 1] & 0x0F) << 4)
        return byte.permute(0, 2, 1).contiguous().view(torch.uint8)
    t = q.T.reshape(in_dim, out_dim // 2, 2)
    byte = (t[..., 0] & 0x0F) | ((t[..., 1] & 0x0F) << 4)
    return byte.T.contiguous().view(torch.uint8)


def unpack_int4_rows(packed: torch.Tensor):
    """Inverse of the byte layout above -> int8 [N, K] (used for the round-trip invariant)."""
    lo = (packed & 0x0F).to(torch.int8)
    hi = (packed >> 4).to(torch.int8)
    lo = torch.where(lo > 7, lo - 16, lo)
    hi = torch.where(hi > 7, hi - 16, hi)
    n2, k = packed.shape[-2], packed.shape[-1]
    out = torch.empty(*packed.shape[:-2], n2 * 2, k, dtype=torch.int8)
    out[..., 0::2, :] = lo
    out[..., 1::2, :] = hi
    return out


def fp8_export_cast(weight: torch.Tensor, wsf: torch.Tensor):
    """FP8 per-tensor export cast.  Follows export/quant_utils.py:759-771 with the scale of
    export/unified_export_hf.py:260-269 (``f32(amax) / 448``, 0-dim or 1-element fp32).

    Pinned by tests/golden/export_vectors.json (outputs of the reference's own
    ``to_quantized_weight``).  ``weight / wsf`` follows torch type promotion: a bf16
    tensor divided by a 0-dim fp32 tensor gives a **bf16** tensor (fp32 quotient rounded to
    bf16), which is then rounded a second time to E4M3; with a dim>=1 fp32 scale the quotient
    stays fp32 and is rounded once.
    """
    return (weight / wsf).to(torch.float8_e4m3fn)


def int8_export_cast(weight: torch.Tensor, wsf: torch.Tensor):
    """Follows export/quant_utils.py:773-774: per-row ``round(w / s[:, None])`` clamp int8."""
    return (weight / wsf[:, None]).round().clamp(-128, 127).to(torch.int8)


def nvfp4_export(weight: torch.Tensor, amax: torch.Tensor, block_size: int = 16):
    """NVFP4 export of one linear weight: scales from export/quant_utils.py:251-293 and
    TQ/qtensor/nvfp4_tensor.py:55-92, codes from export/quant_utils.py:822-834.

    ``amax`` is the calibrated per-tensor weight amax (bf16 scalar).  Returns
    (packed uint8 [N, K/2], weight_scale e4m3 [N, K/bs], weight_scale_2 f32 scalar).
    """
    wsf2 = amax.float() / (6.0 * 448.0)
    wsf, _ = qtensor.nvfp4_block_scales(weight, block_size, wsf2)
    packed, _, _ = qtensor.nvfp4_quantize(weight, block_size, wsf, wsf2)
    return packed, wsf, wsf2
