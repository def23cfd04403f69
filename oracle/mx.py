"""Oracle: block floating point fake quantisation with a shared power-of-two (E8M0) or
minifloat scale per block -- the MX formats and the two-level NVFP4 variant (test infrastructure).

Restates ``fused_amax_convert`` of the reference, TQ/src/tensor_quant_mx.cu:35-57 (``quantize``),
:97-186 (scales), :243-297 (kernel), with the element tables and conversions of
TQ/src/tensor_quant_mx.h:38-178.  The reference exists only as a CUDA kernel built with
``--use_fast_math``; here every fp32 operation is IEEE (correctly rounded division, no flush to
zero), and the places where the reference computes in double do so here too.  Pinned by the
reference's golden tables (tests/golden/mx_vectors.json).
"""

import torch

# values a format can represent (non-negative half), TQ/src/tensor_quant_mx.h:41-77
_TABLES = {
    "E2M1": [0, 0.5, 1, 1.5, 2, 3, 4, 6],
    "E1M2": [0, 0.5, 1, 1.5, 2, 2.5, 3, 3.5],
    "E0M3": [0, 1, 2, 3, 4, 5, 6, 7],
    "E3M0": [0, 0.25, 0.5, 1, 2, 4, 8, 16],
    "E3M2": [0, 0.0625, 0.125, 0.1875, 0.25, 0.3125, 0.375, 0.4375, 0.5, 0.625, 0.75, 0.875, 1,
             1.25, 1.5, 1.75, 2, 2.5, 3, 3.5, 4, 5, 6, 7, 8, 10, 12, 14, 16, 20, 24, 28],
    "E2M3": [0, 0.125, 0.25, 0.375, 0.5, 0.625, 0.75, 0.875, 1, 1.125, 1.25, 1.375, 1.5, 1.625,
             1.75, 1.875, 2, 2.25, 2.5, 2.75, 3, 3.25, 3.5, 3.75, 4, 4.5, 5, 5.5, 6, 6.5, 7, 7.5],
}
FORMAT_MAX = {"E4M3": 448.0, "E5M2": 57344.0, "INT8": 127.0, "E2M1": 6.0, "E0M3": 7.0,
              "E3M0": 16.0, "E1M2": 3.5, "E3M2": 28.0, "E2M3": 7.5}
FORMATS = ["E4M3", "E5M2", "INT8", "E0M3", "E1M2", "E3M0", "E2M1", "E3M2", "E2M3", "E8M0"]


def convert_to_types(x: torch.Tensor, fmt: str) -> torch.Tensor:
    """Nearest representable value of ``fmt`` for every element of fp32 ``x`` (as fp32).
    Follows ``convert_to_types``, TQ/src/tensor_quant_mx.h:156-178."""
    x = x.to(torch.float32)
    if fmt == "E4M3":    # __nv_fp8_e4m3(float): round to nearest even, saturate to +-448, NaN stays
        return x.clamp(-448.0, 448.0).to(torch.float8_e4m3fn).to(torch.float32)
    if fmt == "E5M2":    # __nv_fp8_e5m2(float): the same with +-57344
        return x.clamp(-57344.0, 57344.0).to(torch.float8_e5m2).to(torch.float32)
    if fmt == "INT8":    # rint, clamp to +-127 (:85-95)
        return torch.round(x).clamp(-127, 127)
    values = torch.tensor(_TABLES[fmt], dtype=torch.float32)
    bounds = (values[:-1] + values[1:]) / 2          # the table_bounds of the header: midpoints
    a = x.abs()
    idx = torch.bucketize(a, bounds, right=False)    # number of bounds < a
    tie = (idx < len(bounds)) & (a == bounds[idx.clamp(max=len(bounds) - 1)])
    if fmt == "E3M0":    # ties away from zero (:98-107)
        idx = idx + tie.long()
    else:                # ties to the value whose table index is even (:110-128)
        idx = idx + (tie & (idx % 2 == 1)).long()
    idx = torch.where(torch.isfinite(a), idx, torch.full_like(idx, len(values) - 1))  # inf, NaN -> max
    out = values[idx.clamp(max=len(values) - 1)]
    return torch.where(x < 0, -out, out)


def _scale_e8m0(amax: torch.Tensor, fmt: str):
    """(scale, unscale) = (2^-e, 2^e), e = clamp(ceil(log2(amax / fmax)), -127, 127) read off the
    bits of the fp32 quotient.  Follows ``compute_scale_e8m0_NV``, :97-129."""
    ratio = amax / torch.tensor(FORMAT_MAX[fmt], dtype=torch.float32)
    bits = ratio.view(torch.int32)
    efield = (bits >> 23) & 0xFF
    mant = bits & 0x7FFFFF
    bump = (mant > 0) & (efield != 0xFE) & ~((efield == 0) & (mant <= 0x400000))
    e = torch.where(bump, efield - 126, efield - 127)
    return torch.ldexp(torch.ones_like(ratio), -e), torch.ldexp(torch.ones_like(ratio), e)


def _scale_general(amax: torch.Tensor, fmt: str, scale_fmt: str):
    """Follows ``compute_scale``, :140-148: in double, ``inv = fmt_scale(1 / (fmax / amax))``,
    ``scale = 1 / inv``; both returned as fp32."""
    scale = torch.tensor(FORMAT_MAX[fmt], dtype=torch.float32).double() / amax.double()
    inv = convert_to_types((1.0 / scale).float(), scale_fmt).double()
    return (1.0 / inv).float(), inv.float()


def _scale_with_global(global_amax: torch.Tensor, amax: torch.Tensor, fmt: str, scale_fmt: str):
    """Follows ``compute_scale_with_global``, :151-186."""
    fmax = torch.tensor(FORMAT_MAX[fmt], dtype=torch.float32)
    smax = torch.tensor(FORMAT_MAX[scale_fmt], dtype=torch.float32)
    local_unscale = amax / fmax                                           # fp32
    two_level = smax.double() * (fmax / global_amax).double()             # fp32 quotient, then double
    q = convert_to_types((local_unscale.double() * two_level).float(), scale_fmt).double() / two_level
    return (1.0 / q).float(), q.float()


def block_fp_fake_quant(x: torch.Tensor, block_size: int, fmt: str, scale_fmt: str = "E8M0",
                        global_amax: torch.Tensor | None = None):
    """``fused_amax_convert(x, block_size, fmt, scale_fmt, global_amax)``: blocks of
    ``block_size`` along the last dim (zero padded), one scale per block, every element
    ``sign(x) * fmt(|x| * scale) * unscale``; result in ``x.dtype``.

    ``global_amax``: one element, or one per row of a 2-D ``x`` (:300-316)."""
    shape, dtype = x.shape, x.dtype
    k = shape[-1]
    kp = -(-k // block_size) * block_size
    v = x.reshape(-1, k).to(torch.float32)
    rows = v.shape[0]
    if kp != k:
        v = torch.nn.functional.pad(v, (0, kp - k))
    blocks = v.reshape(rows, kp // block_size, block_size)
    # block abs-max as the kernel reduces it (:189-201, :266): |x| clamped to FLT_MAX, so an
    # infinite element gives a finite amax, and combined with fmaxf, which drops NaN operands
    mags = blocks.abs().clamp(max=torch.finfo(torch.float32).max).nan_to_num(nan=0.0, posinf=None)
    amax = mags.amax(dim=-1)
    bad = (amax == 0) | ~torch.isfinite(amax)
    safe = torch.where(bad, torch.ones_like(amax), amax)
    if global_amax is not None:
        g = global_amax.to(torch.float32).reshape(-1)
        per_row = x.dim() == 2 and g.numel() == shape[0]
        g = g.reshape(rows, 1) if per_row else g[:1].reshape(1, 1)
        g = g.expand_as(amax)
        bad = bad | (g == 0) | ~torch.isfinite(g)
        scale, unscale = _scale_with_global(torch.where(bad, torch.ones_like(g), g), safe, fmt, scale_fmt)
    elif scale_fmt == "E8M0":
        scale, unscale = _scale_e8m0(safe, fmt)
    else:
        scale, unscale = _scale_general(safe, fmt, scale_fmt)
    scale = torch.where(bad, torch.ones_like(scale), scale).unsqueeze(-1)
    unscale = torch.where(bad, torch.ones_like(unscale), unscale).unsqueeze(-1)
    q = convert_to_types(blocks.abs() * scale, fmt) * unscale
    # the reference leaves the sign of a zero or NaN input undefined; +1 here
    y = torch.where(blocks < 0, -q, q)
    return y.reshape(rows, kp)[:, :k].reshape(shape).to(dtype)


# --------------------------------------------------------------------------- packed MXFP4
_E2M1_BOUNDS = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5])
_E2M1_VALUES = torch.tensor([0, 0.5, 1, 1.5, 2, 3, 4, 6])


def mxfp4_quantize(x: torch.Tensor, block_size: int = 32):
    """MXFP4QTensor.quantize, TQ/qtensor/mxfp4_tensor.py:38-83, op for op: fp32 block amax,
    ``e = ceil(max(log2(amax / 6), -127))``, ``x / exp2(e)``, code = sign bit (set unless the value
    is positive) * 8 + number of E2M1 bounds strictly below the magnitude; two codes per byte, even
    index in the low nibble.  Returns (packed uint8 [..., k / 2], scale bytes uint8 [nblocks, 1])."""
    shape = x.shape
    v = x.reshape(-1, block_size)
    amax = v.float().abs().max(dim=-1, keepdim=True).values
    descale = amax / 6.0
    e = torch.ceil(torch.maximum(torch.log2(descale), torch.tensor(-127.0)))
    v = (v / torch.exp2(e)).view(shape)
    sign = torch.sign(v)
    sign_bit = (2 - sign) // 2
    ordinal = torch.sum((v.abs().unsqueeze(-1) - _E2M1_BOUNDS) > 0, dim=-1)
    codes = (sign_bit * 0b1000 + ordinal).to(torch.uint8)
    packed = (codes[..., 1::2] << 4) + codes[..., 0::2]
    return packed, (e + 127).to(torch.uint8)


def mxfp4_dequantize(packed: torch.Tensor, scales: torch.Tensor, block_size: int, shape, dtype):
    """MXFP4QTensor.dequantize, :85-144."""
    codes = torch.stack([packed & 0x0F, (packed >> 4) & 0x0F], dim=-1).reshape(*packed.shape[:-1], -1)
    sign = 1 - 2 * ((codes & 0b1000) >> 3).to(torch.float32)
    mag = _E2M1_VALUES[(codes & 0b0111).long().reshape(-1)].reshape(codes.shape)
    v = (sign * mag).reshape(-1, block_size) * torch.exp2(scales.float() - 127).reshape(-1, 1)
    return v.reshape(shape).to(dtype)
