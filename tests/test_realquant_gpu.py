"""GPU parity of the storage-format kernels (FP8 / INT8 casts, INT4 packs) and the AWQ helpers."""

import json
import os

import pytest
import torch

from conftest import GOLDEN, assert_bits_equal
from modelopt_amd import _hip
from oracle import awq, export, fake_quant, qtensor, reduce

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.bfloat16, torch.float16, torch.float32]
with open(os.path.join(GOLDEN, "reference_vectors.json")) as f:
    VEC = json.load(f)


def _rand(shape, dtype, seed, scale=0.02):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


# ----------------------------------------------------------------------------- FP8
@pytest.mark.parametrize("dtype", DTYPES)
def test_fp8_compress_path_per_tensor_and_channel(dtype):
    x = _rand((48, 96), dtype, 1)
    q_o, s_o = qtensor.fp8_quantize(x)  # scales = amax / 448 in the input dtype
    q = _hip.real_quantize(x.to(DEV), s_o.reshape(1).to(DEV), 1, 1, x.numel(), dtype, _hip.MO_FMT_E4M3)
    assert_bits_equal(q.cpu(), q_o, "per tensor")
    y = _hip.real_dequantize(q, s_o.reshape(1).to(DEV), 1, 1, x.numel(), _hip.MO_FMT_E4M3, dtype)
    assert_bits_equal(y.cpu(), qtensor.fp8_dequantize(q_o, s_o, x.shape, dtype), "dequant")
    q_o, s_o = qtensor.fp8_quantize(x, axis=0)
    q = _hip.real_quantize(x.to(DEV), s_o.reshape(-1).contiguous().to(DEV), 1, 48, 96, dtype,
                           _hip.MO_FMT_E4M3)
    assert_bits_equal(q.cpu(), q_o, "per channel")
    y = _hip.real_dequantize(q, s_o.reshape(-1).contiguous().to(DEV), 1, 48, 96, _hip.MO_FMT_E4M3, dtype)
    assert_bits_equal(y.cpu(), qtensor.fp8_dequantize(q_o, s_o, x.shape, dtype), "dequant channel")


def test_fp8_export_cast_double_and_single_rounding():
    w = _rand((512, 512), torch.bfloat16, 2)
    wsf = reduce.reduce_amax(w).float() / 448.0
    # 0-dim fp32 scale: quotient rounded to bf16 first
    q = _hip.real_quantize(w.to(DEV), wsf.reshape(1).to(DEV), 1, 1, w.numel(), torch.bfloat16,
                           _hip.MO_FMT_E4M3)
    assert_bits_equal(q.cpu(), export.fp8_export_cast(w, wsf), "double rounding")
    # 1-element fp32 scale: fp32 quotient, rounded once
    q1 = _hip.real_quantize(w.to(DEV), wsf.reshape(1).to(DEV), 1, 1, w.numel(), torch.float32,
                            _hip.MO_FMT_E4M3)
    assert_bits_equal(q1.cpu(), export.fp8_export_cast(w, wsf.reshape(1)), "single rounding")
    assert (q.view(torch.uint8) != q1.view(torch.uint8)).any()


@pytest.mark.parametrize("case", [c for c in VEC["qtensor_roundtrip"]
                                  if c["block_sizes"] is None or len(c["block_sizes"]) == 1],
                         ids=lambda c: c["name"])
def test_qtensor_golden_vectors_through_kernels(case):
    """The reference's own golden round trips (tests/gpu/torch/quantization/test_qtensor_cuda.py
    :133-241), computed by the HIP kernels."""
    x = torch.tensor(case["input"], dtype=torch.bfloat16)
    want = torch.tensor(case["output"], dtype=torch.bfloat16)
    xd = x.to(DEV)
    bits, bs, axis = case["num_bits"], case["block_sizes"], case["axis"]
    if bits == 4:
        b = bs["-1"]
        packed, scales = _hip.int4_block_quantize(xd, b)
        y = _hip.int4_block_dequantize(packed, scales, b)[: x.numel()].reshape(x.shape)
    else:
        fmt = _hip.MO_FMT_INT8 if bits == 8 else _hip.MO_FMT_E4M3
        bound = 127.0 if bits == 8 else 448.0
        if bs:  # 1-D blocks along the last dim: rows of length block
            b = bs["-1"]
            nblk = x.numel() // b
            acc = torch.zeros(nblk, dtype=torch.float32, device=DEV)
            _hip.absmax_into(xd, acc, 1, nblk, b)
            outer, ax, inner = 1, nblk, b
        elif axis is None:
            acc = torch.zeros(1, dtype=torch.float32, device=DEV)
            _hip.absmax_into(xd, acc, 1, 1, x.numel())
            outer, ax, inner = 1, 1, x.numel()
        else:
            acc = torch.zeros(x.shape[0], dtype=torch.float32, device=DEV)
            _hip.absmax_into(xd, acc, 1, x.shape[0], x.shape[1])
            outer, ax, inner = 1, x.shape[0], x.shape[1]
        scales = acc.to(torch.bfloat16) / bound
        q = _hip.real_quantize(xd, scales, outer, ax, inner, torch.bfloat16, fmt)
        y = _hip.real_dequantize(q, scales, outer, ax, inner, fmt, torch.bfloat16)
    assert torch.allclose(y.cpu(), want), (y.cpu(), want)


@pytest.mark.parametrize("case", VEC["qtensor_roundtrip"], ids=lambda c: c["name"])
def test_qtensor_golden_vectors_through_the_quantizer(case):
    """The same golden round trips the way the reference's test drives them: a real-quantising
    ``TensorQuantizer`` (quantize on the first call, dequantize on the second), including the
    2-D block and padded cases (tests/gpu/torch/quantization/test_qtensor_cuda.py:243-268)."""
    from modelopt_amd.torch.quantization.config import QuantizerAttributeConfig
    from modelopt_amd.torch.quantization.nn import TensorQuantizer

    bits = tuple(case["num_bits"]) if isinstance(case["num_bits"], list) else case["num_bits"]
    bs = None if case["block_sizes"] is None else {int(k): v for k, v in case["block_sizes"].items()}
    q = TensorQuantizer(QuantizerAttributeConfig(num_bits=bits, block_sizes=bs, fake_quant=False,
                                                 axis=case["axis"])).to(DEV)
    x = torch.tensor(case["input"], dtype=torch.bfloat16, device=DEV)
    packed = q(x)
    out = q(packed)
    want = torch.tensor(case["output"], dtype=torch.bfloat16)
    assert out.shape == x.shape and torch.allclose(out.cpu(), want), (out.cpu(), want)


@pytest.mark.parametrize("fmt", ["fp8", "int8"])
@pytest.mark.parametrize("shape,blocks", [((256, 384), {-1: 128, -2: 128}), ((100, 200), {-1: 64, -2: 32}),
                                           ((3, 40, 96), {-1: 32}), ((130, 70), {-1: 16}),
                                           ((2, 128, 256), {-1: 128, -2: 64}), ((3, 50, 72), {-1: 24, -2: 16}),
                                           ((64, 96), {-1: 12, -2: 16})])
def test_block_scales_on_any_dims_match_restatement(fmt, shape, blocks, monkeypatch):
    """2-D tiles, padding on either dim, 3-D inputs: codes, scales and dequantised values equal
    the CPU restatement of the reference's pad / repeat_interleave formulation bit for bit.
    Tiles on the last two dims whose width is a multiple of 8 are cast in place (no copy that
    gathers every tile into a row)."""
    from modelopt_amd.torch.quantization.qtensor import FP8QTensor, INT8QTensor

    in_place = []
    for name in ("real_quantize_blocks2d", "real_dequantize_blocks2d"):
        real = getattr(_hip, name)
        monkeypatch.setattr(_hip, name, lambda *a, _real=real, _name=name: in_place.append(_name) or _real(*a))
    x = _rand(shape, torch.bfloat16, 21, scale=1.0)
    if fmt == "fp8":
        q_o, s_o = qtensor.fp8_quantize(x, block_sizes=blocks)
        want = qtensor.fp8_dequantize(q_o, s_o, x.shape, torch.bfloat16, blocks)
        qt, s = FP8QTensor.quantize(x.to(DEV), block_sizes=blocks)
    else:
        q_o, s_o = qtensor.int8_quantize(x, block_sizes=blocks)
        want = qtensor.int8_dequantize(q_o, s_o, x.shape, torch.bfloat16, blocks)
        qt, s = INT8QTensor.quantize(x.to(DEV), block_sizes=blocks)
    assert_bits_equal(s.cpu(), s_o, "scales")
    assert_bits_equal(qt._quantized_data.cpu(), q_o, "codes")
    got = qt.dequantize(scale=s, block_sizes=blocks)
    assert_bits_equal(got.cpu(), want, "dequantised")
    tiled = len(blocks) == 2 and blocks[-1] % 8 == 0
    assert in_place == (["real_quantize_blocks2d", "real_dequantize_blocks2d"] if tiled else [])


# ----------------------------------------------------------------------------- INT8 / INT4
@pytest.mark.parametrize("dtype", DTYPES)
def test_int8_quantize_dequantize(dtype):
    x = _rand((40, 64), dtype, 3, scale=1.0)
    q_o, s_o = qtensor.int8_quantize(x, axis=0)
    s = s_o.reshape(-1).contiguous().to(DEV)
    q = _hip.real_quantize(x.to(DEV), s, 1, 40, 64, dtype, _hip.MO_FMT_INT8)
    assert_bits_equal(q.cpu(), q_o, "int8 codes")
    y = _hip.real_dequantize(q, s, 1, 40, 64, _hip.MO_FMT_INT8, dtype)
    assert_bits_equal(y.cpu(), qtensor.int8_dequantize(q_o, s_o, x.shape, dtype), "int8 dequant")


@pytest.mark.parametrize("cls_name", ["FP8QTensor", "INT8QTensor"])
def test_qtensor_scales_on_separated_dims(cls_name):
    """Scales given on two dims with a reduced dim between them ([a, 1, c]): what the reference
    computes by broadcasting, (x / scales) cast to the storage type and back."""
    from modelopt_amd.torch.quantization import qtensor as q_mod
    cls = getattr(q_mod, cls_name)
    bound = 448.0 if cls_name == "FP8QTensor" else 127.0
    x = _rand((6, 10, 16), torch.bfloat16, 21, scale=1.0)
    scales = (x.abs().amax(dim=1, keepdim=True) / bound).to(torch.bfloat16)
    assert scales.shape == (6, 1, 16)
    qt, s_out = cls.quantize(x.to(DEV), scales=scales.to(DEV))
    q = qt._quantized_data.cpu()
    if cls_name == "FP8QTensor":
        q_o, _ = qtensor.fp8_quantize(x, scales=scales)
        want_y = qtensor.fp8_dequantize(q_o, scales, x.shape, torch.bfloat16)
    else:
        q_o, _ = qtensor.int8_quantize(x, scales=scales)
        want_y = qtensor.int8_dequantize(q_o, scales, x.shape, torch.bfloat16)
    assert torch.equal(q.view(torch.uint8), q_o.view(torch.uint8))
    y = qt.dequantize(torch.bfloat16, scale=scales.to(DEV)).cpu()
    assert_bits_equal(y, want_y, "dequantised")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape,bs", [((64, 256), 128), ((32, 64), 64), ((1, 10), 4), ((16, 48), 32)])
def test_int4_block_quantize(dtype, shape, bs):
    x = _rand(shape, dtype, 4, scale=1.0)
    p_o, s_o = qtensor.int4_quantize(x, bs)
    packed, scales = _hip.int4_block_quantize(x.to(DEV), bs)
    assert_bits_equal(scales.cpu(), s_o, "scales")
    assert torch.equal(packed.cpu(), p_o.reshape(-1))  # includes the zero-padded tail block
    y = _hip.int4_block_dequantize(packed, scales, bs)[: x.numel()].reshape(shape)
    y_o = qtensor.int4_dequantize(p_o, s_o, bs, shape, dtype)
    assert_bits_equal(y.cpu(), y_o, "dequant")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(64, 256), (2, 8, 128), (130, 384)])
def test_int4_awq_export_pack(dtype, shape):
    w = _rand(shape, dtype, 5)
    bs = 128
    amax = reduce.reduce_block_amax(w, {-1: bs})
    ws = amax.float() / 7.0
    want = export.pack_int4_in_uint8(w, ws)
    got = _hip.int4_pack_rows(w.to(DEV), ws.to(DEV))
    assert_bits_equal(got.cpu(), want, "packed rows")


# ----------------------------------------------------------------------------- exhaustive / edge
def _all_patterns(dtype):
    """Every 16-bit pattern of a half-width dtype (NaNs, infinities, zeros, subnormals included);
    for fp32 the bf16 patterns widened plus a few million random bit patterns."""
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    if dtype != torch.float32:
        return bits.view(dtype)
    wide = bits.view(torch.bfloat16).float()
    g = torch.Generator().manual_seed(11)
    rnd = torch.randint(-2**31, 2**31 - 1, (1 << 20,), generator=g, dtype=torch.int64).to(torch.int32)
    return torch.cat([wide, rnd.view(torch.float32)])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("fmt", ["e4m3", "int8"])
def test_storage_cast_every_pattern_and_extreme_scales(dtype, fmt):
    x = _all_patterns(dtype)
    code = _hip.MO_FMT_E4M3 if fmt == "e4m3" else _hip.MO_FMT_INT8
    for sv in (1.0, 0.0123, 3.0e-5, 7.7e3, 2.0**-70, 2.0**70, 1.0e-30, 0.0, float("inf"), -0.5):
        scale = torch.tensor([sv], dtype=torch.float32)
        if fmt == "e4m3":
            want = (x / scale).to(torch.float8_e4m3fn)
        else:
            want = (x / scale).round().clamp(-128, 127).to(torch.int8)
        got = _hip.real_quantize(x.to(DEV), scale.to(DEV), 1, 1, x.numel(), torch.float32, code)
        if fmt == "int8":
            # a NaN quotient has no defined int8 value in the reference (float -> int cast of NaN)
            ok = ~torch.isnan(x / scale)
            assert torch.equal(got.cpu()[ok], want[ok]), f"scale {sv}"
        else:
            assert_bits_equal(got.cpu(), want, f"scale {sv}")


@pytest.mark.parametrize("fmt", ["e4m3", "int8"])
def test_storage_cast_bf16_by_bf16_every_pattern_and_every_scale_significand(fmt):
    """bf16 / bf16 rounded to bf16 takes x times the reciprocal of the scale when the scale is
    mid-range: every input pattern under every significand of the scale at several exponents
    (the outermost ones go through the division), per row, per short row and per tensor."""
    x = _all_patterns(torch.bfloat16)
    code = _hip.MO_FMT_E4M3 if fmt == "e4m3" else _hip.MO_FMT_INT8
    sig = 1.0 + torch.arange(128, dtype=torch.float32) / 128.0
    s = torch.cat([sig * 2.0**e for e in (-100, -64, -21, -3, 0, 6, 63, 70)]).to(torch.bfloat16)
    rows = s.numel()
    xs = x.repeat(rows, 1)                                              # [rows, 65536]
    q = xs / s[:, None]                                                 # bf16 by type promotion

    def want_of(q):
        return q.to(torch.float8_e4m3fn) if fmt == "e4m3" else q.round().clamp(-128, 127).to(torch.int8)

    def check(got, q, what):
        if fmt == "int8":
            ok = ~torch.isnan(q)      # a NaN quotient has no defined int8 value in the reference
            assert torch.equal(got.cpu()[ok], want_of(q)[ok]), what
        else:
            assert_bits_equal(got.cpu(), want_of(q), what)

    xd, sd = xs.to(DEV), s.to(DEV)
    check(_hip.real_quantize(xd, sd, 1, rows, 65536, torch.bfloat16, code), q, "one scale per long row")
    short = sd.repeat_interleave(64)                                    # the same data as rows of 1024
    check(_hip.real_quantize(xd.view(rows * 64, 1024), short, 1, rows * 64, 1024, torch.bfloat16, code).view(rows, 65536),
          q, "one scale per short row")
    for i in (0, 77, 5 * 128 + 127, 3 * 128 + 1, 6 * 128 + 64):
        got = _hip.real_quantize(xd[i].contiguous(), sd[i].reshape(1), 1, 1, 65536, torch.bfloat16, code)
        check(got, q[i], f"per tensor, scale {float(s[i])}")


@pytest.mark.parametrize("k", [2048, 2112, 4096, 6144, 14336])
@pytest.mark.parametrize("rows", [3, 37])
def test_storage_cast_row_scales_on_long_rows(rows, k):
    """One scale per row on rows of 256 chunks and more: widths that are a multiple of 2048 take
    flat tiles with one scale per round of 256 chunks, the others one row per workgroup; the
    tensor ends in the middle of a tile either way."""
    g = torch.Generator().manual_seed(rows * 100003 + k)
    x = (torch.randn((rows, k), generator=g) * 2).to(torch.bfloat16)
    x[1, 5] = float("inf"); x[2, :] = 0.0; x[0, 3] = -0.0
    for sdtype in (torch.float32, torch.bfloat16):
        s = (x.float().abs().amax(dim=1).clamp(min=1e-3, max=1e30) / 448.0).to(sdtype)
        quot = x / s[:, None]                 # fp32 scales promote to fp32, bf16 scales stay bf16
        for fmt, code in (("e4m3", _hip.MO_FMT_E4M3), ("int8", _hip.MO_FMT_INT8)):
            got = _hip.real_quantize(x.to(DEV), s.to(DEV), 1, rows, k, quot.dtype, code)
            if fmt == "e4m3":
                want = quot.to(torch.float8_e4m3fn)
                assert_bits_equal(got.cpu(), want, f"{fmt}, {sdtype} scales")
                y = _hip.real_dequantize(got, s.to(DEV), 1, rows, k, code, torch.bfloat16)
                assert_bits_equal(y.cpu(), want.to(torch.bfloat16) * s[:, None].to(torch.bfloat16), "dequant")
            else:
                ok = ~torch.isnan(quot)
                want = quot.round().clamp(-128, 127).to(torch.int8)
                assert torch.equal(got.cpu()[ok], want[ok]), f"{fmt}, {sdtype} scales"
                y = _hip.real_dequantize(got, s.to(DEV), 1, rows, k, code, torch.bfloat16)
                assert_bits_equal(y.cpu()[ok], (want.to(torch.bfloat16) * s[:, None].to(torch.bfloat16))[ok], "dequant")


def test_storage_cast_scales_on_a_middle_dim_of_long_rows():
    """[outer, axis, inner] with outer > 1 and inner a multiple of 2048: the scale index wraps
    around after every ``axis`` rows."""
    g = torch.Generator().manual_seed(21)
    x = (torch.randn((5, 3, 4096), generator=g) * 2).to(torch.bfloat16)
    s = torch.tensor([0.011, 0.5, 3.0])
    quot = x / s[None, :, None]                                    # fp32 by promotion
    want = quot.to(torch.float8_e4m3fn)
    got = _hip.real_quantize(x.to(DEV), s.to(DEV), 5, 3, 4096, torch.float32, _hip.MO_FMT_E4M3)
    assert_bits_equal(got.cpu(), want, "quantize")
    y = _hip.real_dequantize(got, s.to(DEV), 5, 3, 4096, _hip.MO_FMT_E4M3, torch.bfloat16)
    assert_bits_equal(y.cpu(), want.to(torch.bfloat16) * s[None, :, None].to(torch.bfloat16), "dequantize")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_storage_cast_row_scales_and_unaligned_views(dtype):
    g = torch.Generator().manual_seed(12)
    x = (torch.randn((96, 264), generator=g) * 3).to(dtype)
    x[5, 7] = float("inf"); x[6, :] = 0.0; x[9, 3] = float("nan"); x[11, 8] = -0.0
    s = (x.float().abs().amax(dim=1).clamp(min=1e-3) / 448.0)
    want = (x / s[:, None]).to(torch.float8_e4m3fn)        # fp32 [96, 1] scale -> fp32 quotient
    got = _hip.real_quantize(x.to(DEV), s.to(DEV), 1, 96, 264, torch.float32, _hip.MO_FMT_E4M3)
    assert_bits_equal(got.cpu(), want, "row scales, tiled path")
    y = _hip.real_dequantize(got, s.to(DEV), 1, 96, 264, _hip.MO_FMT_E4M3, dtype)
    assert_bits_equal(y.cpu(), want.to(dtype) * s[:, None].to(dtype), "row scales dequant")
    # odd inner size and an odd element offset: the guarded path
    xo = torch.zeros(96 * 263 + 1, dtype=dtype)
    xo[1:] = x[:, :263].reshape(-1)
    xd = xo.to(DEV)[1:].view(96, 263)
    want = (x[:, :263] / s[:, None]).to(torch.float8_e4m3fn)
    got = _hip.real_quantize(xd, s.to(DEV), 1, 96, 263, torch.float32, _hip.MO_FMT_E4M3)
    assert_bits_equal(got.cpu(), want, "row scales, guarded path")
    y = _hip.real_dequantize(got, s.to(DEV), 1, 96, 263, _hip.MO_FMT_E4M3, dtype)
    assert_bits_equal(y.cpu(), want.to(dtype) * s[:, None].to(dtype), "guarded dequant")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bs", [8, 16, 128, 512, 24, 1024])
def test_int4_block_quantize_special_blocks(dtype, bs):
    """Zero blocks (scale = inf), huge and tiny magnitudes, infinities; power-of-two block sizes
    take the tiled kernels, the others (and block sizes above 512) the general ones."""
    g = torch.Generator().manual_seed(13)
    nblk = 40
    x = torch.randn((nblk, bs), generator=g)
    x[0] = 0.0
    x[1] *= 1e30
    x[2] *= 1e-30
    x[3, 1] = float("inf")
    x[4, 0] = -0.0
    x[5] = 7.0
    x = x.to(dtype)
    p_o, s_o = qtensor.int4_quantize(x, bs)
    packed, scales = _hip.int4_block_quantize(x.to(DEV), bs)
    assert_bits_equal(scales.cpu(), s_o, "scales")
    finite = torch.isfinite(s_o.float()).reshape(-1) & (s_o.float().reshape(-1) != 0)
    got = packed.cpu().reshape(nblk, -1)
    assert torch.equal(got[finite], p_o.reshape(nblk, -1)[finite])
    assert int(got[0].max()) == 0      # all-zero block: scale inf, 0 * inf = NaN packs as code 0
    y = _hip.int4_block_dequantize(packed, scales, bs).reshape(nblk, bs)
    y_o = qtensor.int4_dequantize(got.reshape(p_o.shape), s_o, bs, x.shape, dtype)
    assert_bits_equal(y.cpu(), y_o, "dequant")


def test_int4_dequantize_every_code_under_every_bf16_scale():
    """bf16 takes code * reciprocal instead of the division when the scale is mid-range: all 16
    codes under every finite positive and negative bf16 scale (the ends of the exponent range and
    the negative ones go through the division) against the reference's expression."""
    bits = torch.arange(0x10000, dtype=torch.int32)
    scales = bits.to(torch.int16).view(torch.bfloat16)
    scales = scales[torch.isfinite(scales.float()) & (scales.float() != 0)].contiguous()
    nblk = scales.numel()
    codes = torch.arange(16, dtype=torch.uint8)
    packed = (codes[0::2] << 4 | codes[1::2]).repeat(nblk)          # a block of 16 holds each code once
    y = _hip.int4_block_dequantize(packed.to(DEV), scales.to(DEV), 16)
    y_o = qtensor.int4_dequantize(packed, scales.reshape(-1, 1), 16, (nblk, 16), torch.bfloat16)
    assert_bits_equal(y.cpu().reshape(nblk, 16), y_o, "dequant")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_int4_awq_export_pack_large_and_special(dtype):
    g = torch.Generator().manual_seed(14)
    w = (torch.randn((256, 1024), generator=g) * 0.05).to(dtype)
    w[3, 130:140] = 0.0
    w[4, 5] = -0.0
    ws = reduce.reduce_block_amax(w, {-1: 64}).float() / 7.0
    ws[7, 2] = 1e-30      # quotients far outside the clamp range
    ws[8, 1] = 2.0**70    # scale outside the reciprocal path's range
    want = export.pack_int4_in_uint8(w, ws)
    got = _hip.int4_pack_rows(w.to(DEV), ws.to(DEV))
    assert_bits_equal(got.cpu(), want, "packed rows")
    # k not a multiple of 8 chunks per scale: general kernel
    w2 = w[:, :1020].contiguous()
    ws2 = reduce.reduce_block_amax(w2, {-1: 12}).float() / 7.0
    assert_bits_equal(_hip.int4_pack_rows(w2.to(DEV), ws2.to(DEV)).cpu(),
                      export.pack_int4_in_uint8(w2, ws2), "packed rows, block 12")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape,bs", [((256, 1024), 128), ((2, 64, 256), 64), ((66, 1020), 12)])
def test_int4_awq_export_pack_with_scales_in_the_weight_s_own_type(dtype, shape, bs):
    """``weight / scales`` of two tensors of one 16-bit type is rounded to that type before
    ``.round()`` (type promotion in the reference's expression, export/quant_utils.py:704-706): about
    1 % of the codes differ from the fp32 quotient the exporter's fp32 scales give.  Both routes
    against the literal expression on the CPU, the second also with scales of the other 16-bit
    type (promoted to fp32)."""
    from modelopt_amd.torch.export.quant_utils import pack_int4_in_uint8

    g = torch.Generator().manual_seed(16)
    w = (torch.randn(shape, generator=g) * 0.05).to(dtype)
    w[..., 3, 8:24] = 0.0
    ws = (reduce.reduce_block_amax(w, {-1: bs}).float() / 7.0).to(dtype)
    ws[..., 5, 0] = 1e-4 if dtype == torch.float16 else 1e-30   # quotients far outside the clamp range
    if dtype == torch.bfloat16:
        ws[..., 6, 1] = 2.0**70                                 # scale outside the reciprocal path's range
    want = export.pack_int4_in_uint8(w, ws)
    assert not torch.equal(want, export.pack_int4_in_uint8(w, ws.float())), "the case must differ from fp32"
    assert_bits_equal(pack_int4_in_uint8(w.to(DEV), ws.to(DEV)).cpu(), want, "16-bit quotient")
    assert_bits_equal(_hip.int4_pack_rows(w.to(DEV), ws.float().to(DEV), dtype).cpu(), want, "binding")
    other = torch.float16 if dtype == torch.bfloat16 else torch.bfloat16
    ws_o = (reduce.reduce_block_amax(w, {-1: bs}).float() / 7.0).to(other)
    assert_bits_equal(pack_int4_in_uint8(w.to(DEV), ws_o.to(DEV)).cpu(), export.pack_int4_in_uint8(w, ws_o),
                      "mixed 16-bit types promote to fp32")


def test_int4_awq_export_pack_with_a_padded_last_block():
    """in_features that the 128-wide blocks do not tile (reference export/quant_utils.py:701-706:
    block size = in_dim // scales per row, scale index = column // that).  192 columns with two
    scales per row pack with 96-wide groups, as the reference's expression does; 320 columns
    with three scales index past the last scale there, and raise here too."""
    from modelopt_amd.torch.export.quant_utils import pack_int4_in_uint8

    g = torch.Generator().manual_seed(15)
    w = (torch.randn((64, 192), generator=g) * 0.05).to(torch.bfloat16)
    ws = reduce.reduce_block_amax(reduce.reduce_block_padding(w, {-1: 128}), {-1: 128}).float() / 7.0
    assert ws.shape == (64, 2)
    assert_bits_equal(pack_int4_in_uint8(w.to(DEV), ws.to(DEV)).cpu(), export.pack_int4_in_uint8(w, ws),
                      "96-wide groups")
    w = (torch.randn((64, 320), generator=g) * 0.05).to(torch.bfloat16)
    ws = reduce.reduce_block_amax(reduce.reduce_block_padding(w, {-1: 128}), {-1: 128}).float() / 7.0
    with pytest.raises(IndexError):
        export.pack_int4_in_uint8(w, ws)
    with pytest.raises(IndexError):
        pack_int4_in_uint8(w.to(DEV), ws.to(DEV))


# ----------------------------------------------------------------------------- AWQ helpers
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_mul_cols_both_scale_dtypes(dtype):
    x = _rand((33, 72), dtype, 6, scale=1.0)
    s = (torch.rand(72) + 0.5)
    y = _hip.mul_cols(x.to(DEV), s.to(dtype).to(DEV))
    assert_bits_equal(y.cpu(), x * s.to(dtype), "T * T")
    y = _hip.mul_cols(x.to(DEV), s.to(DEV))
    assert_bits_equal(y.cpu(), (x * s[None, :]).to(dtype), "T * fp32 row")


@pytest.mark.parametrize("k", [512, 200])
def test_fused_scale_block_int4_qdq(k):
    w = _rand((96, k), torch.bfloat16, 7)
    s = (torch.rand(k) * 2 + 0.25).to(torch.bfloat16)
    want = awq.int4_block_qdq(w * s, 128)
    got = _hip.scale_block_int_qdq(w.to(DEV), s.to(DEV), 128, 4, False, False)
    assert_bits_equal(got.cpu(), want.contiguous(), "fused scale + block qdq")
    got = _hip.scale_block_int_qdq(w.to(DEV), None, 128, 4, False, False)
    assert_bits_equal(got.cpu(), awq.int4_block_qdq(w, 128).contiguous(), "no scale")


def test_awq_column_statistics_close_to_oracle():
    x = _rand((512, 256), torch.bfloat16, 8, scale=1.0)
    acc = torch.zeros(256, dtype=torch.float32, device=DEV)
    _hip.abs_colsum_into(x.to(DEV), acc)
    got = (acc / 512).to(torch.bfloat16).float().cpu()
    want = awq.awq_act_scale(x)
    assert torch.allclose(got, want, rtol=2 ** -7, atol=0)  # at most one bf16 ulp (summation order)
    assert (got == want).float().mean() > 0.95
    w = _rand((128, 256), torch.bfloat16, 9)
    blk = torch.zeros(128 * 2, dtype=torch.float32, device=DEV)
    _hip.absmax_into(w.to(DEV), blk, 1, 256, 128)
    acc = torch.zeros(256, dtype=torch.float32, device=DEV)
    _hip.abs_colsum_into(w.to(DEV), acc, blk, 128)
    got = (acc / 128).to(torch.bfloat16).float().cpu()
    want = awq.awq_weight_scale(w, 128)
    assert torch.allclose(got, want, rtol=2 ** -7, atol=0)
    assert (got == want).float().mean() > 0.95


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("rows,k,block", [(1100, 4096, 128), (16384, 512, 64), (300, 4096, 128),
                                          (64, 256, 8), (33000, 264, 0), (1000, 264, 0)])
def test_column_sums_two_pass_kernel(dtype, rows, k, block):
    """The vectorised two-pass path (k % 8 == 0, a few million elements and more; the smaller
    cases here take the one-pass kernel and are held to the same figures): every term is rounded as the
    tensor expression rounds it (|x| / T(block amax + tiny) in T), the fp32 sum of the terms is
    compared with their float64 sum; all-zero blocks, NaN and inf included; results do not depend
    on scheduling (no atomics) and add to what the accumulator held."""
    g = torch.Generator().manual_seed(rows + k)
    x = (torch.randn(rows, k, generator=g) * torch.exp(torch.randn(rows, 1, generator=g))).to(dtype)
    if block:
        x[5, :block] = 0                      # an all-zero block: |x| / tiny
        x[7, block:2 * block] *= 1e-3
    xd = x.to(DEV)
    acc = torch.full((k,), 2.5, dtype=torch.float32, device=DEV)
    if block:
        blk = torch.zeros(rows * (k // block), dtype=torch.float32, device=DEV)
        _hip.absmax_into(xd, blk, 1, rows * (k // block), block)
        _hip.abs_colsum_into(xd, acc, blk, block)
        tiny = torch.finfo(dtype).tiny
        peak = x.view(rows, k // block, block).abs().amax(-1, keepdim=True)
        terms = (x.view(rows, k // block, block).abs() / (peak + tiny)).view(rows, k)
        assert terms.dtype == dtype
    else:
        _hip.abs_colsum_into(xd, acc)
        terms = x.abs()
    want = terms.double().sum(0) + 2.5
    got = acc.cpu().double()
    assert torch.allclose(got, want, rtol=3e-6, atol=0), float(((got - want).abs() / want).max())
    again = torch.full((k,), 2.5, dtype=torch.float32, device=DEV)
    _hip.abs_colsum_into(xd, again, blk if block else None, block)
    two_pass = rows * k >= ((1 << 22) if block else (1 << 23))
    if two_pass:          # fixed summation order; the one-pass kernel folds with atomics
        assert torch.equal(again, acc)
    else:
        assert torch.allclose(again, acc, rtol=1e-6)
    # NaN and inf propagate to their columns only
    x2 = x.clone()
    x2[3, 9] = float("nan")
    x2[4, 17] = float("inf")
    acc2 = torch.zeros(k, dtype=torch.float32, device=DEV)
    if block:
        blk2 = torch.zeros(rows * (k // block), dtype=torch.float32, device=DEV)
        _hip.absmax_into(x2.to(DEV), blk2, 1, rows * (k // block), block)
        _hip.abs_colsum_into(x2.to(DEV), acc2, blk2, block)
        peak = x2.view(rows, k // block, block).abs().amax(-1, keepdim=True)
        want2 = (x2.view(rows, k // block, block).abs() / (peak + torch.finfo(dtype).tiny)).view(rows, k).double().sum(0)
    else:
        _hip.abs_colsum_into(x2.to(DEV), acc2)
        want2 = x2.abs().double().sum(0)
    got2 = acc2.cpu().double()
    assert torch.equal(torch.isnan(got2), torch.isnan(want2))
    assert torch.equal(torch.isinf(got2), torch.isinf(want2))
    ok = torch.isfinite(want2)
    assert torch.allclose(got2[ok], want2[ok], rtol=3e-6, atol=0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("rows,k,block", [(1100, 4096, 128), (4100, 1024, 512), (300, 4096, 16),
                                          (64, 256, 8), (1, 512, 32), (2000, 2560, 256), (257, 192, 64)])
def test_weight_scale_sums_in_one_pass(dtype, rows, k, block):
    """Block abs-max, quotient and column sum in one kernel: the same bits as the two-pass
    column sum fed the block abs-max from its own kernel (same slabs, same order), and the
    float64 sum of the tensor expression's terms; all-zero blocks, quotients in fp32's denormal
    range, NaN and inf included."""
    g = torch.Generator().manual_seed(rows + k + block)
    x = (torch.randn(rows, k, generator=g) * torch.exp(torch.randn(rows, 1, generator=g))).to(dtype)
    if rows > 8:
        x[5, :block] = 0                      # an all-zero block: |x| / tiny
        x[7, :block] *= 1e-3
        if dtype != torch.float16:            # tiny elements beside a large one: denormal quotients
            x[2, :block] = torch.tensor(3e-38, dtype=dtype)
            x[2, 1] = 2.0 ** 60
            x[6, :block] = torch.tensor(1e-20, dtype=dtype)
            x[6, 3] = 2.0 ** 63
    xd = x.to(DEV)
    acc = torch.full((k,), 2.5, dtype=torch.float32, device=DEV)
    assert _hip.weight_scale_colsum_into(xd, acc, block)
    tiny = torch.finfo(dtype).tiny
    blocks = x.view(rows, k // block, block)
    terms = (blocks.abs() / (blocks.abs().amax(-1, keepdim=True) + tiny)).view(rows, k)
    assert terms.dtype == dtype
    want = terms.double().sum(0) + 2.5
    got = acc.cpu().double()
    assert torch.allclose(got, want, rtol=3e-6, atol=0), float(((got - want).abs() / want).max())
    if rows == 1:                             # one term per column: exact
        assert torch.equal(acc.cpu(), terms[0].float() + 2.5)
    if rows >= 64:      # over the same row slabs: the bits of the column sum fed the block abs-max
        blk = torch.zeros(rows * (k // block), dtype=torch.float32, device=DEV)
        _hip.absmax_into(xd, blk, 1, rows * (k // block), block)
        slabs = 7
        work = torch.empty(slabs * k, dtype=torch.float32, device=DEV)
        two, one = (torch.full((k,), 2.5, dtype=torch.float32, device=DEV) for _ in range(2))
        _hip.call("mo_abs_colsum_staged", xd, xd.data_ptr(), rows, k, _hip.dtype_code(dtype),
                  blk.data_ptr(), block, two.data_ptr(), work.data_ptr(), slabs, None)
        torch.cuda.synchronize()
        _hip.call("mo_weight_scale_colsum", xd, xd.data_ptr(), rows, k, _hip.dtype_code(dtype),
                  block, one.data_ptr(), work.data_ptr(), slabs, None)
        assert torch.equal(two, one)
        assert torch.allclose(one, acc, rtol=2e-6, atol=0)
    x2 = x.clone()
    x2[0, 9] = float("nan")
    x2[rows // 2, k - 3] = float("inf")
    acc2 = torch.zeros(k, dtype=torch.float32, device=DEV)
    assert _hip.weight_scale_colsum_into(x2.to(DEV), acc2, block)
    b2 = x2.view(rows, k // block, block)
    want2 = (b2.abs() / (b2.abs().amax(-1, keepdim=True) + tiny)).view(rows, k).double().sum(0)
    got2 = acc2.cpu().double()
    assert torch.equal(torch.isnan(got2), torch.isnan(want2))
    ok = torch.isfinite(want2)
    assert torch.allclose(got2[ok], want2[ok], rtol=3e-6, atol=0)


def test_weight_scale_bf16_quotients_term_by_term():
    """One row, so every column sum is a single term: every pair of bf16 significands at
    several exponent distances (subnormal numerators too), each quotient rounded exactly as
    the tensor expression rounds it."""
    sig = torch.arange(128, 256, dtype=torch.float32)
    rows = []
    for shift in (0, 1, 5, 40, 120):
        for d in sig:
            # a block of 256: the first 128 hold d (the abs-max), the rest every numerator
            num = sig * 2.0 ** -shift
            num = torch.where(num <= d, num, num / 2)
            rows.append(torch.cat([d.expand(128), num]))
    x = torch.stack(rows).reshape(1, -1).to(torch.bfloat16)
    sub = torch.arange(1, 129, dtype=torch.float32) * 2.0 ** -133        # bf16 subnormals
    x = torch.cat([x, torch.cat([torch.full((128,), 2.0 ** -120), sub]).to(torch.bfloat16).reshape(1, -1),
                   torch.cat([torch.full((128,), 2.0 ** -126), sub]).to(torch.bfloat16).reshape(1, -1)], 1)
    k = x.shape[1]
    acc = torch.zeros(k, dtype=torch.float32, device=DEV)
    assert _hip.weight_scale_colsum_into(x.to(DEV), acc, 256)
    blocks = x.view(1, k // 256, 256)
    want = (blocks.abs() / (blocks.abs().amax(-1, keepdim=True) + torch.finfo(torch.bfloat16).tiny))
    assert torch.equal(acc.cpu(), want.view(-1).float())


def test_weight_scale_one_pass_refuses_other_blocks():
    x = torch.ones(64, 192, dtype=torch.bfloat16, device=DEV)
    acc = torch.zeros(192, dtype=torch.float32, device=DEV)
    assert not _hip.weight_scale_colsum_into(x, acc, 128)      # does not divide 192
    assert not _hip.weight_scale_colsum_into(x, acc, 24)       # not a power of two
    assert not _hip.weight_scale_colsum_into(x, acc, 4)
    assert float(acc.abs().sum()) == 0.0


def test_sq_diff_loss():
    a, b = _rand((256, 512), torch.bfloat16, 10, 1.0), _rand((256, 512), torch.bfloat16, 11, 1.0)
    acc = torch.zeros(1, dtype=torch.float64, device=DEV)
    _hip.sq_diff_sum_into(a.to(DEV), b.to(DEV), acc)
    want = (a - b).float().pow(2).mean().item()
    assert acc.item() / a.numel() == pytest.approx(want, rel=1e-5)
