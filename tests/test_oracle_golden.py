"""Pins the CPU oracle: reference golden vectors, library routines, brute force, invariants."""

import json
import os

import pytest
import torch

from conftest import GOLDEN, assert_bits_equal, load_export_vectors
from oracle import export, fake_quant, nf4, qtensor, reduce

with open(os.path.join(GOLDEN, "reference_vectors.json")) as f:
    VEC = json.load(f)


def _bs(d):
    return None if d is None else {int(k): v for k, v in d.items()}


# ----------------------------------------------------------------------------- QTensor round trips
@pytest.mark.parametrize("case", VEC["qtensor_roundtrip"], ids=lambda c: c["name"])
def test_qtensor_roundtrip_golden(case):
    x = torch.tensor(case["input"], dtype=torch.bfloat16)
    want = torch.tensor(case["output"], dtype=torch.bfloat16)
    bits, bs, axis = case["num_bits"], _bs(case["block_sizes"]), case["axis"]
    if bits == 4:
        packed, scales = qtensor.int4_quantize(x, bs[-1])
        got = qtensor.int4_dequantize(packed, scales, bs[-1], x.shape, torch.bfloat16)
    elif bits == 8:
        q, scales = qtensor.int8_quantize(x, axis=axis, block_sizes=bs)
        if bs:  # the quantizer pads before quantising; these cases need no padding
            assert all(x.shape[d] % b == 0 for d, b in bs.items())
        got = qtensor.int8_dequantize(q, scales, x.shape, torch.bfloat16, bs)
    else:
        q, scales = qtensor.fp8_quantize(x, axis=axis, block_sizes=bs)
        got = qtensor.fp8_dequantize(q, scales, x.shape, torch.bfloat16, bs)
    assert torch.allclose(got, want), (got, want)


# ----------------------------------------------------------------------------- NVFP4
def _twin_cast_fp4(w):
    """Independent formula from the reference's own test: count of bounds exceeded plus the
    tie mask [0,1,0,1,0,1,0] (tests/gpu/torch/quantization/test_qtensor_cuda.py:416-440)."""
    bounds = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5])
    mask = torch.tensor([0, 1, 0, 1, 0, 1, 0])
    sign = (w < 0).to(torch.uint8)
    ordinal = torch.sum(w.abs().unsqueeze(-1) > bounds, dim=-1).to(torch.uint8)
    tie = torch.sum((w.abs().unsqueeze(-1) == bounds) * mask, dim=-1).to(torch.uint8)
    return (sign * 8 + ordinal + tie).to(torch.uint8)


@pytest.mark.parametrize("rows", VEC["cast_fp4_inputs"])
def test_cast_fp4_equals_brute_force_twin(rows):
    w = torch.tensor(rows, dtype=torch.float32)
    assert torch.equal(qtensor.cast_fp4(w.clone()), _twin_cast_fp4(w))


def test_cast_fp4_twin_on_dense_sweep():
    w = torch.linspace(-7, 7, 56001)
    ties = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0])
    w = torch.cat([w, ties, -ties, torch.nextafter(ties, torch.tensor(9.0)),
                   torch.nextafter(ties, torch.tensor(-9.0))])
    assert torch.equal(qtensor.cast_fp4(w.clone()), _twin_cast_fp4(w))


def test_cast_fp4_special_values():
    w = torch.tensor([float("nan"), float("inf"), -float("inf"), -0.0, 0.0, -1e-30])
    assert qtensor.cast_fp4(w).tolist() == [7, 7, 15, 0, 0, 8]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("values", VEC["nvfp4_quantize_inputs"])
def test_nvfp4_quantize_dequantize_close(values, dtype):
    x = torch.tensor(values).unsqueeze(0).to(dtype)
    packed, wsf, wsf2 = qtensor.nvfp4_quantize(x, 8)
    y = qtensor.nvfp4_dequantize(packed, wsf, wsf2, 8, x.shape, dtype)
    assert torch.allclose(y, x, rtol=2e-1, atol=2e-1)


def test_nvfp4_identity_on_e2m1_grid_and_nibble_order():
    """Values on the E2M1 grid with amax 6 quantise to themselves: scale 448, wsf2 = 6/2688,
    codes are the table indices, byte i = code[2i] | code[2i+1] << 4."""
    lut = [0, 0.5, 1, 1.5, 2, 3, 4, 6, 0, -0.5, -1, -1.5, -2, -3, -4, -6]
    x = torch.tensor(lut).unsqueeze(0).to(torch.bfloat16)
    packed, wsf, wsf2 = qtensor.nvfp4_quantize(x, 8)
    codes = list(range(16))
    codes[8] = 0  # -0 does not exist: the second zero encodes as +0
    want = [codes[2 * i] | (codes[2 * i + 1] << 4) for i in range(8)]
    assert packed.tolist() == [want]
    assert wsf.float().tolist() == [[448.0, 448.0]]
    assert wsf2.item() == pytest.approx(6.0 / 2688.0)
    y = qtensor.nvfp4_dequantize(packed, wsf, wsf2, 8, x.shape, torch.bfloat16)
    assert torch.equal(y, x)


@pytest.mark.parametrize("case", VEC["nvfp4_fake_quant_boundaries"])
@pytest.mark.parametrize("signs", [[1, 1, 1, 1, 1, 1, 1, 1], [-1, 1, -1, -1, 1, -1, 1, -1]])
def test_nvfp4_fake_quant_boundary_vectors(case, signs):
    sign = torch.tensor(signs, dtype=torch.float32)
    x = torch.tensor(case["base"], dtype=torch.float32)
    x[:-1] += case["delta"]
    x = torch.cat([x * sign] * 2).unsqueeze(0)
    want = torch.cat([torch.tensor(case["output"]) * sign] * 2).unsqueeze(0)
    # the QTensor route (exact ties) satisfies every row
    p, wsf, wsf2 = qtensor.nvfp4_quantize(x, 16)
    y = qtensor.nvfp4_dequantize(p, wsf, wsf2, 16, x.shape, torch.float32)
    assert torch.allclose(y, want)
    if case["ladder_checked"]:
        assert torch.allclose(fake_quant.nvfp4_fake_quant(x, x.abs().amax(), 16), want)


# ----------------------------------------------------------------------------- E4M3 bit-level twin
def _e4m3_rne_reference(v: torch.Tensor):
    """Software E4M3 rounding from the format definition (double arithmetic): quantum
    2^(max(e,-6)-3), ties to even, above 464 -> NaN."""
    a = v.abs().double()
    e = torch.floor(torch.log2(torch.clamp(a, min=2.0 ** -20))).clamp(min=-6)
    q = torch.pow(2.0, e - 3)
    r = torch.round(a / q) * q  # torch.round is half-to-even
    r = torch.where(a > 464.0, torch.full_like(r, float("nan")), r)
    return torch.copysign(r, v.double()).float()


def test_e4m3_cast_matches_format_definition_on_all_bf16_patterns():
    allv = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
    finite = allv[torch.isfinite(allv)]
    got = finite.to(torch.float8_e4m3fn).float()
    want = _e4m3_rne_reference(finite)
    both_nan = torch.isnan(got) & torch.isnan(want)
    assert bool(((got == want) | both_nan).all())


def test_fp8_eager_probes():
    x = torch.tensor([449.0, 464.0, 464.1, 2.0 ** -10, 2.0 ** -10 * 1.0001, -1e-9])
    y = fake_quant.fp8_eager(x, None)
    assert y[0] == 448 and y[1] == 448 and torch.isnan(y[2])
    assert y[3] == 0 and y[4] == 2.0 ** -9 and y[5] == 0 and torch.signbit(y[5])


# ----------------------------------------------------------------------------- reductions
@pytest.mark.parametrize("case", VEC["reduce_block_amax"])
def test_reduce_block_amax_golden(case):
    x = torch.tensor(case["input"], dtype=torch.bfloat16)
    got = reduce.reduce_block_amax(x, _bs(case["block_sizes"]))
    assert torch.equal(got, torch.tensor(case["output"], dtype=torch.bfloat16))


def test_max_calibrator_matches_reference_tests():
    g = torch.Generator().manual_seed(0)
    c = reduce.MaxCalibrator(8, None, False)
    a, b = torch.rand(16, generator=g), torch.rand(16, generator=g)
    c.collect(a); c.collect(b)
    assert torch.equal(c.compute_amax(), torch.max(a.max(), b.max()))
    for axis in (0, -4):
        c = reduce.MaxCalibrator(8, axis, False)
        a, b = torch.rand(3, 4, 2, 2, generator=g), torch.rand(3, 4, 2, 2, generator=g)
        c.collect(a); c.collect(b)
        assert c.compute_amax().shape[0] == 3
        assert torch.equal(c.compute_amax(), reduce.reduce_amax(torch.max(a, b), axis=(1, 2, 3)))
        c.reset()
        assert c.compute_amax() is None
    c = reduce.MaxCalibrator(8, 0, False)
    c.collect(torch.rand(3, 4, 2, 2))
    with pytest.raises(RuntimeError, match="shape changed"):
        c.collect(torch.rand(4, 4, 2, 2))


def test_quant_axis_to_reduce_dims():
    x = torch.zeros(2, 3, 4)
    assert reduce.quant_axis_to_reduce_dims(x, None) is None
    assert reduce.quant_axis_to_reduce_dims(x, 0) == [1, 2]
    assert reduce.quant_axis_to_reduce_dims(x, -1) == [0, 1]
    assert reduce.quant_axis_to_reduce_dims(x, (0, -1)) == [1]


# ----------------------------------------------------------------------------- integer QDQ
def _closed_form_int(x, amax, num_bits, narrow_range, unsigned=False):
    """tests/_test_utils/torch/quantization/quant_utils.py:19-30 restated (fake=True).  Its scale
    is ``float / tensor`` (torch computes that as reciprocal * float), one rounding away from
    the true division the quantizer uses, hence the 1e-6 tolerance below."""
    hi = 2.0 ** (num_bits - 1 + int(unsigned)) - 1.0
    lo = 0.0 if unsigned else (-hi if narrow_range else -hi - 1)
    scale = hi / amax
    return torch.clamp((x * scale).round_(), lo, hi) / scale


@pytest.mark.parametrize("num_bits", VEC["int_qdq_grid"]["num_bits"])
@pytest.mark.parametrize("unsigned", VEC["int_qdq_grid"]["unsigned"])
@pytest.mark.parametrize("narrow", [True, False])
def test_int_qdq_equals_closed_form(num_bits, unsigned, narrow):
    g = torch.Generator().manual_seed(num_bits)
    x = torch.randn(31, 47, generator=g)
    if unsigned:
        x = x.abs()
    hi = 2.0 ** (num_bits - 1 + int(unsigned)) - 1.0
    lo = 0.0 if unsigned else (-hi if narrow else -hi - 1)
    for amax in (x.abs().max(), x.abs().amax(dim=1, keepdim=True) * 0.7):  # per tensor / channel
        got = fake_quant.tensor_quant(x, amax, num_bits, unsigned, narrow)
        assert torch.allclose(got, _closed_form_int(x, amax, num_bits, narrow, unsigned),
                              rtol=1e-6, atol=0)
        # outputs sit on the integer grid, inside the range, within half a step of the input
        step = amax.double() / hi
        k = got.double() / step
        assert torch.allclose(k, k.round(), atol=1e-4)
        assert k.round().min() >= lo and k.round().max() <= hi
        inside = (x.double() / step > lo) & (x.double() / step < hi)
        assert ((got.double() - x.double()).abs()[inside] <= step.expand_as(x)[inside] * 0.5001).all()


def test_int_qdq_tiny_amax_gives_zero():
    c = VEC["int_tiny_amax"]
    x = torch.rand(*c["shape"])
    amax = torch.tensor(c["amax"]).unsqueeze(-1).unsqueeze(0)
    y = fake_quant.tensor_quant(x, amax, 8, False, True)
    assert y[:, 1, :].abs().sum() == 0


def test_int_qdq_errors():
    with pytest.raises(TypeError):
        fake_quant.tensor_quant(torch.tensor([-1.0, 1.0]), torch.tensor(1.0), 8, True, True)
    with pytest.raises(ValueError):
        fake_quant.tensor_quant(torch.tensor([1.0]), torch.tensor(-1.0), 8, False, True)


# ----------------------------------------------------------------------------- export
@pytest.mark.parametrize("case", VEC["scaling_factor_from_weight"])
def test_scaling_factor_from_weight_golden(case):
    w = torch.tensor(case["weight"])
    got = export.get_scaling_factor_from_weight(w, case["group_size"])
    want = torch.tensor(case["expected"])
    assert list(got.shape) == list(want.shape)
    assert torch.allclose(got, want, rtol=0.0, atol=0.0)


def test_pack_int4_brute_force_and_round_trip():
    """The byte layout against a pure-Python loop and the unpack(pack) invariant (the reference's
    own outputs pin it in test_export_casts_match_reference_outputs)."""
    g = torch.Generator().manual_seed(5)
    w = (torch.randn(6, 16, generator=g) * 0.3).to(torch.bfloat16)
    wsf = export.get_scaling_factor_from_weight(w, 8)
    packed = export.pack_int4_in_uint8(w, wsf)
    assert packed.shape == (3, 16) and packed.dtype == torch.uint8
    q = [[max(-8, min(7, round(float(w[n, k]) / float(wsf[n, k // 8])))) for k in range(16)]
         for n in range(6)]  # Python round() is half-to-even, like torch.round
    # recompute the quotient in fp32 exactly as torch does before trusting Python's double maths
    qt = (w.float() / wsf[:, torch.arange(16) // 8]).round().clamp(-8, 7).to(torch.int8)
    assert qt.tolist() == q
    for j in range(3):
        for k in range(16):
            assert int(packed[j, k]) == (q[2 * j][k] & 0xF) | ((q[2 * j + 1][k] & 0xF) << 4)
    assert torch.equal(export.unpack_int4_rows(packed), qt)


@pytest.mark.parametrize("case", load_export_vectors(), ids=lambda c: c["name"])
def test_export_casts_match_reference_outputs(case):
    """Outputs recorded from the reference's pack_int4_in_uint8 / to_quantized_weight
    (export/quant_utils.py:697-774) by tests/golden/make_export_vectors.py."""
    w, s, fmt = case["weight"], case["scale"], case["format"]
    if fmt in ("int4_awq", "w4a8_awq"):
        got = export.pack_int4_in_uint8(w, s)
    elif fmt == "fp8":
        got = export.fp8_export_cast(w, s.unsqueeze(-1) if w.dim() == 3 else s)
    elif fmt == "fp8_pc_pt":
        got = export.fp8_export_cast(w, s[:, None])
    else:
        got = export.int8_export_cast(w, s)
    assert_bits_equal(got, case["out"], case["name"])


def test_export_vectors_tell_nibble_orders_apart():
    """The fixture would fail a swapped nibble order and a pairing along K: both variants differ
    from the recorded bytes on the 2-D cases."""
    for case in load_export_vectors():
        if case["format"] not in ("int4_awq", "w4a8_awq") or case["weight"].dim() != 2:
            continue
        w, s = case["weight"], case["scale"]
        bs = w.shape[1] // s.shape[1]
        q = (w / s[:, torch.arange(w.shape[1]) // bs]).round().clamp(-8, 7).to(torch.int8)
        swapped = ((q[1::2] & 0xF) | ((q[0::2] & 0xF) << 4)).view(torch.uint8)
        assert not torch.equal(swapped, case["out"]), case["name"]
        along_k = ((q[:, 0::2] & 0xF) | ((q[:, 1::2] & 0xF) << 4)).view(torch.uint8)
        assert along_k.shape != case["out"].shape or not torch.equal(along_k, case["out"])


def test_fp8_export_cast_double_rounding_rule():
    """bf16 tensor / 0-dim fp32 tensor is a bf16 tensor in torch: the quotient is rounded to
    bf16 and then to E4M3."""
    g = torch.Generator().manual_seed(9)
    w = (0.02 * torch.randn(256, 256, generator=g)).to(torch.bfloat16)
    wsf = w.abs().max().float() / 448.0
    assert (w / wsf).dtype == torch.bfloat16
    assert (w / wsf.reshape(1)).dtype == torch.float32
    twice = (w.float() / wsf).to(torch.bfloat16).to(torch.float8_e4m3fn)
    assert_bits_equal(export.fp8_export_cast(w, wsf), twice, "0-dim scale")
    once = (w.float() / wsf).to(torch.float8_e4m3fn)
    assert_bits_equal(export.fp8_export_cast(w, wsf.reshape(1)), once, "1-elem scale")
    assert (twice.view(torch.uint8) != once.view(torch.uint8)).any()


# ----------------------------------------------------------------------------- NF4
def _nf4_roundtrip(x, block, sblock, bits, dtype=None):
    packed, scales = nf4.nf4_quantize(x, block, sblock)
    q, factor, zero = nf4.double_quantization(scales, sblock, bits)
    return nf4.nf4_dequantize(packed, q, factor, zero, block, x.shape, dtype or x.dtype)


@pytest.mark.parametrize("case", VEC["nf4_roundtrip"], ids=lambda c: c["name"])
def test_nf4_roundtrip_golden(case):
    x = torch.tensor(case["input"], dtype=torch.bfloat16)
    want = torch.tensor(case["output"], dtype=torch.bfloat16)
    got = _nf4_roundtrip(x, case["block_size"], case["scale_block_size"], case["scale_bits"])
    assert torch.allclose(got, want), (got, want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(256, 64), (256, 32)])
def test_nf4_roundtrip_close(dtype, shape):
    """tests/gpu/torch/quantization/test_qtensor_cuda.py:30-68: uniform [0, 1) input, block 64,
    scale block 256, round trip within rtol = atol = 0.1."""
    x = torch.rand(shape, generator=torch.Generator().manual_seed(0)).to(dtype)
    got = _nf4_roundtrip(x, 64, 256, 8)
    assert got.dtype == dtype and torch.allclose(got, x, rtol=1e-1, atol=1e-1)


def test_nf4_nearest_index_brute_force():
    """The table search against a per-element Python loop over the bf16 table (first minimum)."""
    lut = nf4.NF4_TABLE
    v = torch.linspace(-1, 1, 4001).to(torch.bfloat16)
    got = nf4.nearest_table_index(v, lut)
    for x, g in zip(v.tolist(), got.tolist()):
        diffs = [abs(float((torch.tensor(x, dtype=torch.bfloat16) - e))) for e in lut]
        assert g == diffs.index(min(diffs))
