"""Cross-checks the two CPU restatements of the reference arithmetic: the torch one (library
float8 / rounding routines) and the bit-level C one (``oracle/c``).  They share no code, so a
dropped term, a wrong tie rule or a wrong threshold in either shows up here."""

import json
import os

import pytest
import torch

from conftest import GOLDEN, assert_bits_equal
from oracle import cref, export, fake_quant, qtensor, reduce

DTYPES = [torch.bfloat16, torch.float16, torch.float32]
with open(os.path.join(GOLDEN, "reference_vectors.json")) as f:
    VEC = json.load(f)


def _all_bf16_as_f32():
    return torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()


def _edge_f32():
    g = torch.Generator().manual_seed(21)
    rnd = torch.randint(-2**31, 2**31 - 1, (1 << 18,), generator=g, dtype=torch.int64).to(torch.int32)
    near = torch.tensor([464.0, 463.99997, 464.00003, 480.0, 448.0, 2.0**-9, 2.0**-10, 1.5 * 2.0**-10,
                         2.0**-6, 0.0, -0.0, float("inf"), float("-inf")])
    return torch.cat([_all_bf16_as_f32(), rnd.view(torch.float32), near, -near])


def test_e4m3_rounding_matches_torch_cast_on_every_bf16_pattern_and_random_fp32():
    x = _edge_f32()
    got = cref.real_quantize(x, 1.0, torch.float32, "e4m3")
    want = x.to(torch.float8_e4m3fn)
    assert_bits_equal(got, want, "e4m3")           # NaN bytes compare equal whatever their sign
    lib = cref.load()
    assert lib.qr_f32_to_e4m3(464.0) == 0x7E and lib.qr_f32_to_e4m3(464.0001) == 0x7F


def test_e4m3_decode_of_every_byte():
    lib = cref.load()
    b = torch.arange(256, dtype=torch.uint8)
    want = b.view(torch.float8_e4m3fn).float()
    got = torch.tensor([lib.qr_e4m3_to_f32(int(v)) for v in b])
    assert_bits_equal(got, want, "decode")


def test_e2m1_codes_match_searchsorted_cast_and_table():
    lib = cref.load()
    x = torch.cat([_all_bf16_as_f32()[::7],
                   torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0, 7.0, 0.0, -0.0,
                                 0.24999999, 0.25000003, 0.74999994, 0.7500001,
                                 float("inf"), float("nan")])])
    x = torch.cat([x, -x])
    want = qtensor.cast_fp4(x)
    got = torch.tensor([lib.qr_f32_to_e2m1(float(v)) for v in x], dtype=want.dtype)
    assert torch.equal(got, want)
    lut = VEC["nvfp4"]["e2m1_values"] if "e2m1_values" in VEC.get("nvfp4", {}) else \
        [0, 0.5, 1, 1.5, 2, 3, 4, 6, 0, -0.5, -1, -1.5, -2, -3, -4, -6]
    assert [lib.qr_e2m1_to_f32(c) for c in range(16)] == [float(v) for v in lut]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("block", [16, 32])
def test_nvfp4_quantize_and_dequantize_agree(dtype, block):
    g = torch.Generator().manual_seed(22)
    x = (torch.randn((96, 256), generator=g) * 0.03)
    x[0] = 0.0                       # zero blocks: scale byte of 1.0
    x[1] *= 1e-6                     # block scales in the E4M3 subnormal range
    x[2, :16] *= 300.0               # one dominant block
    x[3, 5] = -0.0
    x = x.to(dtype)
    p_c, w_c, w2_c = cref.nvfp4_quantize(x, block)
    p_t, w_t, w2_t = qtensor.nvfp4_quantize(x, block)
    assert float(w2_c) == float(w2_t)
    assert_bits_equal(w_c, w_t, "block scales")
    assert torch.equal(p_c, p_t)
    y_c = cref.nvfp4_dequantize(p_c, w_c, w2_c, block, dtype)
    y_t = qtensor.nvfp4_dequantize(p_t, w_t, w2_t, block, x.shape, dtype)
    assert_bits_equal(y_c, y_t, "dequantize")


def test_nvfp4_dequantize_every_code_and_scale_byte():
    codes = torch.arange(256, dtype=torch.uint8).repeat(8).reshape(-1, 8)
    scales = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).reshape(-1, 1)
    wsf2 = torch.tensor(0.37)
    for dtype in DTYPES:
        y_c = cref.nvfp4_dequantize(codes, scales, wsf2, 16, dtype)
        y_t = qtensor.nvfp4_dequantize(codes, scales, wsf2, 16, (256, 16), dtype)
        assert_bits_equal(y_c, y_t, str(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_fp8_and_int_fake_quant_agree(dtype):
    g = torch.Generator().manual_seed(23)
    x = (torch.randn(20000, generator=g) * 2).to(dtype)
    x[:4] = torch.tensor([0.0, -0.0, 1e-4, -1e-4]).to(dtype)
    amax = reduce.reduce_amax(x)
    assert float(amax) == cref.absmax(x)
    assert_bits_equal(cref.fp8_qdq(x, amax), fake_quant.fp8_eager(x, amax), "fp8 with amax")
    assert_bits_equal(cref.fp8_qdq(x), fake_quant.fp8_eager(x), "fp8 plain")
    for bits, unsigned, narrow in ((8, False, True), (8, False, False), (4, False, False), (8, True, True)):
        xi = x.abs() if unsigned else x         # the reference refuses negatives when unsigned
        got = cref.int_qdq(xi, amax, bits, unsigned, narrow)
        want = fake_quant.tensor_quant(xi, amax, bits, unsigned, narrow)
        want = want[0] if isinstance(want, tuple) else want
        assert_bits_equal(got, want.to(dtype), f"int{bits} u={unsigned} n={narrow}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_int4_compress_and_storage_casts_agree(dtype):
    g = torch.Generator().manual_seed(24)
    x = torch.randn((64, 256), generator=g).to(dtype)
    p_c, s_c = cref.int4_block_quantize(x, 128)
    p_t, s_t = qtensor.int4_quantize(x, 128)
    assert_bits_equal(s_c, s_t, "int4 scales")
    assert torch.equal(p_c, p_t.reshape(-1))
    scale = reduce.reduce_amax(x).float() / 448.0
    # 0-dim fp32 scale: torch keeps the tensor's dtype for the quotient
    assert_bits_equal(cref.real_quantize(x, scale, dtype, "e4m3"),
                      export.fp8_export_cast(x, scale), "fp8 cast, quotient in T")
    assert_bits_equal(cref.real_quantize(x, scale, torch.float32, "e4m3"),
                      export.fp8_export_cast(x, scale.reshape(1)), "fp8 cast, fp32 quotient")
    s8 = reduce.reduce_amax(x).float() / 127.0
    want = (x / s8.reshape(1)).round().clamp(-128, 127).to(torch.int8)
    assert torch.equal(cref.real_quantize(x, s8, torch.float32, "int8"), want)


@pytest.mark.parametrize("case", [c for c in VEC["qtensor_roundtrip"] if c["num_bits"] == 4],
                         ids=lambda c: c["name"])
def test_reference_int4_golden_vectors_through_c(case):
    """The reference's own INT4 round-trip vectors (tests/gpu/torch/quantization/
    test_qtensor_cuda.py:133-189) through the C quantiser and the torch dequantiser."""
    x = torch.tensor(case["input"], dtype=torch.bfloat16)
    want = torch.tensor(case["output"], dtype=torch.bfloat16)
    bs = case["block_sizes"]["-1"]
    if x.numel() % bs:
        pytest.skip("C restatement takes whole blocks only")
    packed, scales = cref.int4_block_quantize(x, bs)
    got = qtensor.int4_dequantize(packed.reshape(*x.shape[:-1], -1), scales, bs, x.shape, torch.bfloat16)
    assert torch.allclose(got, want)
