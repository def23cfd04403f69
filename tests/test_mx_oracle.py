"""Pins the block floating point (MX) oracle: the reference's golden tables, and the torch and C
restatements against each other (they share no code: the C one walks the reference's tables, the
torch one uses library casts and bucketize)."""

import json
import os

import pytest
import torch

from conftest import GOLDEN
from oracle import cref, mx

with open(os.path.join(GOLDEN, "mx_vectors.json")) as f:
    CASES = json.load(f)["cases"]
FORMATS = ["E4M3", "E5M2", "INT8", "E0M3", "E1M2", "E3M0", "E2M1", "E3M2", "E2M3"]


def golden_inputs(case, block_size, dtype, seed=0):
    """Inputs and expected outputs as the reference test builds them: the table repeated to fill
    the block, random signs on both (tests/gpu/torch/quantization/
    test_quantize_mxformats_cuda.py:33-36,87-91)."""
    rep = max(block_size // case["unit"], 1)
    x = torch.tensor(case["input"], dtype=dtype).repeat(1, rep)
    want = torch.tensor(case["output"], dtype=dtype).repeat(1, rep)
    g = torch.Generator().manual_seed(seed)
    sign = (torch.randint(0, 2, x.shape, generator=g) * 2 - 1).to(dtype)
    return x * sign, want * sign


def golden_params():
    for case in CASES:
        dtypes = [torch.float32, torch.float16, torch.bfloat16] if case["test"] == "test_mxfp4" \
            else [torch.float32]
        for bs in case["block_sizes"]:
            for dt in dtypes:
                yield pytest.param(case, bs, dt, id=f"{case['format']}-bs{bs}-{str(dt)[6:]}")


@pytest.mark.parametrize("case,block_size,dtype", list(golden_params()))
@pytest.mark.parametrize("impl", ["torch", "c"])
def test_reference_golden_tables(case, block_size, dtype, impl):
    x, want = golden_inputs(case, block_size, dtype)
    fn = mx.block_fp_fake_quant if impl == "torch" else cref.block_fp_fake_quant
    got = fn(x, block_size, case["format"], "E8M0")
    assert torch.allclose(want, got, atol=max(case["atol"], 1e-8))


def _same(a, b):
    return torch.equal(a.float().nan_to_num(nan=12345.0), b.float().nan_to_num(nan=12345.0))


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_torch_and_c_restatements_agree(fmt, dtype):
    g = torch.Generator().manual_seed(31)
    x = (torch.randn(64, 80, generator=g) * torch.exp(3 * torch.randn(64, 1, generator=g))).to(dtype)
    x[0, :8] = 0
    x[1, 3] = float("inf")
    x[2, 5] = float("nan")
    for bs in (8, 16, 32):                      # 80 columns: the last block of 32 is padded
        assert _same(mx.block_fp_fake_quant(x, bs, fmt), cref.block_fp_fake_quant(x, bs, fmt)), bs
    amax = x[3:].abs().amax().float().reshape(1)
    rows = x[3:].abs().amax(dim=1).float()
    for g_amax in (None, amax, rows):           # minifloat block scale, alone and under a global amax
        a = mx.block_fp_fake_quant(x[3:], 16, fmt, "E4M3", g_amax)
        b = cref.block_fp_fake_quant(x[3:], 16, fmt, "E4M3", g_amax)
        assert _same(a, b)


@pytest.mark.parametrize("fmt", FORMATS)
def test_every_table_value_is_a_fixed_point_and_ties_follow_the_rule(fmt):
    """convert_to_types on the format's own values and on the midpoints between them."""
    lib = cref.load()
    code = cref.FORMATS.index(fmt)
    if fmt in mx._TABLES:
        values = torch.tensor(mx._TABLES[fmt])
    elif fmt == "INT8":
        values = torch.arange(0, 128, dtype=torch.float32)
    else:
        dt = torch.float8_e4m3fn if fmt == "E4M3" else torch.float8_e5m2
        values = torch.arange(0, 127 if fmt == "E4M3" else 124, dtype=torch.uint8).view(dt).float()
    assert torch.equal(mx.convert_to_types(values, fmt), values)
    assert torch.equal(mx.convert_to_types(-values, fmt), -values)
    mids = (values[:-1] + values[1:]) / 2
    got_t = mx.convert_to_types(mids, fmt)
    got_c = torch.tensor([lib.qr_convert_to_types(float(v), code) for v in mids])
    assert torch.equal(got_t, got_c)
    up = got_t == values[1:]
    assert bool((up | (got_t == values[:-1])).all())
    if fmt == "E3M0":
        assert bool(up.all())                                   # ties away from zero
    elif fmt != "INT8":
        assert torch.equal(up, torch.arange(len(mids)) % 2 == 1)  # to the even table index
    big = torch.tensor([1e30, float("inf")])
    assert torch.equal(mx.convert_to_types(big, fmt), torch.full((2,), mx.FORMAT_MAX[fmt]))
