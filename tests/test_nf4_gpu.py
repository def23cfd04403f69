"""NF4 kernels and ``NF4QTensor`` against the CPU restatement of the reference's CPU path (bit
exact for the table codes, the block scales and the dequantised values), plus the reference's
golden round trips through ``TensorQuantizer``."""

import json
import os

import pytest
import torch

from conftest import GOLDEN, assert_bits_equal
from modelopt_amd import _hip
from modelopt_amd.torch.quantization.config import QuantizerAttributeConfig
from modelopt_amd.torch.quantization.nn import TensorQuantizer
from modelopt_amd.torch.quantization.qtensor import NF4QTensor
from oracle import nf4

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.bfloat16, torch.float16, torch.float32]

with open(os.path.join(GOLDEN, "reference_vectors.json")) as f:
    VEC = json.load(f)


def _check_quantize(x, block):
    """kernel == restatement for codes and block scales of a flat tensor"""
    packed, scales = _hip.nf4_quantize(x.to(DEV).contiguous().view(-1), block)
    want_packed, want_scales = nf4.nf4_quantize(x, block, 1)
    assert torch.equal(packed.cpu(), want_packed), (
        (packed.cpu() != want_packed).nonzero()[:8].flatten().tolist())
    assert_bits_equal(scales.cpu(), want_scales)
    return packed, scales


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("block", [64, 8, 128, 512])
def test_quantize_random_matches_restatement(dtype, block):
    g = torch.Generator().manual_seed(block)
    x = (torch.randn(512, 1024, generator=g) * torch.exp(torch.randn(512, 1, generator=g))).to(dtype)
    _check_quantize(x, block)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,block", [(7, 2), (1000, 6), (4100, 64), (8 * 1024 * 4 + 64, 64), (130, 1024)])
def test_quantize_ragged_and_odd_blocks(dtype, n, block):
    """sizes that are not whole blocks (zero padding), block sizes outside the tile kernel's set"""
    g = torch.Generator().manual_seed(n)
    x = torch.randn(n, generator=g).to(dtype)
    _check_quantize(x, block)


def _all_values_in_unit_range(dtype):
    if dtype == torch.float32:
        return None
    bits = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.int16)
    v = bits.view(dtype)
    return v[v.float().abs() <= 1.0]          # drops NaN too


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_quantize_every_scaled_value(dtype):
    """Every 16-bit value of magnitude <= 1 as the scaled value v: each block holds a 1.0, so
    its abs-max is 1 and v = x.  Covers every tie between neighbouring table entries."""
    v = _all_values_in_unit_range(dtype)
    blocks = torch.ones(v.numel(), 8, dtype=dtype)
    blocks[:, 1] = v
    blocks[:, 5] = -v
    _check_quantize(blocks.flatten(), 8)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_quantize_every_scaled_value_on_the_table_path(dtype):
    """Inputs of 4 M elements and more take the table-lookup kernel (16-bit dtypes): every
    16-bit scaled value again, at block scales 2^-3 .. 2^4 (exact, so v stays the same value),
    plus random blocks, all-zero and NaN blocks."""
    v = _all_values_in_unit_range(dtype)
    blocks = torch.ones(v.numel(), 8, dtype=dtype)
    blocks[:, 1] = v
    blocks[:, 5] = -v
    parts = [blocks * (2.0 ** e) for e in range(-3, 5)]
    g = torch.Generator().manual_seed(17)
    rnd = (torch.randn(1 << 22, generator=g) * torch.exp(torch.randn(1 << 22, generator=g))).to(dtype)
    x = torch.cat([p.flatten() for p in parts] + [rnd])
    x = torch.cat([x, torch.zeros((-x.numel()) % (8192 * 8), dtype=dtype)])
    x[-40:] = float("nan")
    assert x.numel() >= 64 * 8 * 8192
    _check_quantize(x, 8)
    _check_quantize(x, 64)


@pytest.mark.parametrize("dtype", DTYPES)
def test_quantize_values_around_the_decision_points(dtype):
    """fp32 neighbours of every midpoint between table entries, at several block scales"""
    t = nf4.NF4_TABLE.float()
    mid = (t[:-1] + t[1:]) / 2
    near = [mid]
    for _ in range(6):
        near.append(torch.nextafter(near[-1], torch.tensor(2.0)))
    lo = mid
    for _ in range(6):
        lo = torch.nextafter(lo, torch.tensor(-2.0))
        near.append(lo)
    v = torch.cat(near + [t])
    for scale in (1.0, 3.0, 0.00731, 2.0 ** -70, 2.0 ** 100, 1e-41):
        s = torch.tensor(scale, dtype=torch.float32).to(dtype).float()
        if not torch.isfinite(s) or s == 0:
            continue
        blocks = torch.zeros(v.numel(), 8)
        blocks[:, 0] = s
        blocks[:, 3] = v * s
        _check_quantize(blocks.to(dtype).flatten(), 8)


@pytest.mark.parametrize("dtype", DTYPES)
def test_quantize_special_blocks(dtype):
    """all-zero block (0 / 0 -> NaN -> index 0), NaN and inf inside a block, -0.0"""
    x = torch.randn(16, 64, generator=torch.Generator().manual_seed(9))
    x[1] = 0
    x[2, 5] = float("nan")
    x[3, 7] = float("inf")
    x[4, 0] = float("-inf")
    x[5, 3] = -0.0
    x[6] = -0.0
    _check_quantize(x.to(dtype), 64)
    _check_quantize(x.to(dtype), 2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("block", [64, 2, 24])
def test_dequantize_every_code(dtype, block):
    g = torch.Generator().manual_seed(3)
    n_blocks = 4096
    packed = torch.randint(0, 256, (n_blocks * block // 2,), generator=g, dtype=torch.uint8)
    packed[:256] = torch.arange(256, dtype=torch.uint8)
    scales = (torch.randn(n_blocks, generator=g) * 3).to(dtype)
    scales[0] = 0
    scales[1] = float("inf")
    got = _hip.nf4_dequantize(packed.to(DEV), scales.to(DEV), block).cpu()
    hi = nf4.NF4_TABLE[(packed >> 4).long()].view(-1, block // 2) * scales.view(-1, 1)
    lo = nf4.NF4_TABLE[(packed & 15).long()].view(-1, block // 2) * scales.view(-1, 1)
    want = torch.stack([hi.flatten(), lo.flatten()], dim=-1).view(-1).to(dtype)
    assert_bits_equal(got, want)


def _nf4_quantizer(block, sblock, bits=8):
    cfg = QuantizerAttributeConfig(
        num_bits=4, block_sizes={-1: block, "scale_bits": bits, "scale_block_sizes": {-1: sblock}},
        fake_quant=False)
    return TensorQuantizer(cfg).to(DEV)


@pytest.mark.parametrize("case", VEC["nf4_roundtrip"], ids=lambda c: c["name"])
def test_golden_roundtrip_through_the_quantizer(case):
    """tests/gpu/torch/quantization/test_qtensor_cuda.py:111-131, 255-268"""
    q = _nf4_quantizer(case["block_size"], case["scale_block_size"], case["scale_bits"])
    x = torch.tensor(case["input"], dtype=torch.bfloat16, device=DEV)
    packed = q(x)
    assert isinstance(packed, NF4QTensor)
    out = q(packed)
    assert torch.allclose(out.cpu(), torch.tensor(case["output"], dtype=torch.bfloat16))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(256, 64), (256, 32)])
def test_quantizer_roundtrip_matches_restatement(dtype, shape):
    """tests/gpu/torch/quantization/test_qtensor_cuda.py:30-68: uniform input, block 64, scale
    block 256; here additionally equal to the restatement (the mean of the scales is a floating
    point sum, so the int8 scales are compared within one step and the output within 2 %)."""
    x = torch.rand(shape, generator=torch.Generator().manual_seed(1)).to(dtype)
    q = _nf4_quantizer(64, 256)
    packed = q(x.to(DEV))
    out = q(packed)
    assert out.dtype == dtype and out.shape == x.shape
    assert torch.allclose(out.cpu(), x, rtol=1e-1, atol=1e-1)
    assert packed._quantized_data.numel() * 2 == x.numel()

    w_packed, w_scales = nf4.nf4_quantize(x, 64, 256)
    w_q, w_factor, w_zero = nf4.double_quantization(w_scales, 256, 8)
    assert torch.equal(packed._quantized_data.cpu().view(-1), w_packed)
    assert q._scale.shape == w_q.shape and q._scale.dtype == torch.int8
    assert (q._scale.cpu().int() - w_q.int()).abs().max() <= 1
    assert torch.allclose(q._double_scale.cpu().float(), w_factor.float(), rtol=2e-2)
    assert torch.allclose(q._scale_zeros.cpu().float(), w_zero.float(), rtol=1e-2)
    want = nf4.nf4_dequantize(w_packed, w_q, w_factor, w_zero, 64, x.shape, dtype)
    assert torch.allclose(out.cpu().float(), want.float(), rtol=2e-2, atol=1e-3)


def test_several_scale_blocks():
    """More blocks than one scale block: each scale block is dequantised with its own factor."""
    x = torch.randn(64, 1024, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16)
    q = _nf4_quantizer(64, 256)
    packed = q(x.to(DEV))
    assert q._scale.shape == (4, 256) and q._double_scale.shape == (4,)
    out = q(packed).cpu()
    w_packed, w_scales = nf4.nf4_quantize(x, 64, 256)
    want = nf4.nf4_dequantize(w_packed, *nf4.double_quantization(w_scales, 256, 8), 64, x.shape,
                              torch.bfloat16)
    assert torch.equal(packed._quantized_data.cpu().view(-1), w_packed)
    assert torch.allclose(out.float(), want.float(), rtol=3e-2, atol=2e-2)
    err = (out.float() - x.float()).norm() / x.float().norm()
    assert err < 0.12


def test_full_size_weight_roundtrip_error():
    """14336 x 4096 bf16 (an 8B model's gate projection): the dequantised tensor is the nearest
    table value times the block scale, so the error per element is below half the widest table
    gap (0.3047 / 2 of the block abs-max) plus the bf16 roundings of the scaled value and of
    the product."""
    g = torch.Generator(device=DEV).manual_seed(5)
    x = (0.02 * torch.randn(14336, 4096, generator=g, device=DEV)).to(torch.bfloat16)
    packed, scales = _hip.nf4_quantize(x.view(-1), 64)
    y = _hip.nf4_dequantize(packed, scales, 64).view_as(x)
    bound = 0.16 * scales.float().view(-1, 1)
    err = (y.float() - x.float()).view(-1, 64).abs()
    assert bool((err <= bound + 1e-6).all())
    # the packed codes of a slab equal the restatement's
    rows = slice(5000, 5064)
    want, _ = nf4.nf4_quantize(x[rows].cpu(), 64, 1)
    assert torch.equal(packed.view(14336, -1)[rows].cpu().view(-1), want)
