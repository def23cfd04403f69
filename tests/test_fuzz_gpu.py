"""Seeded random cases -- shapes, magnitudes from 1e-9 to 1e5, heavy tails, zeros, a few special
values -- through the main kernels, each against the CPU oracle bit for bit.  Small tensors, many
of them: the fixed-shape tests cover the layouts, these cover the value space around them."""

import pytest
import torch

from conftest import assert_bits_equal
from modelopt_amd import _hip
from oracle import fake_quant, qtensor, reduce

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _case(seed, dtype, last_multiple=1):
    g = torch.Generator().manual_seed(seed)
    rows = int(torch.randint(1, 97, (1,), generator=g))
    k = int(torch.randint(1, 40, (1,), generator=g)) * last_multiple
    scale = 10.0 ** float(torch.empty(1).uniform_(-9, 5, generator=g))
    x = torch.randn(rows, k, generator=g)
    kind = seed % 5
    if kind == 1:    # heavy tail
        x = x * torch.exp(2.5 * torch.randn(rows, k, generator=g))
    elif kind == 2:  # sparse
        x = x * (torch.rand(rows, k, generator=g) < 0.15)
    elif kind == 3:  # a few huge outliers
        x.view(-1)[torch.randint(0, x.numel(), (3,), generator=g)] *= 1e4
    elif kind == 4:  # whole rows of zeros and negative zeros
        x[::3] = 0.0
        x[1::7] = -0.0
    return (x * scale).to(dtype)


@pytest.mark.parametrize("seed", range(40))
def test_nvfp4_quantize_pack_and_dequantize(seed):
    dtype = (torch.bfloat16, torch.float16, torch.float32)[seed % 3]
    x = _case(seed, dtype, 16)
    if dtype == torch.float16:
        x = x.clamp(-6e4, 6e4)
    po, wo, w2o = qtensor.nvfp4_quantize(x, 16)
    amax = reduce.reduce_amax(x).float()
    packed, wsf, wsf2 = _hip.nvfp4_quantize(x.to(DEV), amax.to(DEV), 16)
    assert_bits_equal(wsf2.cpu().reshape(()), w2o.reshape(()), f"global scale, seed {seed}")
    assert_bits_equal(wsf.cpu(), wo, f"block scales, seed {seed}")
    assert_bits_equal(packed.cpu(), po, f"codes, seed {seed}")
    y = _hip.nvfp4_dequantize(packed, wsf, wsf2, 16, dtype)
    assert_bits_equal(y.cpu(), qtensor.nvfp4_dequantize(po, wo, w2o, 16, x.shape, dtype), f"dequantised, seed {seed}")


@pytest.mark.parametrize("seed", range(40))
def test_fp8_and_int_fake_quant(seed, cpu_fp8_overflow):
    dtype = (torch.bfloat16, torch.float16, torch.float32)[seed % 3]
    x = _case(seed + 100, dtype, 8 if seed % 2 else 1)
    if dtype == torch.float16:
        x = x.clamp(-6e4, 6e4)
    xd = x.to(DEV)
    amax = reduce.reduce_amax(x)
    clip = amax * (0.5 if seed % 4 == 0 else 1.0)      # every fourth case clips
    got = _hip.fp8_qdq(xd, clip.to(DEV), 1, 1, x.numel()).cpu()
    assert_bits_equal(got, fake_quant.fp8_eager(x, clip), f"fp8 per tensor, seed {seed}")
    bits = (8, 4, 3, 5, 7, 11)[seed % 6]
    unsigned = seed % 7 == 3
    xi = x.abs() if unsigned else x
    got = _hip.int_qdq(xi.to(DEV), clip.to(DEV), 1, 1, x.numel(), bits, unsigned, seed % 2 == 0).cpu()
    assert_bits_equal(got, fake_quant.tensor_quant(xi, clip, bits, unsigned, seed % 2 == 0), f"int{bits}, seed {seed}")
    # per row
    a_row = reduce.reduce_amax(x, axis=[1], keepdims=True)
    got = _hip.int_qdq(xd, a_row.reshape(-1).to(DEV), 1, x.shape[0], x.shape[1], bits, False, False).cpu()
    assert_bits_equal(got, fake_quant.tensor_quant(x, a_row, bits, False, False), f"int{bits} per row, seed {seed}")
    got = _hip.fp8_qdq(xd, a_row.reshape(-1).to(DEV), 1, x.shape[0], x.shape[1]).cpu()
    assert_bits_equal(got, fake_quant.fp8_eager(x, a_row), f"fp8 per row, seed {seed}")


@pytest.mark.parametrize("seed", range(24))
def test_abs_max_reductions(seed):
    dtype = (torch.bfloat16, torch.float16, torch.float32)[seed % 3]
    x = _case(seed + 200, dtype)
    if dtype == torch.float16:
        x = x.clamp(-6e4, 6e4)
    xd = x.to(DEV)
    rows, k = x.shape
    for outer, axis, inner, want in ((1, 1, x.numel(), reduce.reduce_amax(x).reshape(1)),
                                     (1, rows, k, reduce.reduce_amax(x, axis=[1]).reshape(-1)),
                                     (rows, k, 1, reduce.reduce_amax(x, axis=[0]).reshape(-1))):
        acc = torch.zeros(axis, dtype=torch.float32, device=DEV)
        _hip.absmax_into(xd, acc, outer, axis, inner)
        assert_bits_equal(acc.cpu().to(dtype), want, f"abs-max [{outer}, {axis}, {inner}], seed {seed}")
