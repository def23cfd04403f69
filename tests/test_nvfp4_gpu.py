"""GPU parity of the NVFP4 kernels (through the C ABI) against the CPU oracle."""

import pytest
import torch

from conftest import assert_bits_equal
from modelopt_amd import _hip
from oracle import fake_quant, qtensor, reduce

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _rand(shape, dtype, seed, scale=0.02):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(shape, generator=g)).to(dtype)


def _gpu_amax(xd):
    acc = torch.zeros(1, dtype=torch.float32, device=xd.device)
    _hip.absmax_into(xd, acc, 1, 1, xd.numel())
    return acc


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape,bs", [((64, 256), 16), ((33, 48), 16), ((7, 40), 16),
                                      ((5, 24), 8), ((16, 96), 32), ((3, 5, 64), 16),
                                      ((1024, 4096), 16)])
def test_quantize_pack_matches_oracle(dtype, shape, bs):
    x = _rand(shape, dtype, seed=hash((shape, bs)) % 1000)
    packed_o, wsf_o, wsf2_o = qtensor.nvfp4_quantize(x, bs)
    xd = x.to(DEV)
    amax = _gpu_amax(xd)
    assert_bits_equal(amax.cpu().reshape(()).to(dtype), reduce.reduce_amax(x), "amax")
    packed, wsf, wsf2 = _hip.nvfp4_quantize(xd, amax.reshape(()), bs)
    assert_bits_equal(wsf2.cpu(), wsf2_o, "wsf2")
    assert_bits_equal(wsf.cpu(), wsf_o, "wsf")
    assert_bits_equal(packed.cpu(), packed_o, "packed")
    # dequant round trip
    y = _hip.nvfp4_dequantize(packed, wsf, wsf2, bs, dtype)
    y_o = qtensor.nvfp4_dequantize(packed_o, wsf_o, wsf2_o, bs, packed_o.shape[:-1] + (packed_o.shape[-1] * 2,), dtype)
    assert_bits_equal(y.cpu(), y_o, "dequant")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("shape", [(64, 256), (33, 40), (512, 1024)])
def test_fake_quant_matches_oracle(dtype, mode, shape):
    x = _rand(shape, dtype, seed=7, scale=1.0)
    amax = reduce.reduce_amax(x)
    xd = x.to(DEV)
    y = _hip.nvfp4_qdq(xd, amax.to(DEV), 16, mode)
    if mode == 0:
        y_o = fake_quant.nvfp4_fake_quant(x, amax, 16)
    else:
        p, wsf, wsf2 = qtensor.nvfp4_quantize(x, 16)
        kp = p.shape[-1] * 2
        y_o = qtensor.nvfp4_dequantize(p, wsf, wsf2, 16, (shape[0], kp), dtype)[:, : shape[1]]
    assert_bits_equal(y.cpu(), y_o.contiguous(), f"qdq mode {mode}")
