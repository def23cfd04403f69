"""The one-launch abs-max -> quantize kernels (all workgroups resident, the tensor read once) against
the two-launch entry points and the CPU oracle, through the C ABI."""

import pytest
import torch

from conftest import assert_bits_equal
from modelopt_amd import _hip
from oracle import fake_quant, qtensor, reduce

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _exchange_words_are_clear():
    """Arrival count, running maximum and give-up flag are back to zero (the generation word keeps
    counting from call to call)."""
    ws = _hip.fused_scratch(DEV).cpu()
    return int(ws[0]) == 0 and int(ws[32]) == 0 and int(ws[_hip.FUSED_WS_FAIL_OFFSET // 4]) == 0


def _rand(shape, dtype=torch.bfloat16, seed=0, scale=0.02):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(shape, generator=g)).to(dtype)


@pytest.mark.parametrize("shape", [(256, 1024), (3, 16), (1000, 48), (4096, 4096), (1024, 4096), (5, 7, 64)])
def test_nvfp4_quantize_fused_equals_two_launches_and_oracle(shape):
    x = _rand(shape, seed=shape[0])
    xd = x.to(DEV)
    got = _hip.nvfp4_quantize_fused(xd)
    assert got is not None
    packed, wsf, wsf2, amax = got
    acc = torch.zeros(1, dtype=torch.float32, device=DEV)
    _hip.absmax_into(xd, acc, 1, 1, xd.numel())
    p2, w2, s2 = _hip.nvfp4_quantize(xd, acc.reshape(()), 16)
    assert torch.equal(packed, p2) and torch.equal(wsf.view(torch.uint8), w2.view(torch.uint8))
    assert float(wsf2) == float(s2) and float(amax) == float(acc)
    if x.numel() <= 1 << 22:
        po, wo, w2o = qtensor.nvfp4_quantize(x, 16)
        assert_bits_equal(packed.cpu(), po, "packed")
        assert_bits_equal(wsf.cpu(), wo, "block scales")
        assert_bits_equal(wsf2.cpu(), w2o, "global scale")
    assert not _hip.fused_gave_up(DEV)
    assert _exchange_words_are_clear()   # left clean for the next call


def test_nvfp4_quantize_fused_special_values_and_limits():
    x = _rand((64, 256), seed=3)
    x[0, :16] = 0
    x[1, 5] = float("inf")
    got = _hip.nvfp4_quantize_fused(x.to(DEV))
    po, wo, _ = qtensor.nvfp4_quantize(x, 16)
    assert_bits_equal(got[0].cpu(), po, "packed with inf")
    assert_bits_equal(got[1].cpu(), wo, "scales with inf")
    zero = torch.zeros(32, 64, dtype=torch.bfloat16)
    got = _hip.nvfp4_quantize_fused(zero.to(DEV))
    po, wo, _ = qtensor.nvfp4_quantize(zero, 16)
    assert_bits_equal(got[0].cpu(), po, "all-zero packed")
    assert_bits_equal(got[1].cpu(), wo, "all-zero scales")
    # not covered: fp16, K % 16, and a tensor beyond what the registers hold -> two-launch path
    assert _hip.nvfp4_quantize_fused(_rand((8, 64), torch.float16).to(DEV)) is None
    assert _hip.nvfp4_quantize_fused(_rand((8, 40)).to(DEV)) is None
    big = torch.zeros(14336 * 4, 4096, dtype=torch.bfloat16, device=DEV)   # 470 MB
    assert _hip.nvfp4_quantize_fused(big) is None
    assert _exchange_words_are_clear()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("n", [8, 1000, 4096 * 4096, 100003, 1 << 21])
def test_fused_amax_qdq_equals_two_launches_and_oracle(dtype, n):
    x = _rand((n,), dtype, seed=n % 97, scale=1.0)
    xd = x.to(DEV)
    acc = torch.zeros(1, dtype=torch.float32, device=DEV)
    _hip.absmax_into(xd, acc, 1, 1, n)
    for kind, kw in (("fp8", {}), ("int", {"num_bits": 8}), ("int", {"num_bits": 4, "narrow_range": True})):
        got = _hip.fused_amax_qdq(xd, kind, **kw)
        assert got is not None, (kind, n)
        y, amax = got
        assert float(amax) == float(acc)
        if kind == "fp8":
            want = _hip.fp8_qdq(xd, acc, 1, 1, n)
        else:
            want = _hip.int_qdq(xd, acc, 1, 1, n, kw["num_bits"], False, kw.get("narrow_range", False))
        assert torch.equal(y.view(torch.uint8), want.view(torch.uint8)), (kind, n)
        if n <= 1 << 21:
            a = reduce.reduce_amax(x)
            ref = fake_quant.fp8_eager(x, a) if kind == "fp8" else fake_quant.tensor_quant(
                x, a, kw["num_bits"], False, kw.get("narrow_range", False))
            assert_bits_equal(y.cpu(), ref, f"{kind} vs oracle")
    assert not _hip.fused_gave_up(DEV)


def test_dynamic_quantizer_takes_the_fused_path():
    """A TensorQuantizer without calibrated amax (dynamic per-tensor) gives the two-launch result."""
    from modelopt_amd.torch.quantization.config import QuantizerAttributeConfig
    from modelopt_amd.torch.quantization.nn import TensorQuantizer
    from modelopt_amd.torch.quantization.qtensor import NVFP4QTensor

    x = _rand((512, 768), seed=5, scale=1.0)
    for cfg, ref in ((QuantizerAttributeConfig(num_bits=(4, 3)), lambda a: fake_quant.fp8_eager(x, a)),
                     (QuantizerAttributeConfig(num_bits=8), lambda a: fake_quant.tensor_quant(x, a, 8, False, False))):
        q = TensorQuantizer(cfg).to(DEV)
        assert_bits_equal(q(x.to(DEV)).cpu(), ref(reduce.reduce_amax(x)), "dynamic per tensor")
        assert not hasattr(q, "_amax")
    qt, wsf, wsf2 = NVFP4QTensor.quantize(x.to(DEV), 16)
    po, wo, w2o = qtensor.nvfp4_quantize(x, 16)
    assert_bits_equal(qt._quantized_data.cpu(), po, "NVFP4QTensor.quantize (fused)")
    assert_bits_equal(wsf.cpu(), wo, "scales")
    assert_bits_equal(wsf2.cpu().reshape(()), w2o.reshape(()), "wsf2")


def test_a_wait_that_gives_up_ends_the_kernel_and_raises_the_flag():
    """With a spin limit of zero every workgroup that is not the last to arrive gives up at once:
    all wavefronts exit, nothing is written, the flag word of the workspace reports it, and the next
    call works once the workspace has been cleared."""
    x = _rand((4096, 2048), seed=7).to(DEV)
    got = _hip.nvfp4_quantize_fused(x, spin_limit=0)
    assert got is not None
    torch.cuda.synchronize()
    # the workgroups that gave up mark their blocks: NaN scale bytes (only the last one to arrive
    # can have written real scales)
    assert int((got[1].view(torch.uint8) == 0x7F).sum()) > 0
    y = torch.empty_like(x)
    assert _hip.fused_amax_qdq(x, "fp8", out=y, spin_limit=0) is not None
    torch.cuda.synchronize()
    assert int(torch.isnan(y).sum()) > 0
    # until the host clears the workspace every further call on it fails the same loud way: the
    # abandoned exchange may have left its count and maximum behind
    y2 = torch.zeros_like(x)
    assert _hip.fused_amax_qdq(x, "fp8", out=y2) is not None
    torch.cuda.synchronize()
    assert bool(torch.isnan(y2).all())
    assert _hip.fused_gave_up(DEV)                 # clears the workspace
    assert int(_hip.fused_scratch(DEV).abs().sum()) == 0
    packed, wsf, wsf2, _ = _hip.nvfp4_quantize_fused(x)
    acc = torch.zeros(1, dtype=torch.float32, device=DEV)
    _hip.absmax_into(x, acc, 1, 1, x.numel())
    p2, w2, _ = _hip.nvfp4_quantize(x, acc.reshape(()), 16)
    assert torch.equal(packed, p2) and torch.equal(wsf.view(torch.uint8), w2.view(torch.uint8))
    assert not _hip.fused_gave_up(DEV)
