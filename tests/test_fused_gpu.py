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


def test_dynamic_quantizer_takes_the_fused_path_only_on_request():
    """A TensorQuantizer without calibrated amax (dynamic per-tensor) and NVFP4QTensor.quantize
    without scales take the two-launch path by default and the one-launch kernels once
    ``set_one_launch_dynamic_quant(True)`` allows them; the results are the same bits."""
    import modelopt_amd.torch.quantization as mtq
    from modelopt_amd.torch.quantization.config import QuantizerAttributeConfig
    from modelopt_amd.torch.quantization.nn import TensorQuantizer
    from modelopt_amd.torch.quantization.qtensor import NVFP4QTensor

    x = _rand((512, 768), seed=5, scale=1.0)
    assert not mtq.one_launch_dynamic_quant()
    for allowed in (False, True):
        previous = mtq.set_one_launch_dynamic_quant(allowed)
        try:
            with _hip.KernelTimer() as timer:
                for cfg, ref in ((QuantizerAttributeConfig(num_bits=(4, 3)), lambda a: fake_quant.fp8_eager(x, a)),
                                 (QuantizerAttributeConfig(num_bits=8), lambda a: fake_quant.tensor_quant(x, a, 8, False, False))):
                    q = TensorQuantizer(cfg).to(DEV)
                    assert_bits_equal(q(x.to(DEV)).cpu(), ref(reduce.reduce_amax(x)), "dynamic per tensor")
                    assert not hasattr(q, "_amax")
            # the two-launch path goes through the timed ``call``; the fused wrappers do not
            assert bool(timer.calls) == (not allowed), timer.calls
            qt, wsf, wsf2 = NVFP4QTensor.quantize(x.to(DEV), 16)
        finally:
            mtq.set_one_launch_dynamic_quant(previous)
        po, wo, w2o = qtensor.nvfp4_quantize(x, 16)
        assert_bits_equal(qt._quantized_data.cpu(), po, "NVFP4QTensor.quantize")
        assert_bits_equal(wsf.cpu(), wo, "scales")
        assert_bits_equal(wsf2.cpu().reshape(()), w2o.reshape(()), "wsf2")
    assert not _hip.fused_gave_up(DEV)


def test_a_wait_that_expires_falls_back_to_the_workgroup_s_own_abs_max():
    """With a spin limit of zero every workgroup that is not the last to arrive stops waiting at
    once (forced from the host: every wavefront still ends normally) and takes the abs-max of
    the whole tensor by itself: the outputs equal the two-launch path's bit for bit, the flag
    word reports the slow way, the exchange words are clean, and the next call needs no help
    from the host."""
    x = _rand((4096, 2048), seed=7).to(DEV)
    acc = torch.zeros(1, dtype=torch.float32, device=DEV)
    _hip.absmax_into(x, acc, 1, 1, x.numel())
    p2, w2, s2 = _hip.nvfp4_quantize(x, acc.reshape(()), 16)

    got = _hip.nvfp4_quantize_fused(x, spin_limit=0)
    assert got is not None
    packed, wsf, wsf2, amax = got
    assert torch.equal(packed, p2) and torch.equal(wsf.view(torch.uint8), w2.view(torch.uint8))
    assert float(wsf2) == float(s2) and float(amax) == float(acc)
    ws = _hip.fused_scratch(DEV).cpu()
    assert int(ws[0]) == 0 and int(ws[32]) == 0           # count and maximum are back to zero
    assert int(ws[_hip.FUSED_WS_FAIL_OFFSET // 4]) == 1   # ... and the slow way was noted

    # the flag is information only: the next call (normal limit) works without the host clearing
    # anything, and a forced one after it as well
    for kind, kw in (("fp8", {}), ("int", {"num_bits": 8})):
        for dtype in (torch.bfloat16, torch.float16, torch.float32):
            xd = _rand((1000003,), dtype, seed=11, scale=1.0).to(DEV)
            a = torch.zeros(1, dtype=torch.float32, device=DEV)
            _hip.absmax_into(xd, a, 1, 1, xd.numel())
            want = (_hip.fp8_qdq(xd, a, 1, 1, xd.numel()) if kind == "fp8"
                    else _hip.int_qdq(xd, a, 1, 1, xd.numel(), 8, False, False))
            for limit in (_hip.FUSED_SPIN_LIMIT, 0):
                y, amax = _hip.fused_amax_qdq(xd, kind, spin_limit=limit, **kw)
                assert float(amax) == float(a), (kind, dtype, limit)
                assert torch.equal(y.view(torch.uint8), want.view(torch.uint8)), (kind, dtype, limit)
    assert _hip.fused_gave_up(DEV)        # reports and clears the flag
    assert not _hip.fused_gave_up(DEV)
    assert _exchange_words_are_clear()


def test_fused_fake_quant_refuses_to_work_in_place():
    """A workgroup whose wait expired reads x again while others write y: y must not overlap x."""
    x = _rand((1 << 16,), seed=2).to(DEV)
    assert _hip.fused_amax_qdq(x, "fp8", out=x) is None
    both = torch.empty(3 << 15, dtype=torch.bfloat16, device=DEV)
    assert _hip.fused_amax_qdq(both[:1 << 16], "fp8", out=both[1 << 15:]) is None   # half overlapped
    assert _hip.fused_amax_qdq(x, "int", out=torch.empty_like(x)) is not None
