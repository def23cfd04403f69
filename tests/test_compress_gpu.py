"""``mtq.compress``: packed weights of a quantised model against the CPU restatements of the
reference's QTensor classes, and the dequantise-on-forward module."""

import copy

import pytest
import torch
import torch.nn.functional as F
from torch import nn

import modelopt_amd.torch.quantization as mtq
from conftest import assert_bits_equal
from modelopt_amd.torch.quantization.qtensor import (FP8QTensor, INT4QTensor, INT8QTensor,
                                                     NVFP4QTensor, QTensorWrapper)
from oracle import qtensor, reduce

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


class _MLP(nn.Module):
    def __init__(self, seed=0):
        super().__init__()
        g = torch.Generator().manual_seed(seed)
        self.fc1 = nn.Linear(256, 512, bias=False)
        self.fc2 = nn.Linear(512, 128, bias=True)
        self.fc1.weight.data = 0.05 * torch.randn(512, 256, generator=g)
        self.fc2.weight.data = 0.05 * torch.randn(128, 512, generator=g)
        self.to(torch.bfloat16)

    def forward(self, x):
        return self.fc2(F.gelu(self.fc1(x)))


def _batch(seed=1):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(32, 256, generator=g).to(torch.bfloat16)


def _expected(fmt, w):
    """(packed, dequantised) from the CPU restatement for the weight formats of the named configs."""
    if fmt == "nvfp4":
        wsf2 = reduce.reduce_amax(w).float() / 2688.0
        p, s, s2 = qtensor.nvfp4_quantize(w, 16, wsf2=wsf2)
        return p, qtensor.nvfp4_dequantize(p, s, s2, 16, w.shape, w.dtype)
    if fmt == "int4":
        p, s = qtensor.int4_quantize(w, 128)
        return p, qtensor.int4_dequantize(p, s, 128, w.shape, w.dtype)
    if fmt == "fp8":
        q, s = qtensor.fp8_quantize(w, scales=reduce.reduce_amax(w) / 448.0)
        return q, qtensor.fp8_dequantize(q, s, w.shape, w.dtype)
    q, s = qtensor.int8_quantize(w, axis=0)
    return q, qtensor.int8_dequantize(q, s, w.shape, w.dtype)


CASES = [("nvfp4", "NVFP4_DEFAULT_CFG", NVFP4QTensor, torch.uint8),
         ("int4", "INT4_BLOCKWISE_WEIGHT_ONLY_CFG", INT4QTensor, torch.uint8),
         ("fp8", "FP8_DEFAULT_CFG", FP8QTensor, torch.float8_e4m3fn),
         ("int8", "INT8_DEFAULT_CFG", INT8QTensor, torch.int8)]


@pytest.mark.parametrize("fmt,cfg_name,qcls,store_dtype", CASES, ids=[c[0] for c in CASES])
def test_compress_packs_weights_like_the_reference_qtensors(fmt, cfg_name, qcls, store_dtype):
    ref = _MLP()
    model = copy.deepcopy(ref).to(DEV)
    x = _batch().to(DEV)
    mtq.quantize(model, getattr(mtq, cfg_name), lambda m: m(x))
    with torch.no_grad():
        y_fake = model(x)
    assert not mtq.is_real_quantized(model)
    with pytest.warns(UserWarning, match="Real quantization"):
        mtq.compress(model)
    assert mtq.is_real_quantized(model)
    for name in ("fc1", "fc2"):
        lin, w = getattr(model, name), getattr(ref, name).weight.data
        assert isinstance(lin, mtq.nn.RealQuantLinear)
        assert isinstance(lin.weight, QTensorWrapper) and lin.weight.dtype == store_dtype
        assert lin.weight.metadata["qtensor_class"] is qcls
        assert tuple(lin.weight.metadata["shape"]) == tuple(w.shape)
        packed, deq = _expected(fmt, w)
        assert_bits_equal(lin.weight.data.cpu().reshape(packed.shape), packed, f"{name} packed")
        got = lin.weight_quantizer(lin.weight)
        assert_bits_equal(got.cpu(), deq, f"{name} dequantised")
    if fmt in ("nvfp4", "int4"):
        assert model.fc1.weight.numel() * model.fc1.weight.element_size() == 512 * 256 // 2
    with torch.no_grad():
        y_real = model(x)
        h = F.gelu(F.linear(model.fc1.input_quantizer(x), model.fc1.weight_quantizer(model.fc1.weight)))
        y_want = F.linear(model.fc2.input_quantizer(h), model.fc2.weight_quantizer(model.fc2.weight),
                          model.fc2.bias)
    assert torch.equal(y_real, y_want)
    # packing and fake quantisation round the scales differently (e.g. the INT4 QTensor keeps
    # ``7 / amax`` in bf16), so the two models agree only to a few per cent
    rel = (y_real.float() - y_fake.float()).norm() / y_fake.float().norm()
    assert float(rel) < 0.05


def test_compress_pattern_config_and_later_weight_assignment():
    model = _MLP().to(DEV)
    x = _batch().to(DEV)
    mtq.quantize(model, mtq.NVFP4_DEFAULT_CFG, lambda m: m(x))
    with pytest.warns(UserWarning):
        mtq.compress(model, {"*fc1*": False, "default": True})
    assert not isinstance(model.fc1.weight, QTensorWrapper) and model.fc1.weight.dtype == torch.bfloat16
    assert model.fc1.weight_quantizer.fake_quant
    assert isinstance(model.fc2.weight, QTensorWrapper)
    # a fresh high-precision weight is packed on assignment, with the calibrated global amax
    g = torch.Generator().manual_seed(9)
    w_new = (0.05 * torch.randn(128, 512, generator=g)).to(torch.bfloat16)
    amax = model.fc2.weight_quantizer.amax.cpu()
    model.fc2.weight = nn.Parameter(w_new.to(DEV))
    assert isinstance(model.fc2.weight, QTensorWrapper)
    p, s, s2 = qtensor.nvfp4_quantize(w_new, 16, wsf2=amax.float().reshape(()) / 2688.0)
    assert_bits_equal(model.fc2.weight.data.cpu(), p, "re-packed weight")
    assert_bits_equal(model.fc2.weight_quantizer(model.fc2.weight).cpu(),
                      qtensor.nvfp4_dequantize(p, s, s2, 16, w_new.shape, torch.bfloat16), "dequantised")
    model(x)


def test_compressed_state_dict_round_trip():
    x = _batch().to(DEV)
    a, b = _MLP(seed=0).to(DEV), _MLP(seed=5).to(DEV)
    for m in (a, b):
        mtq.quantize(m, mtq.INT4_BLOCKWISE_WEIGHT_ONLY_CFG, lambda mm: mm(x))
        with pytest.warns(UserWarning):
            mtq.compress(m)
    b.load_state_dict(a.state_dict())
    assert torch.equal(b.fc1.weight.data, a.fc1.weight.data)
    assert isinstance(b.fc1.weight, QTensorWrapper)
    with torch.no_grad():
        assert torch.equal(a(x), b(x))
