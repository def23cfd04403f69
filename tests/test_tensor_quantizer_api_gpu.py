"""``TensorQuantizer`` / ``SequentialQuantizer`` behaviours the reference's tester classes pin
(tests/_test_utils/torch/quantization/tensor_quantizer_common.py:28-513), on the GPU.  Expected
values come from the closed form ``round(x * bound / amax).clamp(...) * amax / bound`` in
float64, not from this package's own functional ops."""

import pytest
import torch
import torch.nn.functional as F

from modelopt_amd.torch.quantization.config import QuantizerAttributeConfig
from modelopt_amd.torch.quantization.model_calib import max_calibrate
from modelopt_amd.torch.quantization.nn import QuantLinear, SequentialQuantizer, TensorQuantizer
from modelopt_amd.torch.quantization import tensor_quant

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
Cfg = QuantizerAttributeConfig


def _ref(x, amax, bits=8, narrow=False):
    """closed-form integer fake quantisation in float64 (tests/_test_utils/.../quant_utils.py:19-30)"""
    bound = 2.0 ** (bits - 1) - 1
    lo = -bound if narrow else -bound - 1
    scale = bound / amax.double()
    return (torch.clamp((x.double() * scale).round(), lo, bound) / scale).float()


def _randn(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)).to(DEV)


# ------------------------------------------------------------------ TensorQuantizerTester
def test_default_quantizer_is_int8_per_tensor_fake_quant():
    """:31-47"""
    x = _randn(3, 7)
    q = TensorQuantizer().to(DEV)
    assert torch.allclose(q(x), tensor_quant.fake_tensor_quant(x, x.abs().max(), None))
    x = _randn(31, seed=1)
    assert torch.allclose(TensorQuantizer(Cfg(num_bits=8)).to(DEV)(x), _ref(x, x.abs().max()))


def test_per_channel_scale_disable_and_backward():
    """:49-68, :307-310"""
    x = _randn(5, 5, 4, 8)
    amax = x.abs().amax(dim=(1, 2, 3), keepdim=True)
    q = TensorQuantizer(Cfg(num_bits=8, axis=0)).to(DEV)
    assert torch.allclose(q(x), _ref(x, amax), rtol=1e-2)
    x = _randn(3, 7)
    assert torch.equal(TensorQuantizer(Cfg(enable=False)).to(DEV)(x), x)
    x = _randn(3, 7).requires_grad_()
    TensorQuantizer().to(DEV)(x).sum().backward()
    assert x.grad is not None


def test_state_loading_properties_and_setters():
    """:70-96, :178-184, :203-210"""
    amax = [3.14, 2.718]
    q = TensorQuantizer(Cfg(num_bits=(4, 3)), amax=amax).to(DEV)
    q.load_state_dict(q.state_dict())
    assert torch.allclose(q.amax, torch.tensor(amax, device=DEV))
    q = TensorQuantizer(Cfg(), amax=3.14).to(DEV)
    q.amax = 0.577
    assert q.amax == torch.tensor(0.577, device=DEV)
    assert float(q.step_size) == pytest.approx(0.577 / 127.0, rel=1e-6)
    q2 = TensorQuantizer(Cfg()).to(DEV)
    a = torch.tensor([3.142, 2.718], device=DEV)
    q2.amax = a
    assert torch.allclose(q2.amax, a)
    assert TensorQuantizer(Cfg()).amax is None
    q = TensorQuantizer()
    q.num_bits, q.unsigned = 7, True
    assert q.num_bits == 7 and q.unsigned
    q = TensorQuantizer()
    q.set_from_attribute_config({"num_bits": 4})
    q.set_from_attribute_config({"axis": -1})
    q.set_from_attribute_config({"enable": False})
    assert q.num_bits == 4 and q.axis == -1 and q._disabled


def test_calibration_through_the_quantizer():
    """:98-146"""
    q = TensorQuantizer(Cfg(axis=(0, 1)), if_calib=True, if_quant=False).to(DEV)
    q(torch.rand(7, 6, 7, 7, device=DEV))
    q.load_calib_amax()
    assert q.amax.numel() == 7 * 6
    q = TensorQuantizer(Cfg(axis=0)).to(DEV)
    q.enable_calib()
    with pytest.raises(RuntimeError, match="Calibrator returned None"):
        q.load_calib_amax()
    x1, x2 = torch.rand(7, 6, 7, 7, device=DEV), torch.rand(7, 6, 7, 7, device=DEV)
    q(x1)
    q(x2)
    q.disable_calib()
    want = torch.max(x1.abs().amax(dim=(1, 2, 3), keepdim=True), x2.abs().amax(dim=(1, 2, 3), keepdim=True))
    assert torch.equal(q._calibrator.compute_amax(), want)
    q.load_calib_amax()
    assert torch.equal(q.amax, want)


def test_pre_quant_scale():
    """:186-201"""
    cfg = Cfg(axis=1, num_bits=8)
    q, q2 = TensorQuantizer(cfg, amax=127.0).to(DEV), TensorQuantizer(cfg, amax=127.0).to(DEV)
    x = torch.tensor([[0, 0.4, 1.1, 2.0]], device=DEV)
    assert torch.allclose(q(x), torch.tensor([[0.0, 0, 1, 2]], device=DEV))
    q.pre_quant_scale = 2.0
    assert torch.allclose(q(x), torch.tensor([[0.0, 1, 2, 4]], device=DEV))
    q2.pre_quant_scale = torch.tensor([[1.0, 2.0, 3.0, 4.0]], device=DEV)
    assert torch.allclose(q2(x), torch.tensor([[0.0, 1, 3, 8]], device=DEV))


def test_modelopt_state_round_trip():
    """:212-234, :286-305"""
    ref = TensorQuantizer(Cfg(num_bits=4), amax=10.0).to(DEV)
    state = ref.get_modelopt_state()
    for k in ref._get_properties_for_modelopt_state():
        assert k in state and state[k] == getattr(ref, k)
    assert "_amax" not in state and "_amax" in state["_pytorch_state_metadata"]["buffers"]
    test = TensorQuantizer(Cfg())
    test.set_from_modelopt_state(state)
    test.load_state_dict(ref.state_dict())
    test.to(DEV)
    x = _randn(10, 10)
    assert torch.equal(ref(x), test(x))
    ref = TensorQuantizer(Cfg(num_bits=4, axis=0)).to(DEV)
    ref.enable_calib()
    ref(_randn(4, 6, 8, seed=1))
    ref(_randn(4, 6, 8, seed=2))
    ref.load_calib_amax()
    ref.disable_calib()
    test = TensorQuantizer(Cfg())
    test.set_from_modelopt_state(ref.get_modelopt_state())
    test.load_state_dict(ref.state_dict())
    test.to(DEV)
    x = _randn(4, 6, 8, seed=3)
    assert torch.equal(ref(x), test(x))


def test_amax_export_shapes():
    """:236-284"""
    a = _randn(4, 6, 8)
    for block, last in ((4, 2), (8, 1)):
        q = TensorQuantizer(Cfg(num_bits=4, block_sizes={-1: block})).to(DEV)
        assert not hasattr(q, "_amax_shape_for_export")
        q(a)
        q.enable_calib()
        q(a)
        q.load_calib_amax()
        amax = q.export_amax()
        assert q._amax_shape_for_export == (4, 6, -1) and amax.shape == (4, 6, last)
    q = TensorQuantizer(Cfg(num_bits=4, axis=0)).to(DEV)
    q.enable_calib()
    q(a)
    q.load_calib_amax()
    assert not hasattr(q, "_amax_shape_for_export") and q.export_amax().shape == (4,)
    q = TensorQuantizer(Cfg(num_bits=4)).to(DEV)
    q.enable_calib()
    q(a)
    q.load_calib_amax()
    assert q.export_amax().shape == (1,)


def test_block_sizes_naming_whole_axes():
    """:312-343"""
    w, x = _randn(3, 3), _randn(1, 2, 3, seed=1)
    assert torch.equal(TensorQuantizer(Cfg(num_bits=8, block_sizes={1: None})).to(DEV)(w),
                       TensorQuantizer(Cfg(num_bits=8, axis=0)).to(DEV)(w))
    assert torch.equal(TensorQuantizer(Cfg(num_bits=8, block_sizes={0: None, 1: None})).to(DEV)(x),
                       TensorQuantizer(Cfg(num_bits=8, axis=-1)).to(DEV)(x))


# ------------------------------------------------------------------ BlockQuantTester
def test_block_quantization_simple_and_complex():
    """:349-394"""
    a = _randn(8, 4)
    amax = a.view(-1, 2).abs().amax(dim=-1, keepdim=True)
    want = _ref(a.view(-1, 2), amax).view_as(a)
    for blocks in ({-1: 2}, {1: 2}):
        q = TensorQuantizer(Cfg(num_bits=8, block_sizes=blocks)).to(DEV)
        q.enable_calib()
        got = q(a)
        q.load_calib_amax()
        assert torch.allclose(q.amax, amax) and torch.allclose(got, want)
    a = _randn(2, 6, 4, seed=1)
    amax = a.reshape(2, 2, 3, 2, 2).abs().amax(dim=(2, 4), keepdim=True)
    want = _ref(a.reshape(2, 2, 3, 2, 2), amax).view_as(a)
    for blocks in ({-1: 2, 1: 3}, {1: 3, 2: 2}):
        assert torch.allclose(TensorQuantizer(Cfg(num_bits=8, block_sizes=blocks)).to(DEV)(a), want)


def test_block_quantization_with_padding():
    """:396-448"""
    a = _randn(3, 4, 5)
    padded = F.pad(a, (0, 1))
    amax = padded.view(-1, 2).abs().amax(dim=-1, keepdim=True)
    want = _ref(padded.view(-1, 2), amax).view_as(padded)[:, :, :5]
    for blocks in ({-1: 2}, {2: 2}):
        q = TensorQuantizer(Cfg(num_bits=8, block_sizes=blocks)).to(DEV)
        q.enable_calib()
        got = q(a)
        q.load_calib_amax()
        assert torch.allclose(q.amax, amax) and torch.allclose(got, want)
    a = _randn(2, 10, 5, seed=1)
    padded = F.pad(a, (0, 1, 0, 2))
    amax = padded.view(2, 4, 3, 3, 2).abs().amax(dim=(2, 4), keepdim=True)
    want = _ref(padded.view(2, 4, 3, 3, 2), amax).view_as(padded)[:, :10, :5]
    q = TensorQuantizer(Cfg(num_bits=8, block_sizes={-1: 2, 1: 3})).to(DEV)
    q.enable_calib()
    got = q(a)
    q.load_calib_amax()
    assert torch.allclose(amax, q.amax) and torch.allclose(got, want)
    assert torch.allclose(TensorQuantizer(Cfg(num_bits=8, block_sizes={1: 3, 2: 2})).to(DEV)(a), want)


# ------------------------------------------------------------------ SequentialQuantizerTester
def test_sequential_quantizer_chains_its_members():
    """:454-476"""
    cfgs = [{"num_bits": 4}, {"block_sizes": {-1: 4}}, {"enable": False}]
    nq = SequentialQuantizer(*(TensorQuantizer(Cfg()) for _ in cfgs)).to(DEV)
    singles = [TensorQuantizer().to(DEV) for _ in cfgs]
    for member, single, c in zip(nq, singles, cfgs):
        member.set_from_attribute_config(c)
        single.set_from_attribute_config(c)
    x = _randn(2, 16)
    want = x
    for single in singles:
        want = single(want)
    assert torch.equal(nq(x), want)


def test_sequential_quantizer_replacement_and_delegation():
    """:478-513"""
    model = torch.nn.Module()
    model.model = torch.nn.Sequential(QuantLinear(4, 4), torch.nn.ReLU())
    seq = SequentialQuantizer(TensorQuantizer(Cfg()), TensorQuantizer(Cfg()))
    model.model[0].weight_quantizer = seq
    with SequentialQuantizer.convert_to_single_quantizer(model):
        assert not any(isinstance(m, SequentialQuantizer) for m in model.model.modules())
    assert model.model[0].weight_quantizer is seq
    assert not hasattr(model.model[0], "_original_weight_quantizer")
    sq = SequentialQuantizer(TensorQuantizer(Cfg()), TensorQuantizer(Cfg())).to(DEV)
    sq.disable()
    assert sq[0].is_enabled is False and sq[1].is_enabled is False
    sq.enable()
    assert sq[0].is_enabled is True and sq[1].is_enabled is True
    max_calibrate(sq, lambda q: q(torch.randn(1, 4, device=DEV)))
    assert sq[0].amax is not None
    sq.reset_amax()
    assert sq[0].amax is None and sq[1].amax is None
    assert sq.fake_quant is True
    sq[0]._fake_quant = False
    assert sq.fake_quant is False and sq[1]._fake_quant is True


# ------------------------------------------------------------------ fake_tensor_quant (function)
def test_fake_tensor_quant_function_contract():
    """tests/_test_utils/torch/quantization/tensor_quant_common.py:31-135: positional
    ``(x, amax, bias, num_bits, unsigned, narrow_range)``; doubles are accepted and computed in
    fp32; an amax far below the data does not overflow fp16; the unsigned 8-bit grid is the
    signed 9-bit one; ``narrow_range=False`` opens the lowest code."""
    f = tensor_quant.fake_tensor_quant
    x64 = _randn(2, 3).double() * 100
    got = f(x64, x64.abs().max(), None, 7)
    assert got.dtype == torch.float64
    assert torch.equal(got, f(x64.float(), x64.abs().max().float(), None, 7).double())
    torch.manual_seed(123)
    x = torch.randn(3, 3, 6, 8).to(DEV)
    amax = 0.7 * x.abs().amax(dim=(1, 2, 3), keepdim=True)          # clips
    assert torch.allclose(f(x, amax), _ref(x, amax, narrow=True))
    x = _randn(31).abs()
    assert torch.allclose(f(x, x.max(), None, 8, True), _ref(x, x.max(), bits=9, narrow=True))
    assert torch.allclose(f(x, x.max(), None, 8, True, False), _ref(x, x.max(), bits=9))
    half = f(_randn(31).half(), torch.tensor(1e-4, device=DEV).half(), None, 8, False)
    assert torch.isfinite(half).all()


def test_fake_tensor_quant_gradients():
    """:66-118: the gradient passes straight through inside ``[-amax, amax]`` and is zero outside"""
    f = tensor_quant.fake_tensor_quant
    x = _randn(3, 7).requires_grad_()
    labels = torch.tensor([1, 4, 2], device=DEV)
    y = f(x, x.abs().max().detach(), None, 7)
    y.retain_grad()
    torch.nn.CrossEntropyLoss()(y, labels).backward()
    assert torch.allclose(y.grad, x.grad)
    x = _randn(3, 7, seed=1).requires_grad_()
    amax = (x.abs().max() / 2).detach()
    ((f(x, amax, None, 8) - 0.5) ** 2).sum().backward()
    assert torch.equal(x.grad != 0, (x >= -amax) & (x <= amax))


# ------------------------------------------------------------------ QuantLinear built directly
def _linear(*args, **kwargs):
    return QuantLinear(*args, **kwargs).to(DEV)


def test_quant_linear_constructed_directly():
    """tests/unit/torch/quantization/test_quant_linear.py:33-170: ``QuantLinear(in, out, ...)``
    equals ``F.linear`` over separately fake-quantised operands, bit for bit."""
    f = tensor_quant.fake_tensor_quant
    m = _linear(2, 2, bias=False, quant_desc_weight=Cfg(axis=None))
    m.input_quantizer.disable()
    x, w = _randn(2, 2), m.weight.detach().clone()
    assert torch.equal(m(x), F.linear(x, f(w, w.abs().max())))

    m = _linear(3, 5, bias=False, quant_desc_weight=tensor_quant.QUANT_DESC_8BIT_LINEAR_WEIGHT_PER_ROW)
    m.input_quantizer.disable()
    x, w = _randn(32, 3), m.weight.detach().clone()
    assert torch.equal(m(x), F.linear(x, f(w, w.abs().amax(dim=1, keepdim=True))))

    m = _linear(3, 5, bias=False)
    m.weight_quantizer.disable()
    assert torch.equal(m(x), F.linear(f(x, x.abs().max()), m.weight))

    m = _linear(3, 5, bias=True, quant_desc_weight=Cfg())
    x, w = _randn(4, 17, 9, 3), m.weight.detach().clone()            # more than two dimensions
    assert torch.equal(m(x), F.linear(f(x, x.abs().max()), f(w, w.abs().max()), m.bias))

    qi, qw = Cfg(num_bits=4), Cfg(num_bits=3)
    m = _linear(3, 5, bias=False, quant_desc_input=qi, quant_desc_weight=qw)
    x = _randn(2, 3)
    want = F.linear(TensorQuantizer(qi).to(DEV)(x), TensorQuantizer(qw).to(DEV)(m.weight.detach().clone()))
    assert torch.equal(m(x), want)


def test_quant_linear_state_dict_and_class_defaults():
    """test_quant_linear.py:172-220"""
    from modelopt_amd.torch.quantization.nn.modules import quant_linear

    m = _linear(3, 5, bias=True, quant_desc_input=Cfg(num_bits=16), quant_desc_weight=Cfg(num_bits=16, axis=0))
    plain = torch.nn.Linear(3, 5).to(DEV)
    plain.load_state_dict(m.state_dict())
    m.input_quantizer.disable()
    m.weight_quantizer.disable()
    x = _randn(2, 3)
    assert torch.allclose(m(x), plain(x))

    m = QuantLinear(4, 16)
    assert m.input_quantizer.axis is None and m.weight_quantizer.axis == 0
    saved = (quant_linear.Linear.default_quant_desc_input, quant_linear.Linear.default_quant_desc_weight)
    try:
        quant_linear.Linear.default_quant_desc_input = Cfg(num_bits=11)
        quant_linear.Linear.default_quant_desc_weight = Cfg(num_bits=13, axis=1)
        m = QuantLinear(4, 16)
        assert m.input_quantizer.num_bits == 11 and m.weight_quantizer.axis == 1
    finally:
        quant_linear.Linear.default_quant_desc_input, quant_linear.Linear.default_quant_desc_weight = saved


def test_set_quantizer_by_cfg_context_restores_everything():
    """tests/unit/torch/quantization/test_tensor_quant_cpu.py:103-135 on a W4 (block 128) + INT8
    sequential weight quantizer calibrated with the full AWQ search."""
    import modelopt_amd.torch.quantization as mtq

    cfg = {"quant_cfg": {"*weight_quantizer": [{"num_bits": 4, "block_sizes": {-1: 128, "type": "static"},
                                                "enable": True},
                                               {"num_bits": 8, "axis": 0, "enable": True}],
                         "*input_quantizer": {"num_bits": 8, "enable": True},
                         "default": {"enable": False}},
           "algorithm": "awq_full"}
    torch.manual_seed(0)
    model = torch.nn.Sequential(torch.nn.Linear(16, 32), torch.nn.ReLU(), torch.nn.Linear(32, 64),
                                torch.nn.ReLU(), torch.nn.Linear(64, 16)).to(DEV).eval()
    inputs = _randn(2, 16)
    mtq.quantize(model, cfg, lambda m: m(inputs))
    before = {k: v.clone() for k, v in model.state_dict().items()}
    want = model(inputs)
    mtq.set_quantizer_by_cfg(model, {"*output_quantizer": {"enable": True}})
    with mtq.set_quantizer_by_cfg_context(model, {"*": {"enable": False}, "*output_quantizer": {"enable": True}}):
        for name, mod in model.named_modules():
            if isinstance(mod, TensorQuantizer):
                assert mod.is_enabled == name.endswith("output_quantizer"), name
        mtq.calibrate(model, "max", lambda m: m(inputs * 10))
    mtq.set_quantizer_by_cfg(model, {"*output_quantizer": {"enable": False}})
    assert torch.equal(model(inputs), want)
    for k, v in model.state_dict().items():
        if "output_quantizer" not in k:
            assert torch.equal(v, before[k]), k


class _SdpaAttention(torch.nn.Module):
    def forward(self, q, k, v):
        return F.scaled_dot_product_attention(q, k, v)


def test_kv_cache_config_on_a_registered_attention():
    """``register_attention_for_kv_quant`` + ``FP8_KV_CFG`` (reference: plugins/attention.py:45-216,
    config.py FP8_KV_CFG): keys and values go through per-tensor FP8 fake quantisation with the
    calibrated amax, the query stays as it is."""
    import modelopt_amd.torch.quantization as mtq

    assert mtq.plugins.register_attention_for_kv_quant(_SdpaAttention)
    try:
        model = torch.nn.Sequential()
        model.add_module("attn", _SdpaAttention())
        q, k, v = _randn(2, 4, 16, 32), _randn(2, 4, 16, 32, seed=1) * 3, _randn(2, 4, 16, 32, seed=2) * 0.2
        mtq.quantize(model, mtq.FP8_KV_CFG, lambda m: m.attn(q, k, v))
        attn = model.attn
        assert not attn.q_bmm_quantizer.is_enabled
        assert torch.equal(attn.k_bmm_quantizer.amax, k.abs().max())
        assert torch.equal(attn.v_bmm_quantizer.amax, v.abs().max())
        fq = lambda t: tensor_quant.scaled_e4m3(t, t.abs().max(), None, 4, 3)
        assert torch.equal(attn(q, k, v), F.scaled_dot_product_attention(q, fq(k), fq(v)))
        assert not torch.equal(attn(q, k, v), F.scaled_dot_product_attention(q, k, v))
    finally:
        mtq.unregister(_SdpaAttention)


# ------------------------------------------------------------------ calibrators used on their own
def test_max_calibrator_standalone():
    """tests/unit/torch/quantization/test_calibrator.py:28-91"""
    import numpy as np

    from modelopt_amd.torch.quantization import calib

    a, b = torch.rand(16, device=DEV), torch.rand(16, device=DEV)
    c = calib.MaxCalibrator(8, None, False, track_amax=True)
    c.collect(a)
    c.collect(b)
    assert torch.equal(c.compute_amax(), torch.max(a.max(), b.max()))
    np.testing.assert_array_equal(c.amaxs[0], a.max().cpu().numpy())
    np.testing.assert_array_equal(c.amaxs[1], b.max().cpu().numpy())
    c.reset()
    assert c.compute_amax() is None
    for axis in (0, -4):
        c = calib.MaxCalibrator(8, axis, False)
        a, b = torch.rand(3, 4, 2, 2, device=DEV), torch.rand(3, 4, 2, 2, device=DEV)
        c.collect(a)
        c.collect(b)
        assert torch.equal(c.compute_amax(), torch.max(a, b).amax(dim=(1, 2, 3), keepdim=True))
    with pytest.raises(RuntimeError, match="shape changed"):
        c.collect(torch.rand(4, 4, 2, 2, device=DEV))


def _swap_amax_quant_func(tq):
    """the caller-side ``quant_func`` of the reference's MSE tests (test_mse_calibrator.py:51-67)"""
    from modelopt_amd.torch.quantization.utils import disable_calib, enable_fake_quant, enable_quant

    def quant_func(x, amax):
        held = tq._amax.clone()
        tq._amax = amax
        with enable_quant(tq), disable_calib(tq), enable_fake_quant(tq):
            xq = tq(x)
        tq._amax = held
        return xq
    return quant_func


def test_mse_calibrator_with_a_caller_supplied_quant_func():
    """test_mse_calibrator.py:40-86, :233-319, :321-370: the search never ends above the bulk-only
    loss, honours a custom error function, forgets its state on reset and keeps per-channel shape."""
    from modelopt_amd.torch.quantization import calib

    x = torch.ones(1024, device=DEV)
    x[0] = 10.0
    first = x.abs().max()
    tq = TensorQuantizer(Cfg(num_bits=8, axis=None), amax=first).to(DEV)
    cal = calib.MseCalibrator(amax=first, num_steps=20, start_multiplier=0.1, stop_multiplier=1.5,
                              quant_func=_swap_amax_quant_func(tq))
    cal.collect(x)
    best = cal.compute_amax()
    assert torch.isfinite(best) and 0 < best <= first * 1.5 + 1e-6
    mse = lambda a: ((_ref(x, a, narrow=True) - x) ** 2).mean()
    assert mse(best) <= mse(torch.tensor(1.0, device=DEV)) + 1e-6
    assert torch.equal(tq.amax, first)                              # the quantizer's own amax is back
    cal.reset()
    assert cal.compute_amax() is None

    cal = calib.MseCalibrator(amax=first, num_steps=15, start_multiplier=0.5, stop_multiplier=1.5,
                              quant_func=_swap_amax_quant_func(tq),
                              error_func=lambda t, tq_: (t - tq_).abs().mean())
    cal.collect(x)
    best = cal.compute_amax()
    assert torch.isfinite(best) and 0 < best <= first * 1.5 + 1e-6

    w = torch.tensor([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]], device=DEV)
    first = torch.tensor([[3.0], [6.0]], device=DEV)
    tq = TensorQuantizer(Cfg(num_bits=8, axis=0), amax=first).to(DEV)
    cal = calib.MseCalibrator(amax=first, axis=0, num_steps=10, start_multiplier=0.5, stop_multiplier=2.0,
                              quant_func=_swap_amax_quant_func(tq))
    cal.collect(w)
    cal.collect(w)
    best = cal.compute_amax()
    assert best.shape == first.shape and torch.isfinite(best).all() and (best > 0).all()
