"""GPU tests of the host layer (TensorQuantizer, calibrators, mtq.quantize, SmoothQuant,
AWQ-lite) against the CPU oracle."""

import copy
import json
import os

import pytest
import torch
import torch.nn.functional as F
from torch import nn

import modelopt_amd.torch.quantization as mtq
from conftest import GOLDEN, assert_bits_equal
from modelopt_amd.torch.quantization import calib
from modelopt_amd.torch.quantization.config import QuantizerAttributeConfig
from modelopt_amd.torch.quantization.nn import TensorQuantizer
from modelopt_amd.torch.quantization.qtensor import NVFP4QTensor
from oracle import awq as oawq
from oracle import fake_quant, qtensor, reduce

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
with open(os.path.join(GOLDEN, "reference_vectors.json")) as f:
    VEC = json.load(f)


def _rand(shape, dtype=torch.bfloat16, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


# ----------------------------------------------------------------------------- calibrator
def test_max_calibrator_like_reference_tests():
    c = calib.MaxCalibrator(8, None, False)
    a, b = _rand((16,), torch.float32, 1).abs(), _rand((16,), torch.float32, 2).abs()
    c.collect(a.to(DEV)); c.collect(b.to(DEV))
    assert torch.equal(c.compute_amax().cpu(), torch.max(a.max(), b.max()))
    for axis in (0, -4):
        c = calib.MaxCalibrator(8, axis, False)
        a, b = _rand((3, 4, 2, 2), torch.float32, 3), _rand((3, 4, 2, 2), torch.float32, 4)
        c.collect(a.to(DEV)); c.collect(b.to(DEV))
        o = reduce.MaxCalibrator(8, axis, False)
        o.collect(a); o.collect(b)
        assert c.compute_amax().shape == o.compute_amax().shape
        assert torch.equal(c.compute_amax().cpu(), o.compute_amax())
        c.reset()
        assert c.compute_amax() is None
    c = calib.MaxCalibrator(8, 0, False)
    c.collect(_rand((3, 4, 2, 2), torch.float32, 5).to(DEV))
    with pytest.raises(RuntimeError, match="shape changed"):
        c.collect(_rand((4, 4, 2, 2), torch.float32, 6).to(DEV))


def test_max_calibrator_flags_nan_and_inf_at_compute():
    c = calib.MaxCalibrator(8, None, False)
    x = _rand((64,), torch.float32, 7)
    x[3] = float("nan")
    c.collect(x.to(DEV))
    with pytest.raises(AssertionError, match="nan"):
        c.compute_amax()
    c = calib.MaxCalibrator(8, None, False)
    x[3] = float("inf")
    c.collect(x.to(DEV))
    with pytest.raises(AssertionError, match="inf"):
        c.compute_amax()


# ----------------------------------------------------------------------------- TensorQuantizer
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_quantizer_int8_per_tensor_and_channel(dtype):
    x = _rand((32, 64), dtype, 10)
    q = TensorQuantizer(QuantizerAttributeConfig(num_bits=8)).to(DEV)
    y = q(x.to(DEV))  # dynamic amax
    assert_bits_equal(y.cpu(), fake_quant.tensor_quant(x, reduce.reduce_amax(x), 8, False, False), "dynamic")
    q = TensorQuantizer(QuantizerAttributeConfig(num_bits=8, axis=0), amax=None).to(DEV)
    q.enable_calib(); q.disable_quant()
    q(x.to(DEV)); q(2 * x.to(DEV))
    q.load_calib_amax(); q.enable_quant(); q.disable_calib()
    want_amax = reduce.reduce_amax(2 * x, axis=[1])
    assert_bits_equal(q.amax.cpu(), want_amax, "calibrated per-channel amax")
    y = q(x.to(DEV))
    assert_bits_equal(y.cpu(), fake_quant.tensor_quant(x, want_amax, 8, False, False), "per channel")


@pytest.mark.usefixtures("cpu_fp8_overflow")
def test_quantizer_fp8_and_noncontiguous():
    x = _rand((48, 40), torch.bfloat16, 11)
    q = TensorQuantizer(QuantizerAttributeConfig(num_bits=(4, 3)), amax=3.0).to(DEV)
    y = q(x.to(DEV))
    assert_bits_equal(y.cpu(), fake_quant.fp8_eager(x, torch.tensor(3.0)), "fp8 static amax")
    xt = x.to(DEV).t()  # non-contiguous view
    y = q(xt)
    assert_bits_equal(y.cpu(), fake_quant.fp8_eager(x.t().contiguous(), torch.tensor(3.0)), "transposed")


@pytest.mark.parametrize("k", [256, 200])
def test_quantizer_int4_static_block(k):
    x = _rand((24, k), torch.bfloat16, 12, 0.02)
    q = TensorQuantizer(QuantizerAttributeConfig(num_bits=4, block_sizes={-1: 128})).to(DEV)
    y = q(x.to(DEV))
    assert y.shape == x.shape
    assert_bits_equal(y.cpu().contiguous(), oawq.int4_block_qdq(x, 128).contiguous(), "block 128 dynamic amax")
    # calibrated: amax buffer [rows, 1], export shape [N, K/128]
    q = TensorQuantizer(QuantizerAttributeConfig(num_bits=4, block_sizes={-1: 128})).to(DEV)
    q.enable_calib(); q.disable_quant(); q(x.to(DEV)); q.load_calib_amax()
    q.enable_quant(); q.disable_calib()
    assert q.amax.shape == (24 * (-(-k // 128)), 1)
    assert q.export_amax().shape == (24, -(-k // 128))
    assert_bits_equal(q(x.to(DEV)).cpu().contiguous(), oawq.int4_block_qdq(x, 128).contiguous(), "calibrated")


def test_quantizer_nvfp4_dynamic_and_pre_quant_scale():
    cfg = QuantizerAttributeConfig(num_bits=(2, 1),
                                   block_sizes={-1: 16, "type": "dynamic", "scale_bits": (4, 3)})
    x = _rand((4, 8, 64), torch.bfloat16, 13)
    q = TensorQuantizer(cfg).to(DEV)
    y = q(x.to(DEV))  # global amax computed on the fly
    assert_bits_equal(y.cpu(), fake_quant.nvfp4_fake_quant(x, reduce.reduce_amax(x), 16), "dynamic amax")
    q.amax = torch.tensor(2.5, dtype=torch.bfloat16)
    assert_bits_equal(q(x.to(DEV)).cpu(), fake_quant.nvfp4_fake_quant(x, torch.tensor(2.5), 16), "static amax")
    s = (torch.rand(64) + 0.5).to(torch.bfloat16)
    q.pre_quant_scale = s.to(DEV)
    assert_bits_equal(q(x.to(DEV)).cpu(), fake_quant.nvfp4_fake_quant(x * s, torch.tensor(2.5), 16), "pqs")
    q.disable()
    assert_bits_equal(q(x.to(DEV)).cpu(), x * s, "pre_quant_scale still applied when disabled")


@pytest.mark.parametrize("case", [c for c in VEC["qtensor_roundtrip"]
                                  if c["block_sizes"] is None or len(c["block_sizes"]) == 1],
                         ids=lambda c: c["name"])
def test_real_quantize_golden_through_tensor_quantizer(case):
    """tests/gpu/torch/quantization/test_qtensor_cuda.py:243-262 with the reference's vectors."""
    bits = tuple(case["num_bits"]) if isinstance(case["num_bits"], list) else case["num_bits"]
    bs = None if case["block_sizes"] is None else {int(k): v for k, v in case["block_sizes"].items()}
    q = TensorQuantizer(QuantizerAttributeConfig(num_bits=bits, block_sizes=bs, fake_quant=False,
                                                 axis=case["axis"])).to(DEV)
    x = torch.tensor(case["input"], dtype=torch.bfloat16).to(DEV)
    packed = q(x)
    deq = q(packed)
    assert torch.allclose(deq.cpu(), torch.tensor(case["output"], dtype=torch.bfloat16))


def test_nvfp4_real_quantize_uses_quantizer_amax():
    cfg = QuantizerAttributeConfig(num_bits=(2, 1), fake_quant=False,
                                   block_sizes={-1: 16, "type": "dynamic", "scale_bits": (4, 3)})
    q = TensorQuantizer(cfg).to(DEV)
    q.amax = torch.tensor(1.1)
    x = torch.rand(32, 32, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
    out = q(x.to(DEV))
    assert torch.allclose(q._double_scale.cpu(), torch.tensor(1.1) / 448.0 / 6.0)
    wsf2 = torch.tensor(1.1).float() / (448.0 * 6.0)
    wsf_o, _ = qtensor.nvfp4_block_scales(x, 16, wsf2)
    p_o, _, _ = qtensor.nvfp4_quantize(x, 16, wsf_o, wsf2)
    assert_bits_equal(out._quantized_data.cpu(), p_o, "packed")
    assert_bits_equal(q._scale.cpu(), wsf_o, "block scales")
    deq = q(out)
    assert_bits_equal(deq.cpu(), qtensor.nvfp4_dequantize(p_o, wsf_o, wsf2, 16, x.shape, torch.bfloat16), "deq")


def test_nvfp4_qtensor_classmethods():
    x = _rand((16, 64), torch.bfloat16, 14, 0.02)
    xd = x.to(DEV)
    assert_bits_equal(NVFP4QTensor.get_weights_scaling_factor_2(xd).cpu(), qtensor.nvfp4_global_scale(x), "wsf2")
    wsf, wsf2 = NVFP4QTensor.get_weights_scaling_factor(xd, 16)
    wsf_o, wsf2_o = qtensor.nvfp4_block_scales(x, 16)
    assert_bits_equal(wsf.cpu(), wsf_o, "wsf")
    qt, wsf_b, wsf2_b = NVFP4QTensor.quantize(xd, 16, wsf, wsf2)
    p_o, _, _ = qtensor.nvfp4_quantize(x, 16, wsf_o, wsf2_o)
    assert_bits_equal(qt._quantized_data.cpu(), p_o, "packed with given scales")
    hp, _ = NVFP4QTensor.get_weights_scaling_factor(xd, 16, keep_high_precision=True)
    hp_o, _ = qtensor.nvfp4_block_scales(x, 16, keep_high_precision=True)
    assert_bits_equal(hp.cpu(), hp_o, "high precision scales")


# ----------------------------------------------------------------------------- mtq.quantize
class _MLP(nn.Module):
    def __init__(self, d=64, h=128, dtype=torch.bfloat16, seed=0):
        super().__init__()
        g = torch.Generator().manual_seed(seed)
        self.fc1 = nn.Linear(d, h, bias=True)
        self.fc2 = nn.Linear(h, d, bias=False)
        self.lm_head = nn.Linear(d, 32, bias=False)
        for p in self.parameters():
            p.data = (torch.randn(p.shape, generator=g) * 0.1)
        self.to(dtype)

    def forward(self, x):
        return self.lm_head(self.fc2(F.relu(self.fc1(x))))


def _batches(n=3, d=64, dtype=torch.bfloat16):
    return [_rand((8, 16, d), dtype, 100 + i) for i in range(n)]


def _oracle_linear_inputs(model, batches):
    """CPU activations seen by fc1 / fc2 / lm_head with quantisation off (calibration mode)."""
    acts = {"fc1": [], "fc2": [], "lm_head": []}
    for x in batches:
        acts["fc1"].append(x)
        h = F.relu(F.linear(x, model.fc1.weight, model.fc1.bias))
        acts["fc2"].append(h)
        y = F.linear(h, model.fc2.weight)
        acts["lm_head"].append(y)
    return acts


@pytest.mark.parametrize("cfg_name", ["INT8_DEFAULT_CFG", "FP8_DEFAULT_CFG", "NVFP4_DEFAULT_CFG"])
def test_quantize_max_calibration_amax_matches_oracle(cfg_name):
    ref = _MLP()
    model = copy.deepcopy(ref).to(DEV)
    batches = _batches()
    mtq.quantize(model, getattr(mtq, cfg_name), lambda m: [m(b.to(DEV)) for b in batches])
    assert not model.lm_head.input_quantizer.is_enabled and not model.lm_head.weight_quantizer.is_enabled
    # calibration runs with quantisation off, so GPU activations equal CPU ones up to GEMM
    # rounding; the weight amax is exact, the input amax is compared on GPU-side activations
    w_axis = [1] if cfg_name == "INT8_DEFAULT_CFG" else None
    for name in ("fc1", "fc2"):
        lin = getattr(model, name)
        want = reduce.reduce_amax(getattr(ref, name).weight.data, axis=w_axis)
        assert_bits_equal(lin.weight_quantizer.amax.cpu().reshape(want.shape), want, f"{name} weight amax")
    assert_bits_equal(model.fc1.input_quantizer.amax.cpu(),
                      torch.stack([reduce.reduce_amax(b) for b in batches]).max(), "fc1 input amax")
    assert model.fc2.input_quantizer.amax.numel() == 1 and model.fc2.input_quantizer.amax > 0
    out = model(batches[0].to(DEV))
    assert out.shape == (8, 16, 32) and torch.isfinite(out.float()).all()


def test_fp8_model_clamps_an_outlier_above_the_calibrated_amax():
    """A calibrated FP8_DEFAULT_CFG model (per-tensor amax) and FP8 KV quantizers clamp an input
    beyond the calibrated range, as the reference's CUDA kernel does (tensor_quant.py:62-90,
    src/tensor_quant_gpu_fp8.cu:36-47): the output stays finite."""
    model = _MLP().to(DEV)
    batches = _batches()
    mtq.quantize(model, mtq.FP8_DEFAULT_CFG, lambda m: [m(b.to(DEV)) for b in batches])
    x = batches[0].to(DEV).clone()
    x[0, 0, 0] = float(model.fc1.input_quantizer.amax) * 4
    assert torch.isfinite(model(x).float()).all()
    q = model.fc1.input_quantizer
    y = q(x)
    assert torch.isfinite(y.float()).all() and float(y.float().abs().max()) == float(q.amax)
    kv = TensorQuantizer(QuantizerAttributeConfig(**mtq.FP8_KV_CFG["quant_cfg"]["*[kv]_bmm_quantizer"]),
                         amax=1.0).to(DEV)
    t = torch.tensor([[0.5, 1.0, 1.5, -7.0]], dtype=torch.bfloat16, device=DEV)
    assert torch.equal(kv(t).cpu(), torch.tensor([[0.5, 1.0, 1.0, -1.0]], dtype=torch.bfloat16))


def test_quantized_linear_forward_equals_oracle_composition():
    ref = _MLP()
    model = copy.deepcopy(ref).to(DEV)
    batches = _batches()
    mtq.quantize(model, mtq.INT8_DEFAULT_CFG, lambda m: [m(b.to(DEV)) for b in batches])
    x = batches[1]
    lin = model.fc1
    xq = fake_quant.tensor_quant(x, lin.input_quantizer.amax.cpu(), 8, False, False)
    wq = fake_quant.tensor_quant(ref.fc1.weight.data, lin.weight_quantizer.amax.cpu(), 8, False, False)
    got_x = lin.input_quantizer(x.to(DEV))
    got_w = lin.weight_quantizer(lin.weight)
    assert_bits_equal(got_x.cpu(), xq, "input fake quant")
    assert_bits_equal(got_w.cpu(), wq, "weight fake quant")
    y = lin(x.to(DEV))
    assert torch.allclose(y.cpu().float(), F.linear(xq, wq, ref.fc1.bias).float(), rtol=2e-2, atol=2e-2)


def test_weight_amax_is_cached_inside_a_calibration_pass_only():
    from modelopt_amd.torch.quantization import model_calib
    from modelopt_amd.torch.quantization.nn.modules.tensor_quantizer import calibration_pass

    model = _MLP().to(DEV)
    mtq.replace_quant_module(model)
    mtq.set_quantizer_by_cfg(model, mtq.model_quant._validated(mtq.INT8_DEFAULT_CFG)[0])
    model_calib.enable_stats_collection(model)
    calls = []
    cal = model.fc1.weight_quantizer._calibrator
    orig = cal.collect
    cal.collect = lambda x: (calls.append(1), orig(x))[1]
    with calibration_pass():
        for b in _batches(4):
            model(b.to(DEV))
        assert len(calls) == 1  # the unchanged weight was reduced once, not once per forward
        with torch.no_grad():
            model.fc1.weight.mul_(0.5)  # an in-place update bumps the version
        model(_batches(1)[0].to(DEV))
        assert len(calls) == 2
    for b in _batches(2):  # outside a pass every forward reduces, as in the reference
        model(b.to(DEV))
    assert len(calls) == 4
    model_calib.finish_stats_collection(model)


def test_recalibration_after_an_in_place_data_write_sees_the_new_weight():
    """``weight.data.mul_(2)`` bumps no version counter; a second calibration without
    ``reset_amax`` still re-reduces the weight and the running maximum doubles, as in the
    reference (every forward collects, quant_module.py:148-169)."""
    ref = _MLP()
    model = copy.deepcopy(ref).to(DEV)
    batches = _batches(2)
    loop = lambda m: [m(b.to(DEV)) for b in batches]  # noqa: E731
    mtq.quantize(model, mtq.FP8_DEFAULT_CFG, loop)
    first = model.fc1.weight_quantizer.amax.clone()
    assert_bits_equal(first.cpu().reshape(()), reduce.reduce_amax(ref.fc1.weight.data), "first amax")
    model.fc1.weight.data.mul_(2)
    mtq.calibrate(model, "max", loop)
    assert_bits_equal(model.fc1.weight_quantizer.amax.cpu().reshape(()),
                      reduce.reduce_amax(ref.fc1.weight.data * 2), "amax after the write")
    # a history-tracking calibrator sees every forward
    from modelopt_amd.torch.quantization import calib as calib_mod, model_calib
    from modelopt_amd.torch.quantization.nn.modules.tensor_quantizer import calibration_pass

    q = model.fc1.weight_quantizer
    q._calibrator = calib_mod.MaxCalibrator(q._calibrator._num_bits, q._calibrator._axis,
                                            q._calibrator._unsigned, track_amax=True)
    model_calib.enable_stats_collection(model)
    with calibration_pass():
        loop(model)
    assert len(q._calibrator.amaxs) == len(batches)
    model_calib.finish_stats_collection(model)


# ----------------------------------------------------------------------------- SmoothQuant
def test_smoothquant_matches_oracle():
    ref = _MLP()
    model = copy.deepcopy(ref).to(DEV)
    batches = _batches()
    cfg = copy.deepcopy(mtq.INT8_SMOOTHQUANT_CFG)
    cfg["algorithm"] = {"method": "smoothquant", "alpha": 0.5}
    mtq.quantize(model, cfg, lambda m: [m(b.to(DEV)) for b in batches])
    act_amax = torch.stack([reduce.reduce_amax(b, axis=[0, 1]) for b in batches]).amax(0)  # [1,1,K]
    pqs, w_new, in_amax, w_amax = oawq.smoothquant_linear(ref.fc1.weight.data, act_amax, alpha=0.5)
    lin = model.fc1
    assert_bits_equal(lin.input_quantizer._pre_quant_scale.cpu().reshape(-1), pqs.reshape(-1), "pre_quant_scale")
    assert_bits_equal(lin.weight.data.cpu(), w_new, "smoothed weight")
    assert_bits_equal(lin.input_quantizer.amax.cpu().reshape(()), in_amax.reshape(()), "input amax")
    assert_bits_equal(lin.weight_quantizer.amax.cpu().reshape(w_amax.shape), w_amax, "weight amax")


# ----------------------------------------------------------------------------- AWQ-lite
class _OneLinear(nn.Module):
    def __init__(self, n=128, k=256, seed=0):
        super().__init__()
        g = torch.Generator().manual_seed(seed)
        self.proj = nn.Linear(k, n, bias=False)
        self.proj.weight.data = (0.02 * torch.randn(n, k, generator=g))
        self.to(torch.bfloat16)

    def forward(self, x):
        return self.proj(x)


def _awq_batches(k=256, n=2, tokens=64):
    g = torch.Generator().manual_seed(3)
    c = torch.exp(torch.randn(k, generator=g))
    hot = torch.randperm(k, generator=g)[: max(1, k // 100)]
    c[hot] *= 20
    return [(torch.randn(tokens, k, generator=g) * c).to(torch.bfloat16) for _ in range(n)]


@pytest.mark.parametrize("alpha_step", [0.1, 0.05])
def test_awq_lite_matches_oracle(alpha_step):
    ref = _OneLinear()
    model = copy.deepcopy(ref).to(DEV)
    batches = _awq_batches()
    cfg = copy.deepcopy(mtq.INT4_AWQ_CFG)
    cfg["algorithm"] = {"method": "awq_lite", "alpha_step": alpha_step, "debug": True}
    mtq.quantize(model, cfg, lambda m: [m(b.to(DEV)) for b in batches])
    losses, best_alpha, best_scale, act_scale, weight_scale = oawq.awq_lite_search(
        ref.proj.weight.data, batches, alpha_step, 128)
    h = model.proj.awq_lite
    assert list(h.loss) == list(losses)  # identical fp32 alpha keys
    assert len(h.loss) == (21 if alpha_step == 0.05 else 11)
    for a in losses:
        assert h.loss[a] == pytest.approx(losses[a], rel=1e-3), f"alpha {a}"
    assert h.best_alpha == best_alpha
    assert torch.allclose(h.act_scale.cpu(), act_scale, rtol=2 ** -7)
    assert torch.allclose(h.weight_scale.cpu(), weight_scale, rtol=2 ** -7)
    # folding: input pre_quant_scale and smoothed weight from the oracle's formula on the
    # GPU's own best_scale (the statistics may differ from the CPU's in the last bf16 bit)
    pqs, w_new = oawq.fold_pre_quant_scale(ref.proj.weight.data, 1.0 / h.best_scale.cpu())
    assert_bits_equal(model.proj.input_quantizer._pre_quant_scale.cpu(), pqs, "pre_quant_scale")
    assert_bits_equal(model.proj.weight.data.cpu(), w_new, "folded weight")
    want_amax = reduce.reduce_amax(w_new.reshape(-1, 128), axis=[1], keepdims=True)
    assert_bits_equal(model.proj.weight_quantizer.amax.cpu(), want_amax, "recalibrated block amax")
    assert "forward" not in model.proj.__dict__  # patch removed


def test_awq_search_paths_agree(monkeypatch):
    """Three routes through a search step: (a) one launch for all alphas (weights quantised in
    front of the matrix cores), (b) per alpha a fused weight kernel + library GEMM + loss kernel,
    (c) per alpha through the quantizer modules.  (b) and (c) run the same GEMM on the same
    operands and agree exactly; (a) accumulates in a different order, so its losses agree to
    1e-4 relative -- with the same selected alpha, hence the same folded weight."""
    from modelopt_amd.torch.quantization import model_calib

    batches = _awq_batches()
    results = {}
    for route in "abc":
        model = _OneLinear().to(DEV)
        if route != "a":
            monkeypatch.setattr(model_calib, "_one_launch_search", lambda *a, **k: False)
        if route == "c":
            monkeypatch.setattr(model_calib, "_fused_weight_path", lambda m: False)
        cfg = copy.deepcopy(mtq.INT4_AWQ_CFG)
        cfg["algorithm"] = {"method": "awq_lite", "alpha_step": 0.1, "debug": True}
        mtq.quantize(model, cfg, lambda m: [m(b.to(DEV)) for b in batches])
        h = model.proj.awq_lite
        results[route] = (h.loss, h.best_alpha, model.proj.weight.data.clone())
    assert results["b"][0] == results["c"][0]
    assert torch.equal(results["b"][2], results["c"][2])
    for alpha, want in results["b"][0].items():
        assert results["a"][0][alpha] == pytest.approx(want, rel=1e-4)
    assert results["a"][1] == results["b"][1]
    assert torch.equal(results["a"][2], results["b"][2])


def test_true_divide_is_one_rounding_on_the_gpu():
    """The helper behind every ``amax / constant`` scale equals the CPU's true division."""
    from modelopt_amd.torch.quantization.utils import true_divide

    g = torch.Generator().manual_seed(0)
    t = torch.rand(200000, generator=g) * 10 + 1e-3
    for d in (448.0, 2688.0, 7.0, 127.0):
        want = t / d  # CPU: true division
        got = true_divide(t.to(DEV), d).cpu()
        assert torch.equal(got, want), d
    tb = t[:4096].to(torch.bfloat16)
    assert torch.equal(true_divide(tb.to(DEV), 448.0).cpu(), tb / 448.0)


# ----------------------------------------------------------------------------- AWQ-clip
def test_awq_clip_matches_oracle():
    ref = _OneLinear(n=64, k=256)
    model = copy.deepcopy(ref).to(DEV)
    batches = _awq_batches(k=256, n=2, tokens=96)
    cfg = copy.deepcopy(mtq.INT4_AWQ_CFG)
    cfg["algorithm"] = {"method": "awq_clip", "max_tokens_per_batch": 32, "debug": True}
    mtq.quantize(model, cfg, lambda m: [m(b.to(DEV)) for b in batches])
    losses, best = oawq.awq_clip_search(ref.proj.weight.data, batches, 128, 4, max_tokens_per_batch=32)
    h = model.proj.awq_clip
    assert list(h.loss) == list(losses) and len(losses) == 11
    assert h.num_tokens == 64
    w_amax = reduce.reduce_amax(ref.proj.weight.data.reshape(-1, 128), axis=[1], keepdims=True)
    assert_bits_equal(h.w_amax.cpu(), w_amax, "block amax before clipping")
    # the partial sums are bf16 torch reductions whose last bit can depend on the summation
    # order; in practice the losses agree to 1e-8 and every block picks the same ratio
    for r in losses:
        got, want = h.loss[r].cpu(), losses[r]
        rel = (got - want).abs().sum() / want.abs().sum().clamp(min=1e-30)
        assert float(rel) < 1e-4, f"ratio {r}: {float(rel)}"
    got_best = model.proj.weight_quantizer.amax.cpu()
    same = (got_best == best).float().mean()
    assert float(same) >= 0.99, float(same)
    ratio = (got_best.float() / w_amax.float())
    assert float(ratio.min()) >= 0.49 and float(ratio.max()) <= 1.0
    assert model.proj.weight_quantizer.is_enabled and "forward" not in model.proj.__dict__
    assert torch.isfinite(model(batches[0].to(DEV)).float()).all()


def test_awq_full_runs_lite_then_clip():
    model = _OneLinear(n=64, k=256).to(DEV)
    batches = _awq_batches(k=256, n=2, tokens=64)
    cfg = copy.deepcopy(mtq.INT4_AWQ_CFG)
    cfg["algorithm"] = {"method": "awq_full", "alpha_step": 0.25, "debug": True}
    mtq.quantize(model, cfg, lambda m: [m(b.to(DEV)) for b in batches])
    assert hasattr(model.proj, "awq_lite") and hasattr(model.proj, "awq_clip")
    assert model.proj.input_quantizer._pre_quant_scale is not None
    assert model.proj.weight_quantizer.amax.shape == (64 * 2, 1)
    assert torch.isfinite(model(batches[0].to(DEV)).float()).all()


@pytest.mark.parametrize("cfg", [
    dict(num_bits=8, axis=None),
    dict(num_bits=8, axis=0),
    dict(num_bits=4, block_sizes={-1: 32}),
    dict(num_bits=(4, 3), axis=None),
    dict(num_bits=(2, 1), block_sizes={-1: 16, "type": "dynamic", "scale_bits": (4, 3)}),
    dict(num_bits=(2, 1), block_sizes={-1: 32, "type": "dynamic", "scale_bits": (8, 0)}),
], ids=["int8", "int8-axis0", "int4-block", "fp8", "nvfp4", "mxfp4"])
def test_quantizers_on_views_equal_the_contiguous_result(cfg):
    """tests/gpu/torch/quantization/test_tensor_quantizer_cuda.py:93-107 (non-contiguous FP4
    input), for every quantizer family: a transposed view, a strided slice and an expanded
    tensor quantise to what their contiguous copies do, calibration included."""
    from modelopt_amd.torch.quantization.model_calib import (enable_stats_collection,
                                                              finish_stats_collection)

    g = torch.Generator().manual_seed(4)
    base = torch.randn(96, 128, generator=g).to(torch.bfloat16).to(DEV)
    views = [base.t(), base[::2, 32:96], base[:1].expand(64, 128)]
    for v in views:
        assert not v.is_contiguous()
        results = []
        for x in (v, v.contiguous()):
            q = TensorQuantizer(QuantizerAttributeConfig(**cfg)).to(DEV)
            if not q._dynamic:
                enable_stats_collection(q)
                q(x)
                finish_stats_collection(q)
            amax = q.amax          # the MX formats and dynamic quantizers keep none
            results.append((q(x), None if amax is None else amax.clone()))
        assert results[0][0].shape == v.shape
        assert_bits_equal(results[0][0].cpu(), results[1][0].cpu(), f"{tuple(v.shape)} {v.stride()}")
        if results[0][1] is not None:
            assert_bits_equal(results[0][1].cpu(), results[1][1].cpu(), "amax")


@pytest.mark.parametrize("cfg", [
    dict(num_bits=8, axis=None),
    dict(num_bits=(4, 3), axis=None),
    dict(num_bits=(2, 1), block_sizes={-1: 16, "type": "dynamic", "scale_bits": (4, 3)}),
], ids=["int8", "fp8", "nvfp4"])
def test_straight_through_gradient_with_clipping(cfg):
    """tests/gpu/torch/quantization/test_tensor_quantizer_cuda.py:76-91: with an amax below the
    data's maximum the gradient of sum(q(x)) is 1 where |x| <= amax and 0 beyond it."""
    q = TensorQuantizer(QuantizerAttributeConfig(**cfg)).to(DEV)
    x = torch.rand(2, 1, 16, generator=torch.Generator().manual_seed(0)).to(DEV)
    with torch.no_grad():
        q.amax = torch.median(x.abs())
    x.requires_grad = True
    q(x).sum().backward()
    assert torch.allclose(x.grad, torch.ones_like(x.grad) * (x.abs() <= q.amax))
    assert 0 < float(x.grad.sum()) < x.numel()


def test_per_tensor_calibration_of_a_permuted_view_makes_no_copy(monkeypatch):
    """K / V reach their quantizers as [B, H, S, D] views of a [B, S, H, D] projection: the
    per-tensor abs-max is taken over the memory as it lies and equals the oracle's."""
    from modelopt_amd import _hip
    from modelopt_amd.torch.quantization import kernels

    x = _rand((4, 64, 8, 32), seed=31)
    view = x.to(DEV).transpose(1, 2)
    assert not view.is_contiguous()
    seen = []
    real = _hip.absmax_into
    monkeypatch.setattr(_hip, "absmax_into", lambda t, *a, **k: (seen.append(t.data_ptr()), real(t, *a, **k))[1])
    cal = calib.MaxCalibrator(8, None, False)
    cal.collect(view)
    assert seen == [view.data_ptr()]                       # reduced in place, not through a copy
    assert_bits_equal(cal.compute_amax().cpu(), reduce.reduce_amax(x), "amax of the view")
    sliced = x.to(DEV)[:, :, :4]                           # gaps: falls back to a contiguous copy
    cal2 = calib.MaxCalibrator(8, None, False)
    cal2.collect(sliced)
    assert_bits_equal(cal2.compute_amax().cpu(), reduce.reduce_amax(x[:, :, :4]), "amax of a slice")
    assert kernels.dense_flat_view(sliced) is None


# ----------------------------------------------------------------------------- shared reductions
def test_calibrators_shown_one_tensor_in_a_row_share_its_reduction():
    """Inside a calibration pass the input of q_proj / k_proj / v_proj is read once: the first
    calibrator's launch leaves the tile maxima behind and the others fold those in later."""
    from modelopt_amd import _hip as hip
    from modelopt_amd.torch.quantization.calib import MaxCalibrator
    from modelopt_amd.torch.quantization.nn.modules.tensor_quantizer import calibration_pass

    cals = [MaxCalibrator(8, None, False) for _ in range(3)]
    batches = [_rand((16, 512, 256), torch.bfloat16, 300 + i, scale=1.0 + i).to(DEV) for i in range(3)]
    with calibration_pass(), hip.KernelTimer() as timer:
        for b in batches:
            for c in cals:
                c.collect(b)
    # the first batch finds out that the tensor is shared (three plain reductions); from the
    # second on one reduction per batch serves all three calibrators
    assert timer.calls == {"mo_absmax": 3, "mo_absmax_tensor_parts": 2}
    want = max(float(reduce.reduce_amax(b.cpu(), None)) for b in batches)
    for c in cals:
        assert float(c.compute_amax()) == want
        assert c.compute_amax().dtype == torch.bfloat16

    # a tensor written in place between two calibrators is reduced again; so is an equal copy
    a, b, c = (MaxCalibrator(8, None, False) for _ in range(3))
    x = _rand((64, 1024), torch.bfloat16, 310).to(DEV)
    with calibration_pass(), hip.KernelTimer() as timer:
        a.collect(x)
        x.mul_(2)
        b.collect(x)
        c.collect(x.clone())
    assert timer.calls == {"mo_absmax": 3}
    assert float(b.compute_amax()) == 2 * float(a.compute_amax()) == float(c.compute_amax())

    # outside a pass of the package every collect reduces, as the reference does
    a, b = MaxCalibrator(8, None, False), MaxCalibrator(8, None, False)
    with hip.KernelTimer() as timer:
        a.collect(x)
        b.collect(x)
    assert timer.calls == {"mo_absmax": 2}
    assert float(a.compute_amax()) == float(b.compute_amax())


def test_shared_reductions_fold_after_many_batches_and_keep_nan():
    from modelopt_amd.torch.quantization.calib import MaxCalibrator
    from modelopt_amd.torch.quantization.nn.modules.tensor_quantizer import calibration_pass

    lead, follow = MaxCalibrator(8, None, False), MaxCalibrator(8, None, False)
    g = torch.Generator().manual_seed(320)
    want = 0.0
    with calibration_pass():
        for i in range(150):     # more than one fold of the noted tile maxima
            x = (torch.randn((8, 4096), generator=g) * (1 + i % 7)).to(torch.float16).to(DEV)
            want = max(want, float(x.abs().max()))
            lead.collect(x)
            follow.collect(x)
    assert float(lead.compute_amax()) == want == float(follow.compute_amax())
    with calibration_pass():
        x = torch.ones((8, 4096), dtype=torch.bfloat16, device=DEV)
        x[3, 7] = float("nan")
        lead.collect(x)
        follow.collect(x)
    with pytest.raises(AssertionError, match="nan"):
        follow.compute_amax()


# ----------------------------------------------------------------------------- strict host checks
def test_strict_checks_on_the_device():
    """``mtq.set_strict_checks(True)``: the reference's CPU-path errors (tensor_quant.py:577-587,
    calib/max.py:69-77) for device tensors, at the reference's moment; without it the kernels
    clamp like the reference's CUDA kernel and the calibrator reports in ``compute_amax``."""
    from modelopt_amd.torch.quantization.tensor_quant import fake_tensor_quant

    x = _rand((3, 7), torch.float32, seed=1).to(DEV)
    amax = x.abs().max()
    clamped = fake_tensor_quant(x, amax, None, 8, True)          # default: negatives clamp to 0
    assert float(clamped.min()) == 0.0
    previous = mtq.set_strict_checks(True)
    try:
        with pytest.raises(TypeError, match="Negative values encountered"):
            fake_tensor_quant(x, amax, None, 8, True)
        with pytest.raises(ValueError, match="Negative values in amax"):
            fake_tensor_quant(x, -amax)
        assert_bits_equal(fake_tensor_quant(x.abs(), amax, None, 8, True).cpu(),
                          fake_quant.tensor_quant(x.abs().cpu(), amax.cpu(), 8, True, True), "accepted case")
        c = calib.MaxCalibrator(8, None, False)
        c.collect(_rand((64, 64), seed=2).to(DEV))
        good = c.compute_amax().clone()
        bad = _rand((64, 64), seed=3)
        bad[5, 5] = float("nan")
        with pytest.raises(AssertionError, match="detected nan values in amax. nan in original tensor: True"):
            c.collect(bad.to(DEV))
        assert_bits_equal(c.compute_amax().cpu(), good.cpu(), "the bad batch was not folded in")
        q = TensorQuantizer(QuantizerAttributeConfig(num_bits=8, unsigned=True)).to(DEV)
        with pytest.raises(TypeError, match="Negative values encountered"):
            q(x)
    finally:
        mtq.set_strict_checks(previous)


def test_k_and_v_calibrate_in_one_launch():
    """The K / V cache quantizers of an attention layer are shown their tensors together: while
    both only calibrate per tensor, one launch reduces both (same amax as one by one), a
    transposed dense view included; any other state takes the two ordinary forwards."""
    from modelopt_amd import _hip

    def fresh():
        q = TensorQuantizer(QuantizerAttributeConfig(num_bits=(4, 3), axis=None)).to(DEV)
        q.enable_calib(); q.disable_quant()
        return q

    k = _rand((4, 8, 96, 128), seed=21).to(DEV)
    v = _rand((4, 96, 8, 128), seed=22).to(DEV).transpose(1, 2)            # [B, H, S, D] view
    qk, qv = fresh(), fresh()
    with _hip.KernelTimer() as timer:
        for _ in range(2):
            out_k, out_v = TensorQuantizer.forward_pair(qk, k, qv, v)
    assert timer.calls == {"mo_absmax_pair": 2}
    assert out_k is k and out_v is v
    for q, x in ((qk, k), (qv, v)):
        q.load_calib_amax()
        assert_bits_equal(q.amax.cpu().reshape(()), reduce.reduce_amax(x.cpu()).reshape(()), "amax")
    # a hook on either quantizer must see its call: the ordinary forwards run
    qk3, qv3 = fresh(), fresh()
    calls = []
    handle = qv3.register_forward_pre_hook(lambda m, a: calls.append(tuple(a[0].shape)))
    with _hip.KernelTimer() as timer:
        TensorQuantizer.forward_pair(qk3, k, qv3, v)
    handle.remove()
    assert calls == [tuple(v.shape)] and "mo_absmax_pair" not in timer.calls
    # a quantizer that also quantises (or is disabled, per channel, ...) takes its own forward
    qk2, qv2 = fresh(), fresh()
    qv2.enable_quant(); qv2.amax = torch.tensor(8.0, device=DEV)
    with _hip.KernelTimer() as timer:
        out_k, out_v = TensorQuantizer.forward_pair(qk2, k, qv2, v)
    assert "mo_absmax_pair" not in timer.calls
    assert_bits_equal(out_v.cpu(), fake_quant.fp8_eager(v.cpu().contiguous(), torch.tensor(8.0)), "v fake quant")
    qk2.load_calib_amax()
    assert_bits_equal(qk2.amax.cpu().reshape(()), reduce.reduce_amax(k.cpu()).reshape(()), "k amax")


@pytest.mark.parametrize("seed,n,k,tokens", [(11, 128, 256, 64), (12, 256, 512, 200), (13, 384, 384, 96),
                                             (14, 128, 1024, 512), (15, 512, 256, 33), (16, 256, 256, 300),
                                             (17, 256, 256, 513), (18, 128, 384, 1300), (19, 256, 128, 2048)])
def test_awq_lite_selects_the_oracle_s_alpha_on_several_layers(seed, n, k, tokens, monkeypatch):
    """The one-launch search scores the alphas with arithmetic that differs from the CPU path's by
    an ulp of a rare weight; what matters downstream is which alpha wins.  Several layers and
    seeds: same best alpha as the CPU restatement of the search loop, losses within 1e-3, and the
    scale that is folded is the oracle's formula at that alpha."""
    g = torch.Generator().manual_seed(seed)
    ref = _OneLinear(n=n, k=k, seed=seed)
    c = torch.exp(torch.randn(k, generator=g))
    c[torch.randperm(k, generator=g)[: max(1, k // 64)]] *= 20
    batches = [(torch.randn(tokens, k, generator=g) * c).to(torch.bfloat16) for _ in range(2)]
    model = copy.deepcopy(ref).to(DEV)
    cfg = copy.deepcopy(mtq.INT4_AWQ_CFG)
    cfg["algorithm"] = {"method": "awq_lite", "alpha_step": 0.1, "debug": True}
    # batches of more than 512 tokens go through the search kernel in slices of 512 rows
    from modelopt_amd import _hip
    launches, real = [], _hip.awq_search_losses_into
    monkeypatch.setattr(_hip, "awq_search_losses_into",
                        lambda xs, *a: launches.append(xs.shape[2]) or real(xs, *a))
    mtq.quantize(model, cfg, lambda m: [m(b.to(DEV)) for b in batches])
    per_batch = [min(512, tokens - t) for t in range(0, tokens, 512)]
    assert launches == per_batch * len(batches)
    losses, best_alpha, best_scale, _, _ = oawq.awq_lite_search(ref.proj.weight.data, batches, 0.1, 128)
    h = model.proj.awq_lite
    assert h.best_alpha == best_alpha, (h.loss, losses)
    for a in losses:
        assert h.loss[a] == pytest.approx(losses[a], rel=1e-3), f"alpha {a}"
    assert torch.allclose(h.best_scale.cpu(), best_scale, rtol=2 ** -6)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("losses", [[3.0, 1.0, 2.0, 1.0], [float("nan"), 1.0, 0.5], [2.0, float("nan"), 1.5, float("inf")],
                                    [float("inf"), float("inf")], [5.0]])
def test_pick_scale_equals_the_host_s_min_and_the_tensor_expressions(dtype, losses):
    """mo_awq_pick_scale against ``min(loss, key=loss.get)`` (model_calib.py:633 of the reference)
    and the eager ``1.0 / best_scale``, ``.to(dtype)``, ``1.0 / pre_quant_scale`` of its folding."""
    g = torch.Generator().manual_seed(len(losses))
    k = 1000
    grid = torch.exp(torch.randn(len(losses), k, generator=g)).to(DEV)
    table = dict(enumerate(losses))
    want = min(table, key=table.get)
    from modelopt_amd import _hip

    loss = torch.tensor(losses, dtype=torch.float64, device=DEV)
    best, best_scale, pqs, pqs_t, fold = _hip.awq_pick_scale(loss, grid, dtype)
    assert int(best) == want
    assert torch.equal(best_scale, grid[want])
    eager = 1.0 / grid[want]
    assert torch.equal(pqs, eager) and pqs_t.dtype == dtype
    assert torch.equal(pqs_t.view(torch.int16 if dtype != torch.float32 else torch.int32),
                       eager.to(dtype).view(torch.int16 if dtype != torch.float32 else torch.int32))
    assert torch.equal(fold, 1.0 / eager)


def test_deferred_checks_on_the_device_take_one_launch():
    """Finite / non-negative / positive checks of a block of device tensors: same verdicts from
    the one-launch reduction as from the tensor expressions, for good and for bad values."""
    from modelopt_amd import _hip
    from modelopt_amd.torch.quantization import utils as qutils

    good = [torch.rand(100, device=DEV), torch.rand(7, device=DEV).to(torch.bfloat16), torch.tensor(3.0, device=DEV)]
    with _hip.KernelTimer() as timer:
        with qutils.deferred_scale_checks() as checks:
            assert qutils.all_valid_scales(good)
            assert qutils.all_positive(good[0] + 1)
            checks.report = [good[1]]
    assert checks.report_ok and timer.calls == {"mo_value_ranges": 1}
    for bad in (torch.tensor([1.0, -1e-3], device=DEV), torch.tensor([float("inf")], device=DEV),
                torch.tensor([0.5, float("nan")], device=DEV).to(torch.float16)):
        assert not qutils.all_valid_scales(good + [bad])
        with pytest.raises(AssertionError, match="negative, inf or nan"):
            with qutils.deferred_scale_checks():
                qutils.all_valid_scales(good + [bad])
    with pytest.raises(AssertionError, match="should be positive"):
        with qutils.deferred_scale_checks():
            qutils.all_positive(torch.tensor([1.0, 0.0], device=DEV))
    with qutils.deferred_scale_checks() as checks:
        checks.report = [torch.tensor([-1.0], device=DEV)]
    assert not checks.report_ok


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("alpha", [0.5, 0.3, 1.0, 0.0])
@pytest.mark.parametrize("case", ["plain", "dead channels", "nan"])
def test_smoothquant_in_one_launch_equals_the_tensor_expressions(dtype, alpha, case, monkeypatch):
    """mo_smooth_scales against the eager postprocess of smoothquant (model_calib.py:447-473 and
    384-407 of the reference): pre-quant scale, input amax and folded weight bit for bit, for the
    exponents the scalar pow special-cases and one it does not, with channels that never fired
    (their scale is reset to 1) and with a NaN in the statistics."""
    from modelopt_amd.torch.quantization import model_calib

    g = torch.Generator().manual_seed(int(alpha * 10) + len(case))
    k, n = 512, 256
    w = (0.05 * torch.randn(n, k, generator=g)).to(dtype)
    x = (torch.randn(64, k, generator=g) * torch.exp(torch.randn(k, generator=g))).to(dtype)
    if case != "plain":
        x[:, 5] = 0
        x[:, 77] = 0
        w[:, 9] = 0
    if case == "nan":
        x[3, 100] = float("nan")

    def run(one_launch):
        monkeypatch.setattr(model_calib, "_SMOOTH_IN_ONE_LAUNCH", one_launch)
        model = nn.Sequential(nn.Linear(k, n, bias=False)).to(dtype).to(DEV)
        model[0].weight.data.copy_(w)
        cfg = copy.deepcopy(mtq.INT8_SMOOTHQUANT_CFG)
        cfg["algorithm"] = {"method": "smoothquant", "alpha": alpha}
        try:
            mtq.quantize(model, cfg, lambda m: m(x.to(DEV)))
        except AssertionError as e:   # the deferred checks refuse a NaN scale either way
            return str(e)
        q = model[0].input_quantizer
        return (q.pre_quant_scale.clone(), q.amax.clone(), model[0].weight.data.clone(),
                model[0].weight_quantizer.amax.clone(), q._amax_for_smoothing.clone())

    eager, fused = run(False), run(True)
    if isinstance(eager, str):
        assert eager == fused
        return
    for a, b in zip(eager, fused):
        assert a.dtype == b.dtype and a.shape == b.shape
        assert_bits_equal(a.cpu(), b.cpu(), f"{dtype} alpha {alpha} {case}")


def test_work_goes_to_the_caller_s_current_stream():
    """Kernels are enqueued on the stream that is current when the operator is called: the input
    here is produced late on a side stream (behind a few milliseconds of GEMMs) and consumed on
    that stream without a synchronisation; on any other stream the kernels would read it before it
    exists.  Results against the CPU restatement."""
    from modelopt_amd import _hip
    from modelopt_amd.torch.quantization.utils import reduce_amax

    side = torch.cuda.Stream(device=DEV)
    g = torch.Generator().manual_seed(77)
    host = (torch.randn(2048, 2048, generator=g) * 0.05).to(torch.bfloat16)
    staged = host.to(DEV)
    x = torch.zeros_like(staged)
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        busy = torch.randn(8192, 8192, device=DEV, dtype=torch.bfloat16)
        for _ in range(6):
            busy = (busy @ busy.T) * 1e-2
        x.copy_(staged + (busy[:2048, :2048] * 0).nan_to_num(0.0, 0.0, 0.0))   # depends on the GEMMs
        amax = reduce_amax(x)
        qt, wsf, wsf2 = NVFP4QTensor.quantize(x, 16)
        y = _hip.fp8_qdq(x, amax, 1, 1, x.numel())
        cols = torch.zeros(2048, dtype=torch.float32, device=DEV)
        _hip.absmax_into(x, cols, 2048, 2048, 1)
    side.synchronize()
    assert_bits_equal(amax.cpu(), reduce.reduce_amax(host), "abs-max on the side stream")
    p_o, w_o, _ = qtensor.nvfp4_quantize(host, 16)
    assert_bits_equal(qt._quantized_data.cpu(), p_o, "codes on the side stream")
    assert_bits_equal(wsf.cpu().view(torch.uint8), w_o.view(torch.uint8), "block scales on the side stream")
    assert_bits_equal(y.cpu(), fake_quant.fp8_eager(host, reduce.reduce_amax(host)), "fp8 fake quant on the side stream")
    assert_bits_equal(cols.cpu(), host.abs().amax(dim=0).float(), "per-column abs-max on the side stream")


@pytest.mark.parametrize("tokens", [96, 700])
def test_awq_lite_on_a_layer_with_a_bias_takes_the_search_kernel(tokens, monkeypatch):
    """A linear with a bias goes through the one-launch search (its bias added in the kernel's
    epilogue) and ends where the per-alpha route ends: same alpha, losses within 1e-3, the same
    folded weight and input scale bit for bit."""
    from modelopt_amd.torch.quantization import model_calib

    g = torch.Generator().manual_seed(23)
    ref = _OneLinear(n=256, k=384, seed=23)
    ref.proj.bias = nn.Parameter((0.2 * torch.randn(256, generator=g)).to(torch.bfloat16))
    c = torch.exp(torch.randn(384, generator=g))
    batches = [(torch.randn(tokens, 384, generator=g) * c).to(torch.bfloat16) for _ in range(2)]
    cfg = copy.deepcopy(mtq.INT4_AWQ_CFG)
    cfg["algorithm"] = {"method": "awq_lite", "alpha_step": 0.1, "debug": True}
    results = []
    for one_launch in (True, False):
        model = copy.deepcopy(ref).to(DEV)
        taken = []
        real = model_calib._one_launch_search
        if one_launch:
            monkeypatch.setattr(model_calib, "_one_launch_search",
                                lambda *a: taken.append(real(*a)) or taken[-1])
        else:
            monkeypatch.setattr(model_calib, "_one_launch_search", lambda *a: False)
        mtq.quantize(model, copy.deepcopy(cfg), lambda m: [m(b.to(DEV)) for b in batches])
        monkeypatch.setattr(model_calib, "_one_launch_search", real)
        assert not one_launch or taken == [True, True]
        results.append((model.proj.awq_lite, model.proj.weight.detach().clone(),
                        model.proj.input_quantizer.pre_quant_scale.clone()))
    (fast, w_fast, p_fast), (slow, w_slow, p_slow) = results
    assert fast.best_alpha == slow.best_alpha
    for a in slow.loss:
        assert fast.loss[a] == pytest.approx(slow.loss[a], rel=1e-3), f"alpha {a}"
    assert_bits_equal(w_fast.cpu(), w_slow.cpu(), "folded weight")
    assert_bits_equal(p_fast.cpu(), p_slow.cpu(), "input scale")


@pytest.mark.parametrize("cfg_name", ["NVFP4_AWQ_LITE_CFG", "W4A8_AWQ_BETA_CFG"])
def test_awq_lite_lean_per_alpha_route_equals_the_route_through_the_module(cfg_name, monkeypatch):
    """Weight quantizers the search kernel does not cover (NVFP4 blocks, the INT4 + FP8 pair) are
    scored alpha by alpha; for a plain quantised linear that loop scales the columns itself and
    calls the three quantizers directly instead of writing pre-quant scales onto them and going
    through the module's forward.  Same kernels on the same values: every per-alpha loss, the
    folded weight and the input scale are bit for bit what the route through the module gives."""
    from modelopt_amd.torch.quantization import model_calib

    g = torch.Generator().manual_seed(29)
    ref = _OneLinear(n=256, k=384, seed=29)
    c = torch.exp(torch.randn(384, generator=g))
    batches = [(torch.randn(70, 384, generator=g) * c).to(torch.bfloat16) for _ in range(2)]
    cfg = copy.deepcopy(getattr(mtq, cfg_name))
    algorithm = cfg["algorithm"] if isinstance(cfg["algorithm"], dict) else {"method": cfg["algorithm"]}
    cfg["algorithm"] = {**algorithm, "debug": True}
    results = []
    for lean in (True, False):
        if not lean:
            monkeypatch.setattr(model_calib, "_QuantLinear", type("Other", (), {"forward": None}))
        model = copy.deepcopy(ref).to(DEV)
        mtq.quantize(model, copy.deepcopy(cfg), lambda m: [m(b.to(DEV)) for b in batches])
        results.append((model.proj.awq_lite, model.proj.weight.detach().clone(),
                        model.proj.input_quantizer.pre_quant_scale.clone()))
    (fast, w_fast, p_fast), (slow, w_slow, p_slow) = results
    assert fast.loss == slow.loss and fast.best_alpha == slow.best_alpha
    assert_bits_equal(w_fast.cpu(), w_slow.cpu(), "folded weight")
    assert_bits_equal(p_fast.cpu(), p_slow.cpu(), "input scale")
