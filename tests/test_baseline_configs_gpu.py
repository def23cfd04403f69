"""The single-tensor benchmark configurations at their full shapes, through the public host API,
against the CPU restatements: FP8 calibrate + fake quant of a 4096 x 4096 weight with outliers,
AWQ-lite over 21 alphas on a 4096 x 4096 linear, NVFP4 dynamic fake quant and SmoothQuant + INT8
on 8192 x 8192 activations."""

import copy

import pytest
import torch
from torch import nn

import modelopt_amd.torch.quantization as mtq
from conftest import assert_bits_equal
from oracle import awq as oawq
from oracle import cref, fake_quant, reduce

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


class _OneLinear(nn.Module):
    def __init__(self, weight):
        super().__init__()
        self.proj = nn.Linear(weight.shape[1], weight.shape[0], bias=False)
        self.proj.weight.data = weight.clone()

    def forward(self, x):
        return self.proj(x)


def test_fp8_calibrate_and_fake_quant_4096_square_with_outliers():
    g = torch.Generator().manual_seed(1)
    w = 0.02 * torch.randn(4096, 4096, generator=g)
    w.view(-1)[torch.randperm(w.numel(), generator=g)[:16777]] *= 50     # 0.1 % outliers
    w = w.to(torch.bfloat16)
    x = torch.randn(64, 4096, generator=g).to(torch.bfloat16)
    model = _OneLinear(w).to(torch.bfloat16).to(DEV)
    mtq.quantize(model, mtq.FP8_DEFAULT_CFG, lambda m: m(x.to(DEV)))
    amax = reduce.reduce_amax(w)
    assert_bits_equal(model.proj.weight_quantizer.amax.cpu().reshape(()), amax.reshape(()), "weight amax")
    got = model.proj.weight_quantizer(model.proj.weight.data).cpu()
    assert_bits_equal(got, fake_quant.fp8_eager(w, amax), "fp8 fake quant vs torch restatement")
    assert_bits_equal(got, cref.fp8_qdq(w, amax), "fp8 fake quant vs C restatement")
    xq = model.proj.input_quantizer(x.to(DEV)).cpu()
    assert_bits_equal(xq, fake_quant.fp8_eager(x, reduce.reduce_amax(x)), "input fake quant")


def test_awq_lite_21_alphas_on_4096_square_linear():
    g = torch.Generator().manual_seed(3)
    w = (0.02 * torch.randn(4096, 4096, generator=g)).to(torch.bfloat16)
    c = torch.exp(torch.randn(4096, generator=g))
    c[torch.randperm(4096, generator=g)[:41]] *= 20                      # 1 % hot channels
    x = (torch.randn(512, 4096, generator=g) * c).to(torch.bfloat16)
    model = _OneLinear(w).to(torch.bfloat16).to(DEV)
    cfg = copy.deepcopy(mtq.INT4_AWQ_CFG)
    cfg["algorithm"] = {"method": "awq_lite", "alpha_step": 0.05, "debug": True}
    mtq.quantize(model, cfg, lambda m: m(x.to(DEV)))
    losses, best_alpha, _, act_scale, weight_scale = oawq.awq_lite_search(w, [x], 0.05, 128)
    h = model.proj.awq_lite
    assert list(h.loss) == list(losses) and len(losses) == 21
    for a in losses:
        assert h.loss[a] == pytest.approx(losses[a], rel=1e-3), f"alpha {a}"   # tolerance of the task
    assert h.best_alpha == best_alpha
    assert torch.allclose(h.act_scale.cpu(), act_scale, rtol=2 ** -7)
    assert torch.allclose(h.weight_scale.cpu(), weight_scale, rtol=2 ** -7)
    pqs, w_new = oawq.fold_pre_quant_scale(w, 1.0 / h.best_scale.cpu())
    assert_bits_equal(model.proj.input_quantizer._pre_quant_scale.cpu(), pqs, "pre_quant_scale")
    assert_bits_equal(model.proj.weight.data.cpu(), w_new, "folded weight")
    # the quantised weight the GEMM would see: INT4 block-128 fake quant of the folded weight
    got = model.proj.weight_quantizer(model.proj.weight.data).cpu()
    assert_bits_equal(got, oawq.int4_block_qdq(w_new, 128), "int4 block fake quant")


def _activations_8192():
    g = torch.Generator().manual_seed(4)
    return (torch.randn(8192, 8192, generator=g) * torch.exp(1.5 * torch.randn(8192, generator=g))[None, :]
            ).to(torch.bfloat16)


def test_nvfp4_dynamic_fake_quant_on_8192_square_activations():
    x = _activations_8192()
    q = mtq.nn.TensorQuantizer(mtq.config.QuantizerAttributeConfig(
        **mtq.NVFP4_DEFAULT_CFG["quant_cfg"]["*input_quantizer"])).to(DEV)
    xd = x.to(DEV)
    q.enable_calib(); q.disable_quant()
    q(xd)
    q.load_calib_amax(); q.disable_calib(); q.enable_quant()
    amax = reduce.reduce_amax(x)
    assert_bits_equal(q.amax.cpu().reshape(()), amax.reshape(()), "amax")
    got = q(xd).cpu()
    for r0 in range(0, 8192, 1024):                                      # row slabs bound the CPU memory
        want = fake_quant.nvfp4_fake_quant(x[r0:r0 + 1024], amax, 16)
        assert_bits_equal(got[r0:r0 + 1024], want, f"nvfp4 fake quant, rows {r0}..{r0 + 1023}")
    # every block's values lie on its own grid: at most 8 distinct magnitudes per 16 elements
    mags = got.float().abs().reshape(-1, 16)
    distinct = (mags.sort(dim=1).values.diff(dim=1) != 0).sum(dim=1) + 1
    assert int(distinct.max()) <= 8


def test_smoothquant_int8_on_8192_square():
    x = _activations_8192()
    g = torch.Generator().manual_seed(5)
    w = (0.02 * torch.randn(8192, 8192, generator=g)).to(torch.bfloat16)
    model = _OneLinear(w).to(torch.bfloat16).to(DEV)
    cfg = copy.deepcopy(mtq.INT8_SMOOTHQUANT_CFG)
    cfg["algorithm"] = {"method": "smoothquant", "alpha": 0.5}
    mtq.quantize(model, cfg, lambda m: m(x.to(DEV)))
    act_amax = reduce.reduce_amax(x, axis=[0])
    pqs, w_new, in_amax, w_amax = oawq.smoothquant_linear(w, act_amax, alpha=0.5)
    lin = model.proj
    assert_bits_equal(lin.input_quantizer._pre_quant_scale.cpu().reshape(-1), pqs.reshape(-1), "pre_quant_scale")
    assert_bits_equal(lin.weight.data.cpu(), w_new, "smoothed weight")
    assert_bits_equal(lin.input_quantizer.amax.cpu().reshape(()), in_amax.reshape(()), "input amax")
    assert_bits_equal(lin.weight_quantizer.amax.cpu().reshape(w_amax.shape), w_amax, "weight amax")
    # what the GEMM sees: x * pre_quant_scale -> INT8 per-tensor fake quant; weight per-row INT8
    xq = lin.input_quantizer(x.to(DEV)).cpu()
    want = fake_quant.tensor_quant((x * pqs.reshape(1, -1)), in_amax, 8, False, False)
    want = want[0] if isinstance(want, tuple) else want
    assert_bits_equal(xq, want.to(torch.bfloat16), "smoothed input fake quant")
    wq = lin.weight_quantizer(lin.weight.data).cpu()
    want_w = fake_quant.tensor_quant(w_new, w_amax, 8, False, False)
    want_w = want_w[0] if isinstance(want_w, tuple) else want_w
    assert_bits_equal(wq, want_w.to(torch.bfloat16), "smoothed weight fake quant")
