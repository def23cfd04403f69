"""MSE amax search on the GPU (one-pass kernel and per-candidate route) against the CPU
restatement of the reference's MseCalibrator."""

import copy

import pytest
import torch
from torch import nn

import modelopt_amd.torch.quantization as mtq
from conftest import assert_bits_equal
from modelopt_amd import _hip
from modelopt_amd.torch.quantization.calib import MseCalibrator
from modelopt_amd.torch.quantization.config import QuantizerAttributeConfig
from modelopt_amd.torch.quantization.nn import TensorQuantizer
from oracle import fake_quant, mse, reduce

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
LOSS_RTOL = 2e-5      # fp32 sums in a different order than torch.sum


def _batches(shape, dtype, n=2, seed=51):
    g = torch.Generator().manual_seed(seed)
    out = []
    for _ in range(n):
        x = torch.randn(shape, generator=g)
        x.view(-1)[torch.randperm(x.numel(), generator=g)[: x.numel() // 200]] *= 8   # outliers
        out.append(x.to(dtype))
    return out


def _calibrated_quantizer(cfg, batches):
    q = TensorQuantizer(QuantizerAttributeConfig(**cfg)).to(DEV)
    q.enable_calib(); q.disable_quant()
    for x in batches:
        q(x.to(DEV))
    q.load_calib_amax(); q.disable_calib(); q.enable_quant()
    return q


def _oracle_quant(cfg):
    if cfg["num_bits"] == (4, 3):
        return lambda x, amax: fake_quant.fp8_eager(x, amax)
    return lambda x, amax: fake_quant.tensor_quant(x, amax, cfg["num_bits"], cfg.get("unsigned", False),
                                                   cfg.get("narrow_range", False))


CASES = [
    ("int8_tensor", {"num_bits": 8, "axis": None}, (96, 512)),
    ("int4_tensor_3d", {"num_bits": 4, "axis": None}, (4, 33, 64)),
    ("int8_rows", {"num_bits": 8, "axis": 0}, (192, 1024)),
    ("int4_rows_narrow", {"num_bits": 4, "axis": 0, "narrow_range": True}, (64, 264)),
    ("fp8_tensor", {"num_bits": (4, 3), "axis": None}, (128, 256)),
    ("int8_tensor_odd", {"num_bits": 8, "axis": None}, (7, 13)),
]


@pytest.mark.parametrize("name,cfg,shape", CASES, ids=[c[0] for c in CASES])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.usefixtures("cpu_fp8_overflow")
def test_mse_calibrator_against_oracle(name, cfg, shape, dtype, fused, monkeypatch):
    batches = _batches(shape, dtype)
    q = _calibrated_quantizer(cfg, batches)
    initial = q._amax.clone()
    axis = q._calibrator._axis
    ref_initial = torch.stack([reduce.reduce_amax(
        x, axis=reduce.quant_axis_to_reduce_dims(x, axis)) for x in batches]).amax(0)
    assert_bits_equal(initial.cpu().reshape(ref_initial.shape), ref_initial, "initial amax")

    def quant_func(x, amax):
        saved = q._amax
        q._amax = amax
        try:
            return q(x)
        finally:
            q._amax = saved

    cal = MseCalibrator(initial, axis=axis, num_steps=10, quant_func=quant_func, quantizer=q)
    if not fused:
        monkeypatch.setattr(cal, "_fused_spec", lambda: None)
    elif name == "fp8_tensor":
        # quarter-amax candidates overflow E4M3; the kernel follows the quantizer's NaN-on-overflow
        pass
    for x in batches:
        cal.collect(x.to(DEV))
    want_losses, want_amax = mse.mse_search(batches, ref_initial.reshape(initial.shape), axis,
                                            _oracle_quant(cfg))
    got_losses = torch.stack([l.reshape(want_losses.shape[1:]) for l in cal._losses_sum]).cpu()
    finite = torch.isfinite(want_losses)
    assert torch.equal(torch.isfinite(got_losses), finite)
    assert torch.allclose(got_losses[finite], want_losses[finite], rtol=LOSS_RTOL, atol=0)
    got = cal.compute_amax()
    if finite.all():
        assert_bits_equal(got.cpu(), want_amax, "best amax")
    for k in range(10):
        assert_bits_equal(cal._candidate_amaxs[k].cpu(),
                          mse.candidates(ref_initial.reshape(initial.shape))[k], f"candidate {k}")


def test_fused_kernel_is_taken_and_falls_back_where_it_cannot_run():
    x = _batches((64, 128), torch.bfloat16, 1)[0].to(DEV)
    cand = torch.full((3, 1), 2.0, device=DEV)
    loss = torch.zeros_like(cand)
    assert _hip.qdq_sq_err_into(x, cand, loss, 1, 1, x.numel(), kind="int", num_bits=8)
    assert (loss > 0).all()
    # per-channel along the last dim: not a layout of the kernel
    cand = torch.full((3, 128), 2.0, device=DEV)
    assert not _hip.qdq_sq_err_into(x, cand, torch.zeros_like(cand), 64, 128, 1, kind="int", num_bits=8)
    # 17 candidates: two launches
    cand = torch.linspace(0.5, 4.0, 17, device=DEV).reshape(17, 1).contiguous()
    loss = torch.zeros_like(cand)
    assert _hip.qdq_sq_err_into(x, cand, loss, 1, 1, x.numel(), kind="int", num_bits=8)
    xc = x.cpu().float()
    for k in range(17):
        want = ((xc - fake_quant.tensor_quant(xc, cand[k].cpu().reshape(()), 8, False, False)) ** 2).sum()
        assert loss[k].item() == pytest.approx(want.item(), rel=LOSS_RTOL)


class _Net(nn.Module):
    def __init__(self):
        super().__init__()
        g = torch.Generator().manual_seed(7)
        self.fc = nn.Linear(256, 128, bias=False)
        self.fc.weight.data = 0.05 * torch.randn(128, 256, generator=g)
        self.fc.weight.data[3, 5] = 1.0          # an outlier that clipping should cut off
        self.to(torch.bfloat16)

    def forward(self, x):
        return self.fc(x)


def test_quantize_with_mse_algorithm():
    ref = _Net()
    model = copy.deepcopy(ref).to(DEV)
    batches = _batches((32, 256), torch.bfloat16, 3, seed=52)
    cfg = copy.deepcopy(mtq.INT8_DEFAULT_CFG)
    cfg["algorithm"] = {"method": "mse", "num_steps": 8, "start_multiplier": 0.3, "stop_multiplier": 1.5}
    mtq.quantize(model, cfg, lambda m: [m(b.to(DEV)) for b in batches])
    w = ref.fc.weight.data
    w_init = reduce.reduce_amax(w, axis=[1])
    _, w_amax = mse.mse_search([w], w_init, 0, lambda x, a: fake_quant.tensor_quant(x, a, 8, False, False),
                               8, 0.3, 1.5)
    assert_bits_equal(model.fc.weight_quantizer.amax.cpu(), w_amax, "weight amax")
    x_init = torch.stack([reduce.reduce_amax(b) for b in batches]).amax()
    _, x_amax = mse.mse_search(batches, x_init, None,
                               lambda x, a: fake_quant.tensor_quant(x, a, 8, False, False), 8, 0.3, 1.5)
    # the fp32 winner is copied into the bf16 buffer that max calibration created
    assert_bits_equal(model.fc.input_quantizer.amax.cpu().reshape(()),
                      x_amax.to(torch.bfloat16).reshape(()), "input amax")
    assert model.fc.weight_quantizer.amax[3].cpu() < w_init[3]  # the outlier row was clipped
    assert model.fc.input_quantizer._if_quant and not model.fc.input_quantizer._if_calib
    model(batches[0].to(DEV))


def test_mse_refuses_static_blocks():
    model = _Net().to(DEV)
    cfg = copy.deepcopy(mtq.INT4_BLOCKWISE_WEIGHT_ONLY_CFG)
    cfg["algorithm"] = "mse"
    with pytest.raises(ValueError, match="static block"):
        mtq.quantize(model, cfg, lambda m: m(_batches((4, 256), torch.bfloat16, 1)[0].to(DEV)))
