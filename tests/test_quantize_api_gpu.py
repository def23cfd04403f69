"""``mtq.quantize`` API behaviours the reference's own unit tests pin
(tests/unit/torch/quantization/test_quantize_cpu.py:126-260), on the GPU."""

import copy

import pytest
import torch

import modelopt_amd.torch.quantization as mtq
from modelopt_amd.torch.quantization.calib import MaxCalibrator

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


class SimpleLinear(torch.nn.Module):
    """the shape of tests/_test_utils/torch/quantization/models.py SimpleLinear"""

    def __init__(self):
        super().__init__()
        torch.manual_seed(0)
        self.net = torch.nn.Sequential(torch.nn.Linear(16, 32), torch.nn.ReLU(),
                                       torch.nn.Linear(32, 64), torch.nn.ReLU(), torch.nn.Linear(64, 16))

    def forward(self, x):
        return self.net(x)

    def get_input(self):
        return torch.randn(2, 16, device=DEV)


def test_invalid_cfg_message():
    """:126-133"""
    cfg = {"quant_cfg": {"*": {"num_bits": 4, "axis": 0, "block_sizes": {-1: 128}}}, "algorithm": "max"}
    with pytest.raises(Exception, match="axis must be None when block_sizes is not None."):
        mtq.quantize(SimpleLinear().to(DEV), cfg)


def test_forward_loop_without_arguments_still_works():
    """:136-144: the older calling convention, with a deprecation warning"""
    model = SimpleLinear().to(DEV)
    data = [model.get_input() for _ in range(2)]

    def forward_loop():
        for batch in data:
            model(batch)

    with pytest.warns(DeprecationWarning):
        mtq.quantize(model, mtq.INT8_DEFAULT_CFG, forward_loop=forward_loop)
    want = torch.stack([b.abs().max() for b in data]).max()
    assert torch.equal(model.net[0].input_quantizer.amax.reshape(()), want)


class DoublingMaxCalibrator(MaxCalibrator):
    def compute_amax(self):
        return 2 * self._calib_amax


def test_custom_calibrator_from_a_config_tuple():
    """:73-88, :147-162: ``"calibrator": (class, args)``; the subclass reads ``_calib_amax``"""
    cfg = {"quant_cfg": {"*": {"num_bits": 4, "axis": None, "enable": True,
                               "calibrator": (DoublingMaxCalibrator, (4, None, False))}},
           "algorithm": "max"}
    model = SimpleLinear().to(DEV)
    mtq.quantize(model, cfg, lambda m: m(m.get_input()))
    for name, module in model.named_modules():
        if name.endswith("quantizer"):
            assert type(module._calibrator) is DoublingMaxCalibrator, name
    w = model.net[0].weight
    assert torch.equal(model.net[0].weight_quantizer.amax.reshape(()), 2 * w.abs().max())


def test_class_wise_config():
    """:165-194: a key that names a module class scopes its patterns to that class"""
    cfg = {"quant_cfg": {"nn.Linear": {"*": {"num_bits": 4, "axis": -1, "enable": True}},
                         "*output_quantizer": {"num_bits": 8, "enable": True}},
           "algorithm": "max"}
    model = SimpleLinear().to(DEV)
    mtq.quantize(model, cfg, lambda m: m(m.get_input()))
    for name, module in model.named_modules():
        if isinstance(module, torch.nn.Linear):
            for q in (module.weight_quantizer, module.input_quantizer):
                assert q.num_bits == 4 and q.axis == -1 and q.is_enabled
        if name.endswith("output_quantizer"):
            assert module.is_enabled and module.num_bits == 8


def test_static_weights_with_dynamic_per_token_activations():
    """:56-70, :197-215: dynamic input quantizers need no forward loop; weights are calibrated
    even when none is given"""
    cfg = {"quant_cfg": {"*weight_quantizer": {"num_bits": 8, "axis": 0},
                         "*input_quantizer": {"num_bits": 8, "axis": (0, 1), "type": "dynamic"},
                         "default": {"enable": False}},
           "algorithm": "max"}
    model = SimpleLinear().to(DEV)
    mtq.quantize(model, cfg, lambda m: m(m.get_input()))
    assert all(m.amax is not None for n, m in model.named_modules() if n.endswith("weight_quantizer"))
    assert torch.isfinite(model(model.get_input())).all()
    model = SimpleLinear().to(DEV)
    mtq.quantize(model, cfg)
    for name, module in model.named_modules():
        if name.endswith("weight_quantizer"):
            assert module.amax is not None, name
        if name.endswith("input_quantizer"):
            assert module.amax is None, name


def test_block_sizes_that_name_whole_axes_equal_the_axis_form():
    """:218-262: ``block_sizes: {1: None}`` is per-channel along axis 0, ``{0: None, 1: None}``
    per tensor"""
    ref_cfg = {"quant_cfg": {"*weight_quantizer": {"num_bits": 8, "axis": 0},
                             "*input_quantizer": {"num_bits": 8, "axis": None, "type": "dynamic"},
                             "default": {"enable": False}},
               "algorithm": "max"}
    cfg = {"quant_cfg": {"*weight_quantizer": {"num_bits": 8, "block_sizes": {1: None}},
                         "*input_quantizer": {"num_bits": 8, "block_sizes": {0: None, 1: None}, "type": "dynamic"},
                         "default": {"enable": False}},
           "algorithm": "max"}
    model_ref = SimpleLinear().to(DEV)
    model = copy.deepcopy(model_ref)
    x = model_ref.get_input()
    mtq.quantize(model_ref, ref_cfg, lambda m: m(x))
    mtq.quantize(model, cfg, lambda m: m(x))
    assert torch.equal(model_ref(x), model(x))
    for (name, a), (_, b) in zip(model_ref.named_modules(), model.named_modules()):
        if getattr(a, "amax", None) is not None:
            assert torch.equal(a.amax, b.amax.reshape(a.amax.shape)), name


# ------------------------------------------------------------------ calibration algorithms
# tests/unit/torch/quantization/test_calib.py:280-359
class SimpleMLP(torch.nn.Module):
    def __init__(self, fi=16, f1=32, f2=16, fo=16):
        super().__init__()
        self.net = torch.nn.Sequential(torch.nn.Linear(fi, f1, bias=False), torch.nn.ReLU(),
                                       torch.nn.Linear(f1, f2, bias=False), torch.nn.ReLU(),
                                       torch.nn.Linear(f2, fo, bias=False))

    def forward(self, x):
        return self.net(x)


def _awq_config(algorithm, block_size=8):
    cfg = copy.deepcopy(mtq.INT4_AWQ_CFG)
    cfg["quant_cfg"]["*weight_quantizer"]["block_sizes"] = {-1: block_size}
    cfg["algorithm"] = {"method": algorithm, "debug": True}
    if algorithm != "awq_clip":
        cfg["algorithm"]["alpha_step"] = 0.1
    return cfg


def _loop(batches):
    def run(model):
        for b in batches:
            model(b)
    return run


def test_awq_one_batch_equals_the_same_data_in_four():
    """:280-302: the search sums over batches, so splitting the data must not change the scales"""
    torch.manual_seed(0)
    model = SimpleMLP().to(DEV)
    states = model.state_dict()
    batches = [torch.randn(2, 16, 16, device=DEV) for _ in range(4)]
    single = [torch.cat(batches, dim=0)]
    scales = []
    for data in (single, batches):
        m = SimpleMLP().to(DEV)
        m.load_state_dict(states)
        mtq.quantize(m, _awq_config("awq_full"), _loop(data))
        scales.append([m.net[i].awq_lite.best_scale for i in (0, 2, 4)])
    for a, b in zip(*scales):
        assert torch.allclose(a, b)


def test_awq_with_padded_blocks():
    """:305-310: feature counts the block size does not divide"""
    torch.manual_seed(0)
    model = SimpleMLP(f1=13, f2=19).to(DEV)
    mtq.quantize(model, _awq_config("awq_full"), _loop([torch.randn(2, 16, 16, device=DEV)]))
    assert torch.isfinite(model(torch.randn(2, 16, 16, device=DEV))).all()


def test_smoothquant_can_be_undone_and_redone():
    """:313-344: disable_pre_quant_scale_and_resmooth gives the plain INT8 model's outputs,
    apply_pre_quant_scale_and_smooth brings the smoothed ones back"""
    from modelopt_amd.torch.quantization.model_calib import (apply_pre_quant_scale_and_smooth,
                                                              disable_pre_quant_scale_and_resmooth)

    torch.manual_seed(1234)
    model = SimpleMLP().to(DEV)
    data = [torch.randn(2, 16, 16, device=DEV)]
    x = torch.randn(2, 16, 16, device=DEV)
    plain = SimpleMLP().to(DEV)
    plain.load_state_dict(model.state_dict())
    mtq.quantize(model, mtq.INT8_SMOOTHQUANT_CFG, _loop(data))
    mtq.quantize(plain, mtq.INT8_DEFAULT_CFG, _loop(data))
    out_sq = model(x)
    for module in model.modules():
        if isinstance(module, torch.nn.Linear):
            disable_pre_quant_scale_and_resmooth(module)
            assert module.input_quantizer.pre_quant_scale is None
    assert torch.allclose(model(x), plain(x))
    for module in model.modules():
        if isinstance(module, torch.nn.Linear):
            apply_pre_quant_scale_and_smooth(module)
            assert module.input_quantizer.pre_quant_scale is not None
    assert torch.allclose(model(x), out_sq)


def test_postprocess_amax():
    """:347-358"""
    torch.manual_seed(0)
    model = SimpleMLP().to(DEV)
    mtq.quantize(model, mtq.INT8_DEFAULT_CFG, _loop([torch.randn(2, 16, 16, device=DEV)]))
    mtq.postprocess_amax(model, "*input_quantizer", lambda amax: torch.clamp(amax, max=0.5))
    for name, module in model.named_modules():
        if isinstance(module, mtq.nn.TensorQuantizer) and name.endswith("input_quantizer"):
            assert module.amax.amax() <= 0.5
