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
