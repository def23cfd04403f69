"""Host-layer logic on CPU: configs, conversion, wildcards, block reshaping, export helpers.

Orchestration tests swap the kernel facade for the CPU oracle (``oracle_backend`` fixture): the
oracle is the stand-in for the HIP library here, exactly so that the Python control flow can be
exercised without a GPU.  The product itself never does this -- see ``test_cpu_tensors_raise``.
"""

import copy

import pytest
import torch
import torch.nn.functional as F
from torch import nn

import modelopt_amd.torch.quantization as mtq
from modelopt_amd.torch.export import quant_utils as equ
from modelopt_amd.torch.quantization import kernels
from modelopt_amd.torch.quantization.config import QuantizerAttributeConfig, normalize_algorithm
from modelopt_amd.torch.quantization.nn import SequentialQuantizer, TensorQuantizer
from oracle import fake_quant, mx, reduce


# ----------------------------------------------------------------------------- config
def test_attribute_config_defaults_and_mapping_protocol():
    c = QuantizerAttributeConfig()
    assert c.num_bits == 8 and c.axis is None and c.fake_quant and not c.narrow_range and c.enable
    assert dict(c.items())["calibrator"] == "max" and "block_sizes" in c
    assert c["type"] == "static"


@pytest.mark.parametrize("bad", [
    {"enable": True},
    {"num_bits": 0},
    {"num_bits": (7, 7)},
    {"num_bits": (2, 1)},                                    # FP4 needs dynamic block sizes
    {"num_bits": 8, "axis": 0, "block_sizes": {-1: 128}},     # axis and block_sizes exclude each other
    {"block_sizes": {-1: 16, -2: 16, "type": "dynamic"}},    # dynamic = last axis only
    {"block_sizes": {"bogus": 1}},
    {"type": "sometimes"},
    {"bias": {"type": "static"}},
])
def test_attribute_config_rejects(bad):
    with pytest.raises(Exception):
        QuantizerAttributeConfig(**bad)


def test_named_configs_validate():
    for name in mtq.config.choices:
        quant_cfg, algo = mtq.model_quant._validated(getattr(mtq, name))
        assert "default" in quant_cfg and isinstance(quant_cfg["default"], QuantizerAttributeConfig)
    assert normalize_algorithm("max") == ("max", {"distributed_sync": True})
    assert normalize_algorithm({"method": "awq_lite", "alpha_step": 0.05})[1]["alpha_step"] == 0.05
    assert normalize_algorithm(None) == (None, {})
    with pytest.raises(NotImplementedError):
        normalize_algorithm("svdquant")


# ----------------------------------------------------------------------------- conversion
class _Net(nn.Module):
    def __init__(self):
        super().__init__()
        self.body = nn.Sequential(nn.Linear(16, 32), nn.ReLU(), nn.Linear(32, 16))
        self.lm_head = nn.Linear(16, 8)

    def forward(self, x):
        return self.lm_head(self.body(x))


def _converted(cfg):
    m = _Net()
    mtq.replace_quant_module(m)
    mtq.set_quantizer_by_cfg(m, mtq.model_quant._validated(cfg)[0])
    return m


class _NetWithNorm(_Net):
    def __init__(self):
        super().__init__()
        self.norm = nn.BatchNorm1d(16)      # the named configs carry entries scoped to nn classes
        self.mlp = nn.Sequential(nn.Linear(16, 16))


def _quantizer_state(model):
    keep = ("_num_bits", "_axis", "_block_sizes", "_disabled", "_dynamic", "_unsigned", "_narrow_range",
            "_fake_quant", "_learn_amax", "_trt_high_precision_dtype", "_bias", "_rotate", "_pass_through_bwd")
    out = {}
    for name, q in model.named_modules():
        if isinstance(q, TensorQuantizer):
            out[name] = {k: getattr(q, k, None) for k in keep}
            out[name]["calibrator"] = type(q._calibrator).__name__
    return out


def test_single_pass_configuration_equals_entry_by_entry():
    """With complete attribute sets only, each quantizer takes the last entry that matches it;
    an entry with a filter function in place of a wildcard sends the same config through the
    entry-by-entry route, and both must leave every quantizer in the same state."""
    for name in mtq.config.choices:
        quant_cfg, _ = mtq.model_quant._validated(getattr(mtq, name))
        if any(isinstance(v, list) for v in quant_cfg.values()):
            continue     # lists build SequentialQuantizers: entry-by-entry either way
        a, b = _NetWithNorm(), _NetWithNorm()
        mtq.replace_quant_module(a)
        mtq.replace_quant_module(b)
        mtq.set_quantizer_by_cfg(a, quant_cfg)
        slow = dict(quant_cfg)
        slow[lambda n: False] = quant_cfg["default"]       # matches nothing, forces the other route
        mtq.set_quantizer_by_cfg(b, slow)
        assert _quantizer_state(a) == _quantizer_state(b), name


def test_conversion_adds_quantizers_and_keeps_parameters():
    m = _Net()
    w = m.body[0].weight
    mtq.replace_quant_module(m)
    assert m.body[0].weight is w and isinstance(m.body[0], nn.Linear)
    assert type(m.body[0]).__name__ == "QuantLinear"
    for lin in (m.body[0], m.body[2], m.lm_head):
        assert {"input_quantizer", "weight_quantizer", "output_quantizer"} <= dict(lin.named_children()).keys()
        assert not lin.output_quantizer.is_enabled
    with pytest.raises(AssertionError):
        mtq.replace_quant_module(m)


def test_wildcards_and_lm_head_exclusion():
    m = _converted(mtq.INT4_AWQ_CFG)
    assert m.body[0].weight_quantizer.num_bits == 4 and m.body[0].weight_quantizer.block_sizes[-1] == 128
    assert not m.body[0].input_quantizer.is_enabled
    assert not m.lm_head.weight_quantizer.is_enabled and not m.lm_head.input_quantizer.is_enabled
    mtq.set_quantizer_attribute(m, lambda n: n.endswith("body.2.weight_quantizer"), {"num_bits": 8, "axis": 0})
    assert m.body[2].weight_quantizer.num_bits == 8 and m.body[2].weight_quantizer.axis == 0
    assert m.body[0].weight_quantizer.num_bits == 4
    mtq.disable_quantizer(m, "*body.0*")
    assert not m.body[0].weight_quantizer.is_enabled and m.body[0].weight_quantizer.num_bits == 4


def test_list_attribute_makes_sequential_quantizer():
    m = _converted(mtq.W4A8_AWQ_BETA_CFG)
    wq = m.body[0].weight_quantizer
    assert isinstance(wq, SequentialQuantizer) and len(wq) == 2
    assert wq[0].num_bits == 4 and wq[1].num_bits == (4, 3)
    assert wq.is_enabled and wq.fake_quant
    with SequentialQuantizer.convert_to_single_quantizer(m):
        assert isinstance(m.body[0].weight_quantizer, TensorQuantizer)
    assert isinstance(m.body[0].weight_quantizer, SequentialQuantizer)
    assert equ.get_quantization_format(m.body[0]) == "w4a8_awq"


def test_one_dict_on_a_sequential_quantizer_goes_to_every_member():
    """reference conversion.py:292-301, nn/modules/tensor_quantizer.py:1182-1196: the
    SequentialQuantizer stays, each member takes the attributes; the export's dummy forward
    relies on this to switch W4A8 quantizers off and back on."""
    m = _converted(mtq.W4A8_AWQ_BETA_CFG)
    with mtq.set_quantizer_by_cfg_context(m, {"*": {"enable": False}}):
        wq = m.body[0].weight_quantizer
        assert isinstance(wq, SequentialQuantizer) and not wq[0].is_enabled and not wq[1].is_enabled
    wq = m.body[0].weight_quantizer
    assert isinstance(wq, SequentialQuantizer) and wq[0].is_enabled and wq[1].is_enabled
    assert wq[0].num_bits == 4 and wq[1].num_bits == (4, 3)
    assert equ.get_quantization_format(m.body[0]) == "w4a8_awq"


def test_set_quantizer_by_cfg_context_restores():
    m = _converted(mtq.INT8_DEFAULT_CFG)
    q = m.body[0].input_quantizer
    with mtq.set_quantizer_by_cfg_context(m, {"*input_quantizer": {"enable": False}}):
        assert not q.is_enabled
    assert q.is_enabled and q.num_bits == 8


def test_enable_alone_is_internal_only():
    """``{"enable": True}`` on its own switches a configured quantizer back on (enable_quantizer,
    the AWQ cache pass: reference model_quant.py:enable_quantizer, model_calib.py:667), while a
    user config that says nothing else is rejected when ``mtq.quantize`` parses it
    (reference config.py:683-707)."""
    m = _converted(mtq.INT8_DEFAULT_CFG)
    q = m.body[0].input_quantizer
    mtq.disable_quantizer(m, "*input_quantizer")
    assert not q.is_enabled
    mtq.enable_quantizer(m, "*input_quantizer")
    assert q.is_enabled and q.num_bits == 8
    q.disable()
    with mtq.set_quantizer_by_cfg_context(q, {"*": {"enable": True}}):
        assert q.is_enabled
    assert not q.is_enabled
    with pytest.raises(Exception, match="Cannot specify only"):
        mtq.model_quant._validated({"quant_cfg": {"*weight_quantizer": {"enable": True}},
                                    "algorithm": "max"})


# ----------------------------------------------------------------------------- TensorQuantizer
def test_quantizer_properties_and_state():
    q = TensorQuantizer(QuantizerAttributeConfig(num_bits=(4, 3)))
    assert q.maxbound == 448.0 and q.amax is None and "per-tensor" in repr(q)
    q.amax = 2.0
    assert q.amax.item() == 2.0
    with pytest.raises(RuntimeError, match="shape"):
        q.amax = [1.0, 2.0]
    q2 = TensorQuantizer(QuantizerAttributeConfig(
        num_bits=(2, 1), block_sizes={-1: 16, "type": "dynamic", "scale_bits": (4, 3)}))
    assert q2.maxbound == 6.0 and not q2.is_static_block_quant and not q2.is_mx_format
    assert TensorQuantizer(QuantizerAttributeConfig(num_bits=4, block_sizes={-1: 128})).is_static_block_quant
    assert TensorQuantizer(QuantizerAttributeConfig(num_bits=8, unsigned=True)).maxbound == 255
    state = q.get_modelopt_state()
    q3 = TensorQuantizer()
    q3.set_from_modelopt_state(state)
    assert q3.num_bits == (4, 3) and q3._amax.shape == ()
    q.reset_amax()
    assert q.amax is None
    with pytest.raises(RuntimeError, match="Calibrator returned None"):
        q.load_calib_amax()


def test_cpu_tensors_raise_instead_of_falling_back():
    q = TensorQuantizer(QuantizerAttributeConfig(num_bits=8))
    with pytest.raises(RuntimeError, match="GPU memory"):
        q(torch.randn(4, 4))
    with pytest.raises(RuntimeError, match="GPU memory"):
        mtq.utils.reduce_amax(torch.randn(4, 4))


def test_layout_helpers():
    assert kernels.amax_layout((4, 5, 6), []) == (1, 1, 120)
    assert kernels.amax_layout((4, 5, 6), [0]) == (1, 4, 30)
    assert kernels.amax_layout((4, 5, 6), [-1]) == (20, 6, 1)
    assert kernels.amax_layout((4, 5, 6), [1]) == (4, 5, 6)
    assert kernels.amax_layout((4, 5, 6), [0, 1]) == (1, 20, 6)
    assert kernels.amax_layout((4, 5, 6), [0, 2]) is None
    assert kernels.amax_layout((4, 1, 6), [0, 2]) == (1, 24, 1)
    assert kernels.layout_from_amax_shape((4, 5, 6), (1, 5, 1)) == (4, 5, 6)
    assert kernels.layout_from_amax_shape((4, 5, 6), ()) == (1, 1, 120)
    assert kernels.layout_from_amax_shape((8, 16), (8,)) == (1, 8, 16)
    assert kernels.layout_from_amax_shape((4, 5, 6), (4, 1, 6)) is None


@pytest.fixture
def oracle_backend(monkeypatch):
    """Route the kernel facade to the CPU oracle so host control flow runs without a GPU."""
    def accumulate(x, acc, layout, reread=False):
        outer, axis, inner = layout
        v = x.reshape(outer, axis, inner).abs().float().amax(dim=(0, 2))
        acc.copy_(torch.maximum(acc, v))
        return acc

    def reduce_gpu(x, dims, keepdims=True, reread=False):
        return reduce.reduce_amax(x, axis=dims, keepdims=keepdims, squeeze_scalar=False) if dims is not None \
            else reduce.reduce_amax(x)

    monkeypatch.setattr(kernels, "absmax_accumulate", accumulate)
    monkeypatch.setattr(kernels, "reduce_amax_gpu", reduce_gpu)
    monkeypatch.setattr(kernels, "fake_quant_int", fake_quant.tensor_quant)
    monkeypatch.setattr(kernels, "fake_quant_fp8", lambda x, amax=None, saturate=False: fake_quant.fp8_eager(x, amax))
    monkeypatch.setattr(kernels, "fake_quant_nvfp4",
                        lambda x, amax, bs=16, mode=0: fake_quant.nvfp4_fake_quant(x, amax, bs))
    monkeypatch.setattr(kernels, "mul_last_dim", lambda x, s: x * s)
    monkeypatch.setattr(kernels, "fake_quant_block_fp", mx.block_fp_fake_quant)


@pytest.mark.parametrize("shape,block_sizes,amax_shape,export_shape", [
    ((6, 256), {-1: 128}, (12, 1), (6, 2)),
    ((6, 200), {-1: 128}, (12, 1), (6, 2)),          # padded to 256
    ((2, 3, 64), {-1: 32}, (12, 1), (2, 3, 2)),
])
def test_static_block_reshape_and_amax_shapes(oracle_backend, shape, block_sizes, amax_shape, export_shape):
    """Shapes follow tests/_test_utils/torch/quantization/tensor_quantizer_common.py:346-449."""
    x = torch.randn(*shape)
    q = TensorQuantizer(QuantizerAttributeConfig(num_bits=4, block_sizes=block_sizes))
    q.enable_calib(); q.disable_quant()
    y = q(x)
    assert y.shape == x.shape and torch.equal(y, x)
    q.load_calib_amax()
    assert tuple(q.amax.shape) == amax_shape
    if export_shape is not None:
        assert tuple(q.export_amax().shape) == export_shape
        q.enable_quant(); q.disable_calib()
        out = q(x)
        want = fake_quant.static_block_fake_quant(
            x, block_sizes[-1], lambda x2, a: fake_quant.tensor_quant(x2, a, 4, False, False))
        assert torch.equal(out, want)
    with pytest.raises(ValueError, match="shape has changed"):
        q(torch.randn(shape[0] + 1, *shape[1:]))


def test_two_axis_blocks(oracle_backend):
    """2-D blocks take the general reshape ([2, 4, 2, 32], amax on dims 0 and 2): calibration and
    fake quantisation follow the reference's reshape -> quantise -> reshape back
    (nn/modules/tensor_quantizer.py:755-800)."""
    q = TensorQuantizer(QuantizerAttributeConfig(num_bits=8, block_sizes={-1: 32, -2: 4}))
    x = torch.randn(8, 64)
    q.enable_calib(); q.disable_quant()
    q(x)
    assert tuple(q._block_reshape_size) == (2, 4, 2, 32) and q.axis == (0, 2)
    q.load_calib_amax()
    blocks = x.reshape(2, 4, 2, 32)
    assert torch.equal(q.amax, blocks.abs().amax(dim=(1, 3), keepdim=True))
    q.enable_quant(); q.disable_calib()
    want = fake_quant.tensor_quant(blocks, q.amax, 8, False, False).reshape(8, 64)
    assert torch.equal(q(x), want)


def test_block_sizes_none_means_per_channel(oracle_backend):
    q = TensorQuantizer(QuantizerAttributeConfig(num_bits=8, block_sizes={-1: None}))
    x = torch.randn(5, 7)
    y = q(x)
    assert q.block_sizes is None and q.axis == (0,)
    assert torch.equal(y, fake_quant.tensor_quant(x, reduce.reduce_amax(x, axis=[1]), 8, False, False))


def test_quantize_flow_on_cpu_with_oracle_backend(oracle_backend):
    m = _Net()
    data = [torch.randn(4, 16) for _ in range(3)]
    mtq.quantize(m, mtq.INT8_DEFAULT_CFG, lambda mod: [mod(d) for d in data])
    lin = m.body[0]
    assert torch.equal(lin.input_quantizer.amax, torch.stack([reduce.reduce_amax(d) for d in data]).max())
    assert torch.equal(lin.weight_quantizer.amax, reduce.reduce_amax(lin.weight.data, axis=[1]))
    assert lin.input_quantizer._if_quant and not lin.input_quantizer._if_calib
    x = data[0]
    want = F.linear(fake_quant.tensor_quant(x, lin.input_quantizer.amax, 8, False, False),
                    fake_quant.tensor_quant(lin.weight.data, lin.weight_quantizer.amax, 8, False, False), lin.bias)
    assert torch.allclose(lin(x), want)
    # straight-through gradient with clipping
    x = (data[0] * 3).requires_grad_()
    lin.input_quantizer(x).sum().backward()
    assert torch.equal(x.grad, (x.detach().abs() <= lin.input_quantizer.amax).float())


# ----------------------------------------------------------------------------- export helpers
def test_postprocess_state_dict_renames_like_reference():
    """Key handling of tests/gpu/torch/export/test_export.py:199-253."""
    sd = {
        "layers.0.self_attn.k_bmm_quantizer._amax": torch.tensor(896.0),
        "layers.0.self_attn.v_bmm_quantizer._amax": torch.tensor(4.48),
        "layers.0.self_attn.q_proj.input_quantizer._pre_quant_scale": torch.ones(4),
        "layers.0.self_attn.q_proj.input_quantizer._amax": torch.tensor(1.0),
        "layers.0.self_attn.q_proj.weight_quantizer._amax": torch.tensor(1.0),
        "layers.0.self_attn.q_proj.output_quantizer._amax": torch.tensor(1.0),
        "layers.0.self_attn.q_proj.weight": torch.zeros(2, 2),
        "layers.0.self_attn.q_proj.weight_scale": torch.ones(1, 2, 3),
    }
    out = equ.postprocess_state_dict(sd, 448, "FP8")
    assert set(out) == {"layers.0.self_attn.k_proj.k_scale", "layers.0.self_attn.v_proj.v_scale",
                        "layers.0.self_attn.q_proj.pre_quant_scale", "layers.0.self_attn.q_proj.weight",
                        "layers.0.self_attn.q_proj.weight_scale"}
    assert out["layers.0.self_attn.k_proj.k_scale"].item() == 2.0
    assert out["layers.0.self_attn.v_proj.v_scale"].item() == 1.0       # clamped to at least 1
    assert out["layers.0.self_attn.q_proj.weight_scale"].shape == (2, 3)  # leading 1 squeezed


def test_hf_quant_config_sections():
    layers = {"model.layers.0.q_proj.quantization": "nvfp4", "model.layers.0.q_proj.awq_block_size": 16,
              "lm_head.quantization": None, "lm_head.awq_block_size": 0}
    out = equ.process_layer_quant_config(layers)
    assert out == {"quant_algo": "NVFP4", "kv_cache_quant_algo": None, "group_size": 16,
                   "exclude_modules": ["lm_head"]}
    layers["model.layers.0.k_proj.quantization"] = "fp8"
    layers["model.layers.0.k_proj.awq_block_size"] = 0
    out = equ.process_layer_quant_config(layers)
    assert out["quant_algo"] == "MIXED_PRECISION" and set(out["quantized_layers"]) == {
        "model.layers.0.q_proj", "model.layers.0.k_proj"}
    awq = equ.process_layer_quant_config({"a.b.quantization": "int4_awq", "a.b.awq_block_size": 128})
    assert awq["quant_algo"] == "W4A16_AWQ" and awq["group_size"] == 128 and awq["pre_quant_scale"] is True


def test_quantization_format_detection():
    for cfg, fmt in [(mtq.INT8_DEFAULT_CFG, "int8_sq"), (mtq.INT8_WEIGHT_ONLY_CFG, "int8_wo"),
                     (mtq.FP8_DEFAULT_CFG, "fp8"), (mtq.INT4_AWQ_CFG, "int4_awq"),
                     (mtq.NVFP4_DEFAULT_CFG, "nvfp4")]:
        m = _converted(cfg)
        assert equ.get_quantization_format(m.body[0]) == fmt
        assert equ.get_quantization_format(m.lm_head) is None
        assert equ.get_quantization_format(m) == fmt
    m = _converted(mtq.NVFP4_DEFAULT_CFG)
    assert equ.get_weight_block_size(m.body[0]) == 16 and equ.get_weight_block_size(m.lm_head) == 0


def test_compress_surface_without_a_gpu():
    """Names and config handling of ``mtq.compress`` (the packing itself needs the GPU)."""
    import modelopt_amd.torch.quantization as mtq

    assert mtq.CompressConfig().compress == {"*": True} and mtq.CompressConfig().quant_gemm is True
    model = torch.nn.Sequential(torch.nn.Linear(8, 8))
    assert not mtq.is_real_quantized(model)
    with pytest.raises(ValueError, match="expected a boolean"):
        mtq.compress(model, {"*": "yes"})
    assert issubclass(mtq.nn.RealQuantLinear, mtq.nn.QuantModule)


def test_mx_quantizer_control_flow(oracle_backend):
    """An MX quantizer needs no amax, ignores calibration and pads the last block."""
    cfg = mtq.MXFP4_DEFAULT_CFG["quant_cfg"]["*input_quantizer"]
    q = TensorQuantizer(QuantizerAttributeConfig(**cfg))
    assert q.is_mx_format
    x = torch.randn(3, 5, 40).to(torch.bfloat16)
    assert torch.equal(q(x), mx.block_fp_fake_quant(x, 32, "E2M1"))
    q.enable_calib()
    q(x)
    assert q.amax is None
    assert mtq.MXFP8_DEFAULT_CFG["algorithm"] is None


def test_public_names_of_the_reference_package():
    """``modelopt.torch.quantization`` re-exports the ``__all__`` of model_quant.py:40-49,
    conversion.py:46-53, compress.py:18 and config.py, plus ``QuantModuleRegistry``,
    ``update_quant_cfg_with_kv_cache_quant`` and the ``plugins`` / ``utils`` modules
    (__init__.py:19-27)."""
    names = ["auto_quantize", "calibrate", "disable_quantizer", "enable_quantizer", "fold_weight",
             "postprocess_amax", "print_quant_summary", "quantize", "register", "replace_quant_module",
             "set_quantizer_attribute", "set_quantizer_by_cfg", "set_quantizer_by_cfg_context",
             "unregister", "compress", "QuantModuleRegistry", "update_quant_cfg_with_kv_cache_quant",
             "plugins", "utils", "QuantizeConfig", "QuantizerAttributeConfig", "CompressConfig", "choices"]
    for name in names + sorted(mtq.config.choices):
        assert hasattr(mtq, name), name
    with pytest.raises(NotImplementedError):
        mtq.auto_quantize(None)
    assert torch.nn.Linear in mtq.QuantModuleRegistry


def test_quantizer_attribute_config_validation():
    """The constructor-time checks of the reference's config
    (tests/unit/torch/quantization/test_tensor_quant_cpu.py:33-85): defaults, ``dict()`` round
    trip, ``{"enable": True}`` alone is refused, bit widths must be positive."""
    cfg = QuantizerAttributeConfig(num_bits=5)
    assert cfg.num_bits == 5 and cfg.axis is None
    cfg = QuantizerAttributeConfig(axis=(0, 1, 3))
    assert cfg.num_bits == 8 and cfg.axis == (0, 1, 3)
    for kw in ({"num_bits": 2, "fake_quant": True, "axis": (1, 2)}, {"num_bits": 2, "unsigned": True}):
        cfg = QuantizerAttributeConfig(**kw)
        assert cfg == QuantizerAttributeConfig(**cfg.dict())
    with pytest.raises(ValueError, match="Invalid quantizer config: Cannot specify only {'enable': True}. "
                                         "Additional parameters are required when enabling quantization."):
        QuantizerAttributeConfig(enable=True)
    for bits in (0, -1, (0, 3), (-1, 2)):
        with pytest.raises(ValueError, match="num_bits must be a positive integer or a tuple of positive integers."):
            QuantizerAttributeConfig(enable=True, num_bits=bits)


def test_quant_linear_is_constructible_without_conversion():
    """``QuantLinear(in, out)`` is an ``nn.Linear`` with its quantizers attached and the same
    state dict keys (reference: nn/modules/quant_linear.py:56-62)."""
    from modelopt_amd.torch.quantization.nn import QuantLinear
    m = QuantLinear(4, 6, bias=False, quant_desc_weight=QuantizerAttributeConfig(num_bits=4, axis=0))
    assert isinstance(m, nn.Linear) and m.bias is None and m.weight.shape == (6, 4)
    assert m.weight_quantizer.num_bits == 4 and m.input_quantizer.num_bits == 8
    assert not m.output_quantizer.is_enabled
    assert list(m.state_dict()) == ["weight"]
    assert QuantLinear(4, 6).weight_quantizer.num_bits == 8      # the override stayed on its instance


class _SdpaAttention(nn.Module):
    def forward(self, qkv, extra_arg=None):
        q, k, v = qkv
        return F.scaled_dot_product_attention(q, k, v)


class _MatmulAttention(nn.Module):
    def forward(self, qkv):
        q, k, v = qkv
        w = torch.matmul(q, k.transpose(-1, -2)) * 0.25
        out = torch.matmul(w.softmax(-1), v)
        return out


class _AtAttention(nn.Module):
    def forward(self, qkv):
        q, k, v = qkv
        w = (q @ k.transpose(-1, -2)) * 0.25
        out = w.softmax(-1) @ v
        return out if super().__call__ is not None else None      # a zero-argument super() survives


class _NoAttention(nn.Module):
    def forward(self, x):
        return x


@pytest.mark.parametrize("cls,q_seen", [(_SdpaAttention, (1, 4, 8)), (_MatmulAttention, (1, 8, 4)),
                                        (_AtAttention, (1, 4, 8))])
def test_register_attention_for_kv_quant_rewrites_the_products(cls, q_seen):
    """Three attention spellings (reference: plugins/attention.py:45-216 and
    tests/unit/torch/quantization/test_quantize_replace.py:34-58): the converted module owns the
    three quantizers, each sees its operand in the documented layout (the ``matmul`` form hands
    the query over transposed), and with them disabled the output is the original's."""
    assert mtq.plugins.register_attention_for_kv_quant(cls) is True
    try:
        model = nn.Sequential(cls())
        mtq.replace_quant_module(model)
        attn = model[0]
        assert isinstance(attn, cls) and type(attn).__mro__[1].__name__ == "_Quant" + cls.__name__
        seen = {}
        for n in "qkv":
            quantizer = getattr(attn, f"{n}_bmm_quantizer")
            assert quantizer.is_enabled and quantizer.num_bits == 8
            quantizer.register_forward_hook(lambda m, inp, out, n=n: seen.__setitem__(n, tuple(inp[0].shape)))
        mtq.set_quantizer_attribute(model, "*", {"enable": False})
        g = torch.Generator().manual_seed(0)
        qkv = (torch.randn(1, 4, 8, generator=g), torch.randn(1, 6, 8, generator=g), torch.randn(1, 6, 8, generator=g))
        assert torch.equal(attn(qkv), cls()(qkv))
        assert seen == {"q": q_seen, "k": (1, 6, 8), "v": (1, 6, 8)}
        assert "_kvq_original_class_" not in globals()
    finally:
        mtq.unregister(cls)
    assert mtq.QuantModuleRegistry.get(cls) is None


def test_register_attention_for_kv_quant_refuses_other_modules(capsys):
    assert mtq.plugins.register_attention_for_kv_quant(_NoAttention) is False
    assert "not attached" in capsys.readouterr().out
    assert mtq.QuantModuleRegistry.get(_NoAttention) is None


def test_need_calibration():
    """tests/unit/torch/quantization/test_config_validation.py:29-35"""
    from modelopt_amd.torch.quantization import config as C
    assert C.need_calibration(C.FP8_DEFAULT_CFG)
    assert not C.need_calibration(C.FP8_PER_CHANNEL_PER_TOKEN_CFG)
    assert not C.need_calibration(C.FP8_2D_BLOCKWISE_WEIGHT_ONLY_CFG)
    assert C.need_calibration(C.INT4_AWQ_CFG)
    assert C.need_calibration(C.W4A8_AWQ_BETA_CFG)
    assert C.need_calibration(C.NVFP4_DEFAULT_CFG)
    assert not C.need_calibration(C.INT4_BLOCKWISE_WEIGHT_ONLY_CFG)
    assert not C.need_calibration(C.MXFP4_MLP_WEIGHT_ONLY_CFG)


def test_reprs_do_not_raise():
    """tests/unit/torch/quantization/test_print.py:25-53 (the parts on this path)"""
    from modelopt_amd.torch.quantization import calib, nn as qnn, tensor_quant
    assert "num_bits" in repr(tensor_quant.QUANT_DESC_8BIT_LINEAR_WEIGHT_PER_ROW)
    assert "TensorQuantizer" in repr(TensorQuantizer())
    holder = nn.Module()
    holder.linear, holder.quant_linear = nn.Linear(33, 65), qnn.Linear(33, 65)
    assert "weight_quantizer" in repr(holder)
    assert repr(calib.MaxCalibrator(7, 1, False)) == (
        "MaxCalibrator(num_bits=7 axis=1 unsigned=False calib_amax=None track_amax=False)")
    assert str(calib.MaxCalibrator(7, 1, False, track_amax=True)) == "MaxCalibrator(track_amax=True)"
    assert "amaxs=[]" in repr(calib.MaxCalibrator(7, 1, False, track_amax=True))
    from modelopt_amd.torch.quantization.calib.calibrator import _Calibrator
    assert issubclass(calib.MaxCalibrator, _Calibrator)


def test_library_operators_are_registered_with_fake_implementations():
    """``tensorrt::quantize_op`` / ``tensorrt::dynamic_block_quantize_op`` exist with the
    reference's schemas (tensor_quant.py:221-273) and trace under fake tensors without a device."""
    from torch.fx.experimental.proxy_tensor import make_fx

    from modelopt_amd.torch.quantization import tensor_quant as tq

    assert "Tensor amax, int num_bits, int exponent_bits, bool unsigned, bool narrow_range" in str(
        torch.ops.tensorrt.quantize_op.default._schema)
    assert "int block_size, Tensor amax" in str(torch.ops.tensorrt.dynamic_block_quantize_op.default._schema)
    assert hasattr(torch.ops.tensorrt.dynamic_block_quantize_op, "overload")

    def f(x, a):
        y = tq.quantize_op(x, a, 8, 4, False, False)
        return tq.dynamic_block_quantize_op(y, 16, a, 4, 2, 8, 4)

    graph = make_fx(f, tracing_mode="fake")(torch.randn(4, 32), torch.tensor(1.0)).graph
    targets = [str(n.target) for n in graph.nodes if n.op == "call_function"]
    assert targets == ["tensorrt.quantize_op.default", "tensorrt.dynamic_block_quantize_op.default"]
    with pytest.raises(RuntimeError, match="GPU memory"):   # the CPU implementation is the loud failure
        torch.ops.tensorrt.quantize_op(torch.randn(4), torch.tensor(1.0), 8, 0, False, False)


def test_dense_flat_view_covers_permuted_blocks_only():
    from modelopt_amd.torch.quantization.kernels import dense_flat_view

    x = torch.arange(2 * 3 * 4 * 5, dtype=torch.float32).reshape(2, 3, 4, 5)
    for t in (x, x.transpose(1, 2), x.permute(3, 0, 2, 1), x.transpose(1, 2)[1:], x.unsqueeze(0).transpose(2, 3),
              torch.zeros(3, 1, 4).transpose(0, 2)):
        v = dense_flat_view(t)
        assert v is not None and v.dim() == 1 and sorted(v.tolist()) == sorted(t.flatten().tolist())
    for t in (x[:, :2], x[..., ::2], x.transpose(1, 2)[:, :, :2], x[0, 0].expand(3, 4, 5)):
        assert dense_flat_view(t) is None


def test_all_valid_scales_groups_by_dtype_and_skips_what_is_not_a_tensor():
    from modelopt_amd.torch.quantization.utils import all_valid_scales
    ok = [torch.ones(3), torch.ones(2, dtype=torch.bfloat16), None, torch.tensor(2), torch.empty(0)]
    assert all_valid_scales(ok) and all_valid_scales([])
    assert not all_valid_scales(ok + [torch.tensor([1.0, -1.0], dtype=torch.bfloat16)])
    assert not all_valid_scales([torch.tensor([float("nan")])])
    assert not all_valid_scales([torch.tensor([float("inf")], dtype=torch.float16), torch.ones(1)])


def test_max_calibrator_reports_whether_it_has_seen_anything_without_computing():
    from modelopt_amd.torch.quantization import calib
    c = calib.MaxCalibrator(8, None, False)
    assert not c.has_amax() and c.compute_amax() is None
    c.collect(torch.empty(4, 4, device="meta"))
    assert c.has_amax() and c.compute_amax().is_meta


def test_plan_inputs_notice_a_reallocated_tensor():
    from modelopt_amd import _hip
    a, b = torch.nn.Parameter(torch.zeros(8)), torch.zeros(8)
    pinned = _hip._PinnedInputs([a, b])
    pinned.verify()
    a.data = torch.ones(8)
    with pytest.raises(RuntimeError, match="reallocated"):
        pinned.verify()


def test_first_minimum_picks_what_min_over_the_loss_dict_picks():
    """AWQ-lite chooses ``min(loss, key=loss.get)`` in the reference: the first smallest value,
    where a NaN never replaces the running best and a NaN in front is never replaced."""
    from modelopt_amd.torch.quantization.model_calib import _first_minimum
    nan = float("nan")
    cases = [[3.0, 1.0, 2.0], [1.0, 1.0, 0.5, 0.5], [nan, 1.0, 0.5], [2.0, nan, 1.0], [2.0, nan, 3.0],
             [nan, nan], [0.0], [5.0, 4.0, nan, 4.0], [float("inf"), float("inf")]]
    for values in cases:
        keys = list(range(len(values)))
        want = min(keys, key=dict(zip(keys, values)).get)
        got = int(_first_minimum(torch.tensor(values, dtype=torch.float64)))
        assert got == want, (values, got, want)


def test_deferred_scale_checks_make_one_check_at_the_end():
    from modelopt_amd.torch.quantization.utils import all_valid_scales, deferred_scale_checks
    with deferred_scale_checks() as pending:
        assert all_valid_scales([torch.ones(2), None])
        with deferred_scale_checks():                      # a nested block hands over to the outer one
            assert all_valid_scales([torch.ones(1)])
        assert len(pending) == 2
    with pytest.raises(AssertionError, match="negative, inf or nan"):
        with deferred_scale_checks():
            assert all_valid_scales([torch.tensor([1.0, float("nan")])])   # recorded, reported later
    assert not all_valid_scales([torch.tensor([-1.0])])                  # outside a block: checked at once


def test_best_clip_from_stacked_losses_equals_the_loop_over_ratios():
    """model_calib.py:958-966 of the reference, ratio by ratio, against the stacked selection:
    ties (the first smallest wins), NaN losses (never win), blocks with no finite loss (clip 0)."""
    import types

    from modelopt_amd.torch.quantization.model_calib import _best_clip, _clip_ratios

    ratios = _clip_ratios(0.5, 0.05)
    assert ratios == (0.5, 0.55, 0.6, 0.65, 0.7, 0.75, 0.8, 0.85, 0.9, 0.95, 1.0)
    g = torch.Generator().manual_seed(0)
    for dtype in (torch.bfloat16, torch.float16, torch.float32):
        w_amax = (torch.rand(40, 1, generator=g) + 0.01).to(dtype)
        loss_all = torch.rand(len(ratios), 8, 5, generator=g).round(decimals=1)    # many ties
        loss_all[3, 0, 0] = float("nan")
        loss_all[:, 1, 1] = float("nan")
        loss_all[:, 2, 2] = float("inf")
        loss_all[0, 3, 3] = -1.0
        helper = types.SimpleNamespace(w_amax=w_amax, loss_all=loss_all,
                                       loss={r: loss_all[i] for i, r in enumerate(ratios)})
        best_loss = torch.ones_like(w_amax) * float("inf")
        best_clip = torch.zeros_like(w_amax)
        for shrink, loss in helper.loss.items():
            loss = loss.view_as(w_amax)
            better = loss < best_loss
            best_loss = torch.where(better, loss, best_loss)
            best_clip = torch.where(better, w_amax * shrink, best_clip)
        got_loss, got_clip = _best_clip(helper)
        assert got_clip.dtype == dtype and torch.equal(got_clip, best_clip)
        assert torch.equal(got_loss, best_loss.float())
        assert float(got_clip.view(8, 5)[1, 1]) == 0 and float(got_clip.view(8, 5)[2, 2]) == 0


def test_deferred_checks_of_three_kinds_share_the_block_s_end():
    from modelopt_amd.torch.quantization.utils import (DeferredCheckError, all_positive, all_valid_scales,
                                                        deferred_scale_checks)
    assert all_positive(torch.tensor([1.0, 2.0])) and not all_positive(torch.tensor([1.0, 0.0]))
    with deferred_scale_checks() as block:
        assert all_positive(torch.tensor([0.5]))
        assert all_valid_scales([torch.zeros(3)])
        block.report = [torch.tensor([1.0, float("inf")])]     # reported, never raised
    assert block.report_ok is False
    with pytest.raises(DeferredCheckError, match="pre_quant_scale should be positive"):
        with deferred_scale_checks():
            with deferred_scale_checks():                       # handed to the enclosing block
                assert all_positive(torch.tensor([1.0, -1.0]))
    with deferred_scale_checks() as outer:
        with deferred_scale_checks() as inner:
            inner.report = [torch.tensor([float("nan")])]       # a nested owner gets its answer at once
        assert inner.report_ok is False and outer.report_ok


def test_quantize_reports_a_bad_calibration_batch_in_the_calibrator_s_words(oracle_backend):
    """Inside mtq.quantize every validity check waits for the end of the algorithm; a NaN that a
    calibrator has seen is then reported with the reference's message (calib/max.py:74-77)."""
    model = nn.Sequential(nn.Linear(16, 16))
    x = torch.randn(4, 16)
    x[1, 3] = float("nan")
    with pytest.raises(AssertionError, match="detected nan values in amax"):
        mtq.quantize(model, mtq.INT8_DEFAULT_CFG, lambda m: m(x))


# ----------------------------------------------------------------------------- strict host checks
@pytest.fixture
def strict_checks():
    previous = mtq.set_strict_checks(True)
    yield
    mtq.set_strict_checks(previous)


@pytest.fixture
def lenient_int_kernel(oracle_backend, monkeypatch):
    """An integer kernel stand-in that, like the HIP kernel, never looks at the data on the host
    (the oracle follows the reference's CPU path and raises by itself): whatever raises in these
    tests is the product's host layer."""
    monkeypatch.setattr(kernels, "fake_quant_int", lambda x, amax, *args: x.clone())


def test_strict_checks_unsigned_quantization_of_negative_values_raises(oracle_backend, strict_checks, monkeypatch):
    """tests/_test_utils/torch/quantization/tensor_quant_common.py:86-101 (``test_unsigned``): the
    accepted case quantises like a signed grid of one more bit, the negative case raises the
    reference's ``TypeError`` (tensor_quant.py:577-578)."""
    from modelopt_amd.torch.quantization.tensor_quant import fake_tensor_quant

    torch.manual_seed(0)
    x = torch.randn(31).abs()
    got = fake_tensor_quant(x, torch.max(x.abs()), None, 8, True)
    assert torch.equal(got, fake_quant.tensor_quant(x, torch.max(x.abs()), 9, False, True))
    monkeypatch.setattr(kernels, "fake_quant_int", lambda x, amax, *args: x.clone())
    x = torch.randn(3, 7)
    with pytest.raises(TypeError, match="Negative values encountered"):
        fake_tensor_quant(x, torch.max(torch.abs(x)), None, 8, True)
    with pytest.raises(TypeError, match="Negative values encountered"):
        TensorQuantizer(QuantizerAttributeConfig(num_bits=8, unsigned=True))(x)


def test_strict_checks_negative_amax_raises(lenient_int_kernel, strict_checks):
    """tensor_quant.py:585-587 of the reference: ``ValueError("Negative values in amax")``, also
    when only one channel's amax is negative."""
    from modelopt_amd.torch.quantization.tensor_quant import fake_tensor_quant

    x = torch.randn(4, 8)
    with pytest.raises(ValueError, match="Negative values in amax"):
        fake_tensor_quant(x, torch.tensor(-1.0))
    amax = torch.tensor([[1.0], [2.0], [-0.5], [1.0]])
    with pytest.raises(ValueError, match="Negative values in amax"):
        fake_tensor_quant(x, amax)
    assert fake_tensor_quant(x, amax.abs()).shape == x.shape


def test_strict_checks_are_off_by_default(lenient_int_kernel):
    from modelopt_amd.torch.quantization.tensor_quant import fake_tensor_quant

    assert not mtq.strict_checks()
    x = torch.randn(3, 7)
    fake_tensor_quant(x, torch.max(torch.abs(x)), None, 8, True)   # no host look at the data


def test_strict_checks_max_calibrator_asserts_at_the_batch_that_is_bad(oracle_backend, strict_checks):
    """calib/max.py:69-77 of the reference: the assertions fire inside ``collect`` on the batch
    that holds the inf / NaN, and that batch is not folded into the running maximum."""
    from modelopt_amd.torch.quantization.calib import MaxCalibrator

    cal = MaxCalibrator(8, None, False)
    cal.collect(torch.tensor([1.0, -3.0, 2.0]))
    bad = torch.tensor([1.0, float("inf")])
    with pytest.raises(AssertionError, match="detected inf values in amax. inf in original tensor: True"):
        cal.collect(bad)
    with pytest.raises(AssertionError, match="detected nan values in amax. nan in original tensor: True"):
        cal.collect(torch.tensor([float("nan"), 5.0]))
    cal.collect(torch.tensor([0.5]))
    assert float(cal.compute_amax()) == 3.0
    # per channel, and the history of tracked maxima
    cal = MaxCalibrator(8, 0, False, track_amax=True)
    cal.collect(torch.tensor([[1.0, -2.0], [0.5, 0.25]]))
    with pytest.raises(AssertionError, match="detected nan"):
        cal.collect(torch.tensor([[1.0, float("nan")], [0.5, 0.25]]))
    assert torch.equal(cal.compute_amax().flatten(), torch.tensor([2.0, 0.5])) and len(cal.amaxs) == 1


def test_default_max_calibrator_reports_a_bad_batch_in_compute_amax(oracle_backend):
    from modelopt_amd.torch.quantization.calib import MaxCalibrator

    cal = MaxCalibrator(8, None, False)
    cal.collect(torch.tensor([1.0, float("inf")]))     # no assertion here: no host synchronisation
    cal.collect(torch.tensor([2.0]))
    with pytest.raises(AssertionError, match="detected inf values in amax"):
        cal.compute_amax()


def test_forward_loop_argument_count_matches_inspect():
    """The shortcut for plain functions and lambdas gives what inspect.signature gives, and
    everything else goes through inspect.signature."""
    import functools
    import inspect

    from modelopt_amd.torch.quantization.model_quant import _takes_no_argument

    class Callable_:
        def __call__(self):
            return None

        def method(self):
            return None

    def wrapped_inner(model):
        return None

    @functools.wraps(wrapped_inner)
    def wrapper():
        return wrapped_inner(None)

    def star(*args):
        return None

    def keyword_only(*, model=None):
        return None

    cases = [lambda: None, lambda m: None, lambda m=None: None, star, keyword_only, Callable_(),
             Callable_().method, functools.partial(wrapped_inner, None), wrapper, len.__call__]
    for fn in cases:
        assert _takes_no_argument(fn) == (len(inspect.signature(fn).parameters) == 0), fn


def test_validated_config_is_kept_by_content_for_plain_configs_only():
    import enum

    from modelopt_amd.torch.quantization import model_quant

    cfg = {"quant_cfg": {"*weight_quantizer": {"num_bits": 4, "block_sizes": {-1: 32}, "enable": True},
                         "default": {"enable": False}}, "algorithm": {"method": "max"}}
    model_quant._VALIDATED.clear()
    first, algo = model_quant._validated(cfg)
    assert len(model_quant._VALIDATED) == 1
    second, algo2 = model_quant._validated(copy.deepcopy(cfg))
    assert len(model_quant._VALIDATED) == 1 and algo == algo2 and algo is not algo2
    assert second["*weight_quantizer"] is first["*weight_quantizer"]      # shared, never written to
    # another order of the patterns is another config: later entries win
    swapped = {"quant_cfg": dict(reversed(list(cfg["quant_cfg"].items()))), "algorithm": {"method": "max"}}
    model_quant._validated(swapped)
    assert len(model_quant._VALIDATED) == 2

    class Bits(enum.IntEnum):
        FOUR = 4

    odd = copy.deepcopy(cfg)
    odd["quant_cfg"]["*weight_quantizer"]["num_bits"] = Bits.FOUR          # not a plain value
    assert model_quant._content_key(odd) is None
    model_quant._validated(odd)
    assert len(model_quant._VALIDATED) == 2


def test_is_quantized_linear_on_modules_and_other_objects():
    from modelopt_amd.torch.quantization.utils import is_quantized_linear

    lin = nn.Linear(8, 8)
    assert not is_quantized_linear(lin) and not is_quantized_linear(object()) and not is_quantized_linear(3)
    mtq.replace_quant_module(seq := nn.Sequential(lin))
    assert is_quantized_linear(seq[0]) and not is_quantized_linear(seq)
    conv = nn.Sequential(nn.Conv2d(3, 3, 1))
    mtq.replace_quant_module(conv)
    assert not is_quantized_linear(conv[0])                                 # a 4-D weight
    plain = nn.Module()                                                     # quantizers as plain attributes
    plain.__dict__["input_quantizer"] = seq[0].input_quantizer
    plain.__dict__["weight_quantizer"] = seq[0].weight_quantizer
    plain.weight = nn.Parameter(torch.zeros(4, 4))
    assert is_quantized_linear(plain)


def test_small_helpers_of_the_quantization_utils():
    """reference: utils.py:247-273 (attribute names), :339-379 (replace_function, multi_context,
    export mode, is_pow2), :489-511 (quantizer state dicts)."""
    import contextlib
    import math

    from modelopt_amd.torch.quantization import utils as U

    names = U.quantizer_attr_names()
    assert names.weight_quantizer == "weight_quantizer" and names.weight_scale_2 == "weight_scale_2"
    names = U.quantizer_attr_names("gate_up_proj")
    assert names == U.QuantizerAttrNames(
        "gate_up_proj_weight_quantizer", "gate_up_proj_input_quantizer", "gate_up_proj_output_quantizer",
        "gate_up_proj_weight_scale", "gate_up_proj_weight_scale_2", "gate_up_proj_input_scale",
        "gate_up_proj_output_scale")
    assert [n for n in range(0, 20) if U.is_pow2(n)] == [1, 2, 4, 8, 16]
    with U.replace_function(math, "floor", lambda v: "patched"):
        assert math.floor(1.5) == "patched" and math._floor(1.5) == 1
    assert math.floor(1.5) == 1 and not hasattr(math, "_floor")
    seen = []

    @contextlib.contextmanager
    def tag(t):
        seen.append(t)
        yield t

    with U.multi_context(tag("a"), tag("b")) as entered:
        assert entered == ["a", "b"] and seen == ["a", "b"]
    assert not U.is_torch_export_mode()
    with U.export_torch_mode():
        assert U.is_torch_export_mode()
    assert not U.is_torch_export_mode()
    model = nn.Sequential(nn.Linear(8, 8))
    mtq.replace_quant_module(model)
    model[0].input_quantizer.amax = torch.tensor(3.0)
    state = U.get_quantizer_state_dict(model)
    assert set(state) == {"0.input_quantizer", "0.weight_quantizer", "0.output_quantizer"}
    state = {name: {k: v.clone() for k, v in entries.items()} for name, entries in state.items()}
    assert float(state["0.input_quantizer"]["_amax"]) == 3.0
    model[0].input_quantizer.amax = torch.tensor(5.0)
    U.set_quantizer_state_dict(model, state)
    assert float(model[0].input_quantizer.amax) == 3.0
    with U.enable_weight_access_and_writeback(model[0], model):
        assert model[0].weight.shape == (8, 8)


def test_private_names_of_the_functional_module():
    """tensor_quant.py:42-59 and :286-292 by name; the eager body's errors need no strict mode
    (checked before the kernel is reached)."""
    from modelopt_amd.torch.quantization import tensor_quant as tq

    assert tq._fp8_eager is tq.fp8_eager and tq.DISABLE_TRITON_KERNEL is False
    assert tq.QUANT_DESC_8BIT_CONV2D_WEIGHT_PER_CHANNEL.axis == 0
    with pytest.raises(TypeError, match="unsigned"):
        tq._tensor_quant(torch.tensor([-1.0, 2.0]), torch.tensor(2.0), 8, True)
    with pytest.raises(ValueError, match="amax"):
        tq._tensor_quant(torch.tensor([1.0, 2.0]), torch.tensor(-2.0))
