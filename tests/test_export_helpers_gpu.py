"""Helpers of the layer-wise export in ``export/quant_utils.py`` that the Hugging Face exporter does
not call itself: attention amax unification, KV cache scales, and the inverse of
``to_quantized_weight``.  Vectors and expectations follow the reference's own tests."""

import pytest
import torch

# ------------------------------------------------------------------ helpers of the layer-wise export
class _Attn(torch.nn.Module):
    def __init__(self, weights):
        super().__init__()
        for name, w in zip(("q_proj", "k_proj", "v_proj", "o_proj"), weights):
            lin = torch.nn.Linear(w.shape[1], w.shape[0], bias=False)
            lin.weight.data.copy_(w)
            setattr(self, name, lin)

    def forward(self, x):
        return self.o_proj(self.q_proj(x) + self.k_proj(x) + self.v_proj(x))


@pytest.mark.gpu
@pytest.mark.parametrize("sign", [1.0, -1.0])
@pytest.mark.parametrize("cfg_name", ["FP8_DEFAULT_CFG", "NVFP4_DEFAULT_CFG"])
def test_adjust_attn_amax_values(cfg_name, sign):
    """vectors of the reference's tests/gpu/torch/export/test_export.py:275-318"""
    import modelopt_amd.torch.quantization as mtq
    from modelopt_amd.torch.export.quant_utils import adjust_attn_amax_values

    weights = [torch.tensor([[0.1, 0.3], [0.22, 0.45]]), torch.tensor([[0.44, 0.32], [0.11, sign * 0.95]]),
               torch.tensor([[0.9, 0.03], [0.92, 0.8]]), torch.tensor([[0.01, sign * 0.97], [0.29, 0.77]])]
    model = _Attn(weights).to("cuda:0")
    mtq.quantize(model, getattr(mtq, cfg_name), lambda m: m(torch.randn(1, 4, 2, device="cuda:0")))
    adjust_attn_amax_values(model)
    for name in ("q_proj", "k_proj", "v_proj"):
        assert getattr(model, name).weight_quantizer.amax == torch.tensor(0.95, device="cuda:0")
    assert model.o_proj.weight_quantizer.amax == torch.tensor(0.97, device="cuda:0")
    with pytest.raises(ValueError, match="No projection layers"):
        adjust_attn_amax_values(torch.nn.Sequential(torch.nn.Linear(2, 2)))


@pytest.mark.gpu
def test_from_quantized_weight_inverts_to_quantized_weight():
    """reference: quant_utils.py:768-857; the round trip error is at most half a quantisation step"""
    from modelopt_amd.torch.export import quant_utils as Q

    w = torch.randn(32, 64, device="cuda:0", generator=torch.Generator("cuda:0").manual_seed(0)).bfloat16()
    scale = (w.float().abs().max() / 448.0).reshape(1)
    packed = Q.to_quantized_weight(w, scale, Q.QUANTIZATION_FP8)
    back = Q.from_quantized_weight(packed, scale, Q.QUANTIZATION_FP8, torch.float32)
    assert packed.element_size() == 1 and back.dtype == torch.float32
    assert torch.equal(back, packed.view(torch.float8_e4m3fn).float() * scale)
    assert ((back - w.float()).abs() <= w.float().abs() / 16 + scale * 2.0 ** -10).all()
    rows = w.float().abs().amax(dim=1) / 127.0
    packed = Q.to_quantized_weight(w, rows, Q.QUANTIZATION_INT8_SQ)
    back = Q.from_quantized_weight(packed, rows, Q.QUANTIZATION_INT8_SQ, torch.float32)
    assert packed.dtype == torch.int8 and ((back - w.float()).abs() <= rows[:, None] * 0.5 + 1e-7).all()
    assert Q.from_quantized_weight(w, None, "", torch.float16).dtype == torch.float16
    with pytest.raises(NotImplementedError):
        Q.from_quantized_weight(packed, rows, Q.QUANTIZATION_INT4_AWQ, torch.float16)


@pytest.mark.gpu
def test_get_kv_cache_scaling_factor():
    """reference: quant_utils.py:348-370: FP8 scales are amax / 448 but never below 1"""
    from modelopt_amd.torch.export import quant_utils as Q
    from modelopt_amd.torch.quantization.config import QuantizerAttributeConfig
    from modelopt_amd.torch.quantization.nn import TensorQuantizer

    attn = torch.nn.Module()
    assert Q.get_kv_cache_scaling_factor(attn) == [None, None]
    fp8 = QuantizerAttributeConfig(num_bits=(4, 3), axis=None)
    attn.k_bmm_quantizer = TensorQuantizer(fp8, amax=896.0).to("cuda:0")
    attn.v_bmm_quantizer = TensorQuantizer(fp8, amax=4.48).to("cuda:0")
    with pytest.warns(UserWarning, match="Large KV activation"):
        k_scale, v_scale = Q.get_kv_cache_scaling_factor(attn)
    assert k_scale.tolist() == [2.0] and v_scale.tolist() == [1.0]


def _export_cases():
    from conftest import load_export_vectors

    return load_export_vectors()


@pytest.mark.gpu
@pytest.mark.parametrize("case", _export_cases(), ids=lambda c: c["name"])
def test_to_quantized_weight_matches_reference_outputs(case):
    """The recorded outputs of the reference's to_quantized_weight / pack_int4_in_uint8
    (export/quant_utils.py:697-774, tests/golden/export_vectors.json) through the kernels."""
    from conftest import assert_bits_equal
    from modelopt_amd.torch.export import quant_utils as Q

    w, s = case["weight"].to("cuda:0"), case["scale"].to("cuda:0")
    got = Q.to_quantized_weight(w, s, case["format"])
    want = case["out"]
    if want.dtype == torch.float8_e4m3fn:
        got = got.view(torch.float8_e4m3fn)
    assert_bits_equal(got.cpu(), want, case["name"])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fp8_pc_pt_cast_of_stacked_expert_weights(dtype):
    """FP8 per-channel casts of a 3-D (experts, output, input) weight: the three scale layouts the
    reference tells apart by shape and its three errors (export/quant_utils.py:780-810), each
    against the literal expression on the CPU."""
    from conftest import assert_bits_equal
    from modelopt_amd.torch.export import quant_utils as Q
    from oracle import export

    g = torch.Generator().manual_seed(21)
    w = (torch.randn((3, 48, 80), generator=g) * 0.05).to(dtype)
    per_expert = w.abs().amax(dim=(1, 2)).float() / 448.0
    per_input = w.abs().amax(dim=1).float() / 448.0
    per_output = w.abs().amax(dim=2).float() / 448.0
    for name, s, view in (("per expert", per_expert, per_expert[:, None, None]),
                          ("per input channel", per_input, per_input.unsqueeze(-2)),
                          ("per output channel", per_output, per_output.unsqueeze(-1)),
                          ("per output channel, 16-bit scales", per_output.to(dtype),
                           per_output.to(dtype).unsqueeze(-1))):
        got = Q.to_quantized_weight(w.to("cuda:0"), s.to("cuda:0"), "fp8_pc_pt")
        assert_bits_equal(got.view(torch.float8_e4m3fn).cpu(), export.fp8_export_cast(w, view), name)
    dev = w.to("cuda:0")
    with pytest.raises(ValueError, match="num_experts"):
        Q.to_quantized_weight(dev, torch.ones(2, 48, device="cuda:0"), "fp8_pc_pt")
    with pytest.raises(ValueError, match="Ambiguous"):
        Q.to_quantized_weight(dev[:, :, :48].contiguous(), torch.ones(3, 48, device="cuda:0"), "fp8_pc_pt")
    with pytest.raises(ValueError, match="unsqueeze"):
        Q.to_quantized_weight(dev, torch.ones(3, 7, device="cuda:0"), "fp8_pc_pt")


@pytest.mark.gpu
@pytest.mark.parametrize("quantization", ["int4_awq", "nvfp4_awq"])
def test_resmooth_and_get_scale_of_row_chunks(quantization):
    """Two row chunks smoothed with their own scales brought to the mean scale, block scales
    recomputed (export/quant_utils.py:126-185), against the same expressions on the CPU."""
    from conftest import assert_bits_equal
    from modelopt_amd.torch.export import quant_utils as Q
    from oracle import export, qtensor

    g = torch.Generator().manual_seed(41)
    w = (torch.randn((64, 256), generator=g) * 0.05).to(torch.bfloat16)
    pqs = [torch.rand(256, generator=g) + 0.5 for _ in range(2)]
    group = 128 if quantization == "int4_awq" else 16
    weights, scales, shared = Q.resmooth_and_get_scale(w.to("cuda:0"), [p.to("cuda:0") for p in pqs], 2, group,
                                                       quantization=quantization)
    mean = torch.stack(pqs).mean(dim=0)
    assert_bits_equal(shared.cpu(), mean, "shared scale")
    want_w = torch.cat([c * p.type(c.dtype) / mean.type(c.dtype) for c, p in zip(torch.chunk(w, 2, dim=0), pqs)])
    assert_bits_equal(weights.cpu(), want_w, "re-smoothed weights")
    if quantization == "int4_awq":
        want_s = torch.cat([export.get_scaling_factor_from_weight(c, group) for c in torch.chunk(want_w, 2, dim=0)])
        assert_bits_equal(scales.cpu(), want_s, "block scales")
    else:
        want_s = torch.cat([qtensor.nvfp4_block_scales(c, group)[0].view(torch.uint8)
                            for c in torch.chunk(want_w, 2, dim=0)])
        assert scales.dtype == torch.float8_e4m3fn
        assert torch.equal(scales.cpu().view(torch.uint8), want_s)
    t, ts = Q.maybe_transpose_expert_weight_dimensions(torch.zeros(2, 3, 4), torch.zeros(2, 3, 1))
    assert t.shape == (2, 4, 3) and ts.shape == (2, 1, 3)
    same, none = Q.maybe_transpose_expert_weight_dimensions(torch.zeros(3, 4))
    assert same.shape == (3, 4) and none is None
