"""``mtq.quantize`` / export on a Hugging Face ``transformers`` model (random-init tiny Llama):
the attention modules get KV-cache quantizers through the on-the-fly plugin, as the reference's
``register_hf_attentions_on_the_fly`` does (plugins/huggingface.py:176-235), and the exported
checkpoint has the reference's key layout (tests/gpu/torch/export/test_export.py:199-253)."""

import copy
import json
import os

import pytest
import torch

import modelopt_amd.torch.quantization as mtq
from modelopt_amd.torch.export import export_hf_checkpoint
from oracle import reduce

transformers = pytest.importorskip("transformers")
pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _tiny_llama(seed=0):
    cfg = transformers.LlamaConfig(vocab_size=512, hidden_size=256, intermediate_size=512,
                                   num_hidden_layers=2, num_attention_heads=4,
                                   num_key_value_heads=2, max_position_embeddings=128)
    torch.manual_seed(seed)
    return transformers.LlamaForCausalLM(cfg).to(torch.bfloat16).to(DEV)


def _ids(seed=1):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, 512, (4, 32), generator=g).to(DEV)


def _with_kv(base):
    return mtq.utils.update_quant_cfg_with_kv_cache_quant(copy.deepcopy(base),
                                                          mtq.FP8_KV_CFG["quant_cfg"])


def test_attention_modules_get_kv_quantizers_and_the_dispatch_table_is_restored():
    from transformers.models.llama import modeling_llama

    model, ids = _tiny_llama(), _ids()
    ref = model(ids).logits
    before = modeling_llama.ALL_ATTENTION_FUNCTIONS[model.config._attn_implementation]
    seen = {}

    def spy(attn, q, k, v, *a, **kw):  # what reaches the attention kernel during calibration
        seen.setdefault(id(attn), []).append((k.detach().clone(), v.detach().clone()))
        return before(attn, q, k, v, *a, **kw)

    modeling_llama.ALL_ATTENTION_FUNCTIONS[model.config._attn_implementation] = spy
    try:
        mtq.quantize(model, _with_kv(mtq.FP8_DEFAULT_CFG), lambda m: m(ids))
    finally:
        modeling_llama.ALL_ATTENTION_FUNCTIONS[model.config._attn_implementation] = before
    assert modeling_llama.ALL_ATTENTION_FUNCTIONS[model.config._attn_implementation] is before

    names = [n for n, _ in model.named_modules() if n.endswith("quantizer")]
    assert len(names) == 2 * (7 * 3 + 3) + 3
    for layer in model.model.layers:
        attn = layer.self_attn
        assert not attn.q_bmm_quantizer.is_enabled
        k, v = seen[id(attn)][0]
        # the quantizers saw exactly the key / value states handed to the attention kernel
        assert torch.equal(attn.k_bmm_quantizer.amax.cpu(), reduce.reduce_amax(k.cpu()))
        assert torch.equal(attn.v_bmm_quantizer.amax.cpu(), reduce.reduce_amax(v.cpu()))
    out = model(ids).logits
    assert torch.isfinite(out).all()
    assert (out.float() - ref.float()).norm() / ref.float().norm() < 0.15


@pytest.mark.parametrize("name,quant_algo", [("FP8_DEFAULT_CFG", "FP8"), ("NVFP4_DEFAULT_CFG", "NVFP4"),
                                             ("INT4_AWQ_CFG", "W4A16_AWQ")])
def test_quantize_and_export(tmp_path, name, quant_algo):
    from safetensors.torch import load_file

    model, ids = _tiny_llama(), _ids()
    cfg = _with_kv(getattr(mtq, name))
    previous = mtq.set_fp8_overflow_behavior("saturate")  # folding moves V a hair past its amax
    try:
        mtq.quantize(model, cfg, lambda m: m(ids))
        assert torch.isfinite(model(ids).logits).all()
    finally:
        mtq.set_fp8_overflow_behavior(previous)
    export_hf_checkpoint(model, export_dir=str(tmp_path))
    tensors = {}
    for f in os.listdir(tmp_path):
        if f.endswith(".safetensors"):
            tensors.update(load_file(os.path.join(tmp_path, f)))
    prefix = "model.layers.1.self_attn."
    assert tensors[prefix + "k_proj.k_scale"].dtype == torch.float32
    assert tensors[prefix + "v_proj.v_scale"].dtype == torch.float32
    assert not any("quantizer" in k or "_amax" in k for k in tensors)
    w = tensors[prefix + "q_proj.weight"]
    if quant_algo == "FP8":
        assert w.dtype == torch.float8_e4m3fn and w.shape == (256, 256)
        assert tensors[prefix + "q_proj.input_scale"].numel() == 1
    elif quant_algo == "NVFP4":
        assert w.dtype == torch.uint8 and w.shape == (256, 128)
        assert tensors[prefix + "q_proj.weight_scale"].dtype == torch.float8_e4m3fn
        assert tensors[prefix + "q_proj.weight_scale"].shape == (256, 16)
        assert tensors[prefix + "q_proj.weight_scale_2"].numel() == 1
    else:
        assert w.dtype == torch.uint8 and w.shape == (128, 256)
        assert tensors[prefix + "q_proj.weight_scale"].shape == (256, 2)
        assert tensors[prefix + "o_proj.pre_quant_scale"].shape == (256,)
    assert tensors["lm_head.weight"].dtype == torch.bfloat16
    with open(os.path.join(tmp_path, "hf_quant_config.json")) as f:
        q = json.load(f)["quantization"]
    assert q["quant_algo"] == quant_algo and q["kv_cache_quant_algo"] == "FP8"
    assert q["exclude_modules"] == ["lm_head"]
    with open(os.path.join(tmp_path, "config.json")) as f:
        assert "quantization_config" in json.load(f)


def test_fp8_overflow_switch():
    """Values above the amax: NaN with the eager (CPU) semantics, +-amax with the CUDA kernel's.
    The default follows the reference's dispatch on a device tensor (tensor_quant.py:62-90):
    per-tensor and per-axis amax go to the clamping kernel, amax None or on two dims to the
    eager cast."""
    from modelopt_amd.torch.quantization.tensor_quant import fp8_eager, scaled_e4m3_impl
    from oracle import fake_quant

    x = torch.tensor([0.5, 1.0, 1.03, 1.04, 2.0, -3.0], dtype=torch.bfloat16)
    amax = torch.tensor(1.0, dtype=torch.bfloat16)
    assert mtq.get_fp8_overflow_behavior() == "auto"
    clamped = torch.tensor([0.5, 1.0, 1.0, 1.0, 1.0, -1.0], dtype=torch.bfloat16)
    assert torch.equal(scaled_e4m3_impl(x.to(DEV), amax.to(DEV)).cpu(), clamped)
    per_axis = scaled_e4m3_impl(x.to(DEV).reshape(2, 3), amax.to(DEV).expand(2, 1).contiguous())
    assert torch.equal(per_axis.cpu().reshape(-1), clamped)
    assert torch.isnan(scaled_e4m3_impl((x * 300).to(DEV), None)).sum() == 2       # plain cast: eager
    two_dims = scaled_e4m3_impl(x.to(DEV).reshape(2, 3), amax.to(DEV).expand(2, 3).contiguous())
    assert torch.isnan(two_dims).sum() == 3                                          # eager fallback
    assert torch.isnan(fp8_eager(x.to(DEV), amax.to(DEV))).sum() == 3
    previous = mtq.set_fp8_overflow_behavior("nan")
    try:
        got = scaled_e4m3_impl(x.to(DEV), amax.to(DEV)).cpu()
    finally:
        mtq.set_fp8_overflow_behavior(previous)
    want = fake_quant.fp8_eager(x, amax)
    assert torch.equal(torch.isnan(got), torch.isnan(want)) and torch.isnan(got).sum() == 3
    assert torch.equal(got[~torch.isnan(got)], want[~torch.isnan(want)])
    previous = mtq.set_fp8_overflow_behavior("saturate")
    try:
        sat = scaled_e4m3_impl(x.to(DEV), amax.to(DEV)).cpu()
    finally:
        mtq.set_fp8_overflow_behavior(previous)
    assert torch.equal(sat, torch.tensor([0.5, 1.0, 1.0, 1.0, 1.0, -1.0], dtype=torch.bfloat16))
    with pytest.raises(ValueError):
        mtq.set_fp8_overflow_behavior("wrap")


@pytest.mark.parametrize("name", sorted(n for n in mtq.config.choices if not n.endswith("KV_CFG")))
def test_every_named_config_runs_on_the_hf_model(name):
    """Each stock config (with the FP8 KV-cache quantizers merged in, as the reference's
    llm_ptq example does) converts, calibrates and runs a forward on the tiny Llama; the
    quantised logits stay within the error a 4- to 8-bit format gives on a random model."""
    model, ids = _tiny_llama(), _ids()
    ref = model(ids).logits
    previous = mtq.set_fp8_overflow_behavior("saturate")
    try:
        mtq.quantize(model, _with_kv(getattr(mtq, name)), lambda m: m(ids))
        out = model(ids).logits
    finally:
        mtq.set_fp8_overflow_behavior(previous)
    assert torch.isfinite(out).all()
    err = ((out.float() - ref.float()).norm() / ref.float().norm()).item()
    assert err < 0.5, err
    assert any(getattr(m, "is_enabled", False) for n, m in model.named_modules()
               if n.endswith("weight_quantizer"))
