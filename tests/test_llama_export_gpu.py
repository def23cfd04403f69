"""End-to-end on a small Llama-shaped decoder: mtq.quantize calibration sweep and HF-layout export."""

import copy
import json

import pytest
import torch

import modelopt_amd.torch.quantization as mtq
from conftest import assert_bits_equal
from modelopt_amd.testing.llama_decoder import LlamaConfig, LlamaForCausalLM
from modelopt_amd.torch.export import export_hf_checkpoint
from modelopt_amd.torch.quantization.nn import TensorQuantizer
from oracle import export as oexport
from oracle import reduce

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
CFG = LlamaConfig(vocab_size=512, hidden_size=128, intermediate_size=256, num_hidden_layers=2,
                  num_attention_heads=4, num_key_value_heads=2)


def _ids(n=4, b=2, s=32):
    g = torch.Generator().manual_seed(5)
    return [torch.randint(0, CFG.vocab_size, (b, s), generator=g) for _ in range(n)]


def _loop(batches):
    def run(model):
        for ids in batches:
            model(ids.to(DEV))
    return run


def _quantized(cfg):
    model = LlamaForCausalLM(CFG, device=DEV, seed=1)
    ref_weights = {n: p.detach().cpu().clone() for n, p in model.named_parameters()}
    mtq.quantize(model, cfg, _loop(_ids()))
    return model, ref_weights


def test_nvfp4_fp8kv_calibration_sweep_and_export(tmp_path):
    cfg = mtq.utils.update_quant_cfg_with_kv_cache_quant(mtq.NVFP4_DEFAULT_CFG, mtq.FP8_KV_CFG["quant_cfg"])
    model, w = _quantized(cfg)
    enabled = [n for n, m in model.named_modules() if isinstance(m, TensorQuantizer) and m.is_enabled]
    assert len(enabled) == 2 * (7 * 2 + 2)
    for n, m in model.named_modules():
        if isinstance(m, TensorQuantizer) and m.is_enabled:
            assert m.amax is not None and m.amax.numel() == 1 and m.amax > 0, n
    for name in ("model.layers.0.self_attn.q_proj", "model.layers.1.mlp.down_proj"):
        got = model.get_submodule(name).weight_quantizer.amax
        assert_bits_equal(got.cpu(), reduce.reduce_amax(w[name + ".weight"]), name)
    out = model(_ids(1)[0].to(DEV))
    assert torch.isfinite(out.float()).all()

    state, qcfg = export_hf_checkpoint(model, export_dir=tmp_path)
    assert qcfg["quantization"]["quant_algo"] == "NVFP4"
    assert qcfg["quantization"]["group_size"] == 16
    assert qcfg["quantization"]["kv_cache_quant_algo"] == "FP8"
    assert qcfg["quantization"]["exclude_modules"] == ["lm_head"]
    assert not any("_amax" in k or "quantizer" in k for k in state)

    # fused projections share the weight amax: packed bytes == oracle on the shared amax
    attn = "model.layers.0.self_attn."
    shared = torch.stack([reduce.reduce_amax(w[attn + p + ".weight"]) for p in ("q_proj", "k_proj", "v_proj")]).max()
    for p in ("q_proj", "k_proj", "v_proj"):
        packed_o, wsf_o, wsf2_o = oexport.nvfp4_export(w[attn + p + ".weight"], shared, 16)
        assert_bits_equal(state[attn + p + ".weight"].cpu(), packed_o, p + " packed")
        assert_bits_equal(state[attn + p + ".weight_scale"].cpu(), wsf_o, p + " weight_scale")
        assert_bits_equal(state[attn + p + ".weight_scale_2"].cpu().reshape(()), wsf2_o.reshape(()), p + " weight_scale_2")
        assert state[attn + p + ".input_scale"].dtype == torch.float32
    o = "model.layers.1.self_attn.o_proj"
    packed_o, wsf_o, wsf2_o = oexport.nvfp4_export(w[o + ".weight"], reduce.reduce_amax(w[o + ".weight"]), 16)
    assert_bits_equal(state[o + ".weight"].cpu(), packed_o, "o_proj packed")
    assert state[o + ".weight"].dtype == torch.uint8 and state[o + ".weight"].shape == (128, 64)
    assert state[o + ".weight_scale"].dtype == torch.float8_e4m3fn and state[o + ".weight_scale"].shape == (128, 8)
    k_scale = state[attn + "k_proj.k_scale"]
    assert k_scale.dtype == torch.float32 and k_scale.item() >= 1.0
    assert state["lm_head.weight"].dtype == torch.bfloat16

    from safetensors.torch import load_file

    saved = load_file(str(tmp_path / "model.safetensors"))
    assert set(saved) == set(state)
    assert torch.equal(saved[o + ".weight"], state[o + ".weight"].cpu())
    hf = json.load(open(tmp_path / "hf_quant_config.json"))
    assert hf["producer"]["name"] == "modelopt" and hf["quantization"]["quant_algo"] == "NVFP4"
    conf = json.load(open(tmp_path / "config.json"))
    assert conf["quantization_config"]["quant_algo"] == "NVFP4" and conf["quantization_config"]["ignore"] == ["lm_head"]


def test_fp8_export(tmp_path):
    model, w = _quantized(mtq.FP8_DEFAULT_CFG)
    state, qcfg = export_hf_checkpoint(model, export_dir=tmp_path)
    assert qcfg["quantization"]["quant_algo"] == "FP8"
    name = "model.layers.0.mlp.down_proj"
    amax = reduce.reduce_amax(w[name + ".weight"])
    wsf = torch.tensor(amax.float().item() / 448.0)
    assert_bits_equal(state[name + ".weight"].cpu(), oexport.fp8_export_cast(w[name + ".weight"], wsf), "fp8 weight")
    assert state[name + ".weight_scale"].dtype == torch.float32
    assert state[name + ".weight_scale"].item() == pytest.approx(wsf.item(), rel=1e-6)


def test_int4_awq_export(tmp_path):
    cfg = copy.deepcopy(mtq.INT4_AWQ_CFG)
    model, w = _quantized(cfg)
    lin = model.get_submodule("model.layers.0.mlp.down_proj")
    w_folded = lin.weight.data.cpu().clone()
    amax = lin.weight_quantizer.export_amax().cpu()
    assert amax.shape == (128, 2)
    state, qcfg = export_hf_checkpoint(model, export_dir=tmp_path)
    # q/k/v (and gate/up) were re-smoothed to one shared input scale, which then went into the
    # layernorm in front of them: no pre_quant_scale is exported for those five projections
    layer = model.get_submodule("model.layers.0")
    for lin_ in (layer.self_attn.q_proj, layer.self_attn.k_proj, layer.self_attn.v_proj,
                 layer.mlp.gate_proj, layer.mlp.up_proj):
        assert not hasattr(lin_.input_quantizer, "_pre_quant_scale") and lin_.fused_with_prequant
    for proj in ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "mlp.gate_proj", "mlp.up_proj"):
        assert f"model.layers.0.{proj}.pre_quant_scale" not in state
    assert "model.layers.0.self_attn.o_proj.pre_quant_scale" in state
    assert not torch.equal(state["model.layers.0.input_layernorm.weight"].cpu(),
                           w["model.layers.0.input_layernorm.weight"])
    q = qcfg["quantization"]
    assert q["quant_algo"] == "W4A16_AWQ" and q["group_size"] == 128 and q["pre_quant_scale"] is True
    name = "model.layers.0.mlp.down_proj"
    ws = amax.float() / 7.0
    assert_bits_equal(state[name + ".weight_scale"].cpu(), ws, "weight_scale")
    assert_bits_equal(state[name + ".weight"].cpu(), oexport.pack_int4_in_uint8(w_folded, ws), "packed int4")
    assert state[name + ".weight"].shape == (64, 256)
    assert state[name + ".pre_quant_scale"].shape == (256,)


def test_fusion_pre_pass_keeps_the_model_function():
    """Shared scales, re-smoothed weights and the fold into the layernorm change how the
    computation is written, not what it computes (up to bf16 rounding of the folded weights)."""
    from modelopt_amd.torch.export import requantize_resmooth_fused_llm_layers

    model, w = _quantized(copy.deepcopy(mtq.INT4_AWQ_CFG))
    ids = _ids(1)[0].to(DEV)
    attn = model.get_submodule("model.layers.1.self_attn")
    pqs = [p.input_quantizer._pre_quant_scale.float().cpu() for p in (attn.q_proj, attn.k_proj, attn.v_proj)]
    norm_w = model.get_submodule("model.layers.1.input_layernorm").weight.detach().float().cpu()
    off = {"*": {"enable": False}}     # a disabled quantizer still applies its pre_quant_scale
    with torch.no_grad(), mtq.set_quantizer_by_cfg_context(model, off):
        before = model(ids).float()
    requantize_resmooth_fused_llm_layers(model)
    with torch.no_grad(), mtq.set_quantizer_by_cfg_context(model, off):
        after = model(ids).float()
    rel = (after - before).norm() / before.norm()
    assert float(rel) < 0.02          # bf16 rounding of the re-smoothed and folded weights
    avg = torch.stack(pqs).mean(0).to(torch.bfloat16).float()
    got = model.get_submodule("model.layers.1.input_layernorm").weight.detach().float().cpu()
    assert torch.allclose(got, (norm_w.to(torch.bfloat16) * avg.to(torch.bfloat16)).float(), rtol=2 ** -7)
    # o_proj and down_proj read tensors no layernorm produced: their scales stay
    assert hasattr(attn.o_proj.input_quantizer, "_pre_quant_scale")
    # the block amax of a re-smoothed weight was recalibrated on the new weight
    k = attn.k_proj
    want = reduce.reduce_amax(k.weight.data.cpu().reshape(-1, 128), axis=[1], keepdims=True)
    assert_bits_equal(k.weight_quantizer.amax.cpu().reshape(want.shape), want, "recalibrated amax")


# ------------------------------------------------------------------ the remaining export formats
from oracle import mx as omx          # noqa: E402
from oracle import qtensor as oq      # noqa: E402


def test_w4a8_nvfp4_fp8_export(tmp_path):
    """reference export/quant_utils.py:275-287, :308-311: the per-tensor scale is amax / 448 (the
    consumer dequantises to FP8), the block scales and codes follow from it; :660-666."""
    model, w = _quantized(copy.deepcopy(mtq.W4A8_NVFP4_FP8_CFG))
    state, qcfg = export_hf_checkpoint(model, export_dir=tmp_path)
    q = qcfg["quantization"]
    assert q["quant_algo"] == "W4A8_NVFP4_FP8" and q["group_size"] == 32
    assert q["exclude_modules"] == ["lm_head"]
    name = "model.layers.1.self_attn.o_proj"
    wsf2 = reduce.reduce_amax(w[name + ".weight"]).float() / 448.0
    packed, wsf, _ = oq.nvfp4_quantize(w[name + ".weight"], 32, wsf2=wsf2)
    assert_bits_equal(state[name + ".weight_scale_2"].cpu().reshape(()), wsf2.reshape(()), "weight_scale_2")
    assert_bits_equal(state[name + ".weight_scale"].cpu(), wsf, "weight_scale")
    assert_bits_equal(state[name + ".weight"].cpu(), packed, "packed")
    assert state[name + ".input_scale"].dtype == torch.float32 and state[name + ".input_scale"].numel() == 1
    # fused projections share the weight amax
    attn = "model.layers.0.self_attn."
    shared = torch.stack([reduce.reduce_amax(w[attn + p + ".weight"]) for p in ("q_proj", "k_proj", "v_proj")]).max()
    packed, wsf, _ = oq.nvfp4_quantize(w[attn + "k_proj.weight"], 32, wsf2=shared.float() / 448.0)
    assert_bits_equal(state[attn + "k_proj.weight"].cpu(), packed, "k_proj packed")
    assert_bits_equal(state[attn + "k_proj.weight_scale"].cpu(), wsf, "k_proj weight_scale")


@pytest.mark.parametrize("cfg_name,algo", [("MXFP4_DEFAULT_CFG", "mxfp4"),
                                           ("W4A8_MXFP4_FP8_CFG", "W4A8_MXFP4_FP8")])
def test_mxfp4_exports(tmp_path, cfg_name, algo):
    """reference export/quant_utils.py:289-292, :831-832, :667-671"""
    model, w = _quantized(copy.deepcopy(getattr(mtq, cfg_name)))
    state, qcfg = export_hf_checkpoint(model, export_dir=tmp_path)
    assert qcfg["quantization"]["quant_algo"] == algo
    if algo == "W4A8_MXFP4_FP8":
        assert qcfg["quantization"]["group_size"] == 32
    for name in ("model.layers.0.self_attn.k_proj", "model.layers.1.mlp.down_proj"):
        weight = w[name + ".weight"]
        packed, scales = omx.mxfp4_quantize(weight, 32)
        assert_bits_equal(state[name + ".weight"].cpu(), packed, name + " packed")
        assert_bits_equal(state[name + ".weight_scale"].cpu(), scales.reshape(weight.shape[0], -1),
                          name + " weight_scale")
        # both configs say ``"algorithm": None``: nothing is calibrated, so the FP8 input
        # quantizer of the W4A8 variant has no amax to export either
        assert name + ".input_scale" not in state
        assert name + ".weight_scale_2" not in state


def test_fp8_block_weight_only_export(tmp_path):
    """reference export/quant_utils.py:474-480, :776-779: 128 x 128 blocks, scale = amax / 448"""
    model, w = _quantized(copy.deepcopy(mtq.FP8_2D_BLOCKWISE_WEIGHT_ONLY_CFG))
    state, qcfg = export_hf_checkpoint(model, export_dir=tmp_path)
    assert qcfg["quantization"]["quant_algo"] == "fp8_pb_wo"
    blocks = {-1: 128, -2: 128}
    for name in ("model.layers.0.mlp.gate_proj", "model.layers.1.mlp.down_proj",
                 "model.layers.0.self_attn.k_proj"):
        weight = w[name + ".weight"]          # k_proj is 64 x 128: its rows are padded to a block
        amax = reduce.reduce_block_amax(reduce.reduce_block_padding(weight, blocks), blocks)
        if name.endswith("k_proj"):
            # q, k and v are one block each here, which the fusion pre-pass takes for per-tensor
            # scales and unifies (reference export/quant_utils.py:1056-1070)
            attn = name.rsplit(".", 1)[0]
            amax = torch.stack([reduce.reduce_amax(w[f"{attn}.{p}.weight"])
                                for p in ("q_proj", "k_proj", "v_proj")]).max().reshape(amax.shape)
        codes, scales = oq.fp8_quantize(weight, (amax.float() / 448.0).squeeze(), block_sizes=blocks)
        assert state[name + ".weight"].dtype == torch.float8_e4m3fn
        assert_bits_equal(state[name + ".weight"].cpu().view(torch.uint8), codes.view(torch.uint8), name)
        got = state[name + ".weight_scale"].cpu()
        assert got.dtype == torch.float32 and got.numel() == amax.numel()
        assert_bits_equal(got.reshape(-1), (amax.float() / 448.0).reshape(-1), name + " weight_scale")
        assert name + ".input_scale" not in state


def test_fp8_block_real_export(tmp_path):
    """A model packed by ``mtq.compress`` first (reference quant_utils.py:480, unified_export_hf
    .py:292-297): the packed weight goes out as it is, the quantizer's scales as fp32."""
    model, w = _quantized(copy.deepcopy(mtq.FP8_2D_BLOCKWISE_WEIGHT_ONLY_CFG))
    mtq.compress(model)
    name = "model.layers.1.mlp.down_proj"
    lin = model.get_submodule(name)
    codes = lin.weight.data.clone()
    scales = lin.weight_quantizer._scale.clone()
    state, qcfg = export_hf_checkpoint(model, export_dir=tmp_path)
    assert qcfg["quantization"]["quant_algo"] == "fp8_pb_real"
    assert_bits_equal(state[name + ".weight"].cpu().view(torch.uint8), codes.cpu().view(torch.uint8), name)
    assert state[name + ".weight_scale"].dtype == torch.float32
    assert torch.equal(state[name + ".weight_scale"].cpu(), scales.float().cpu())
    want, _ = oq.fp8_quantize(w[name + ".weight"], block_sizes={-1: 128, -2: 128})
    assert_bits_equal(codes.cpu().view(torch.uint8), want.view(torch.uint8), "compressed codes")


def test_w4a8_awq_export(tmp_path):
    """A SequentialQuantizer (INT4 blocks, then FP8 per tensor) survives the fusion pre-pass and
    exports as W4A8_AWQ with both scales (reference export/quant_utils.py:446-459, :265-266,
    :313-320)."""
    model, w = _quantized(copy.deepcopy(mtq.W4A8_AWQ_BETA_CFG))
    name = "model.layers.1.mlp.down_proj"
    lin = model.get_submodule(name)
    folded = lin.weight.data.cpu().clone()
    amax4 = lin.weight_quantizer[0].export_amax().cpu()
    amax8 = lin.weight_quantizer[1].export_amax().cpu()
    state, qcfg = export_hf_checkpoint(model, export_dir=tmp_path)
    q = qcfg["quantization"]
    assert q["quant_algo"] == "W4A8_AWQ" and q["group_size"] == 128 and q["pre_quant_scale"] is True
    ws = amax4.float() / 7.0
    assert_bits_equal(state[name + ".weight_scale"].cpu(), ws, "weight_scale")
    assert_bits_equal(state[name + ".weight_scale_2"].cpu().reshape(()), (amax8.float() / 448.0).reshape(()),
                      "weight_scale_2")
    assert_bits_equal(state[name + ".weight"].cpu(), oexport.pack_int4_in_uint8(folded, ws), "packed int4")
    assert name + ".pre_quant_scale" in state and name + ".input_scale" in state


def test_nvfp4_awq_clip_real_quantization_follows_the_overflow_mode(tmp_path):
    """awq_clip shrinks the per-tensor amax of an NVFP4 weight (reference model_calib.py:869-876),
    so block scales can exceed E4M3's range.  The reference's cast (qtensor/nvfp4_tensor.py:84-91)
    then stores NaN; "saturate" stores 448, and the compressed model then computes what the
    fake-quantised one does."""
    ids = _ids(1)[0].to(DEV)
    for mode in ("nan", "saturate"):
        previous = mtq.set_fp8_overflow_behavior(mode)
        try:
            model, w = _quantized(copy.deepcopy(mtq.NVFP4_AWQ_CLIP_CFG))
            lin = model.get_submodule("model.layers.0.self_attn.q_proj")
            weight = lin.weight.data.cpu().clone()
            # whether the search clips this particular layer depends on the data: apply the
            # smallest shrink it considers, as model_calib.py:872 does when that one wins
            lin.weight_quantizer.amax = lin.weight_quantizer.amax * 0.5
            amax = lin.weight_quantizer.amax.float().cpu()
            assert float(amax) < float(reduce.reduce_amax(weight))
            fake = model(ids).float()
            mtq.compress(model)
            real = model(ids).float()
            wsf = lin.weight_quantizer._scale.cpu()
            want_scales, _ = oq.nvfp4_block_scales(weight, 16, amax / 2688.0, keep_high_precision=True)
            if mode == "nan":
                want = want_scales.to(torch.float8_e4m3fn)
                assert_bits_equal(wsf.view(torch.uint8), want.view(torch.uint8), "block scales")
                assert bool(torch.isnan(wsf.float()).any()) == bool((want_scales > 464).any())
            else:
                want = want_scales.clamp(max=448.0).to(torch.float8_e4m3fn)
                assert_bits_equal(wsf.view(torch.uint8), want.view(torch.uint8), "saturated block scales")
                assert torch.isfinite(real).all()
                assert float((real - fake).norm() / fake.norm()) < 1e-2
        finally:
            mtq.set_fp8_overflow_behavior(previous)


@pytest.mark.parametrize("cfg_name", ["INT4_AWQ_CFG", "NVFP4_AWQ_LITE_CFG"])
@pytest.mark.parametrize("heads", [(4, 4), (4, 2), (4, 1)], ids=["mha", "gqa", "mqa"])
def test_pattern_fuse_prequant(cfg_name, heads):
    """tests/gpu/torch/export/test_quant_utils.py:43-103: o_proj's input scale goes into v_proj's
    rows (averaged per KV head for grouped heads), down_proj's into up_proj's; the scales and the
    model function stay."""
    from modelopt_amd.torch.export.quant_utils import fuse_prequant_to_linear

    cfg = LlamaConfig(vocab_size=256, hidden_size=64, intermediate_size=128, num_hidden_layers=2,
                      num_attention_heads=heads[0], num_key_value_heads=heads[1])
    model = LlamaForCausalLM(cfg, device=DEV, seed=3)
    ids = torch.randint(0, 256, (1, 16), generator=torch.Generator().manual_seed(0)).to(DEV)
    mtq.quantize(model, copy.deepcopy(getattr(mtq, cfg_name)), lambda m: m(ids))
    off = {"*": {"enable": False}}
    with torch.no_grad():
        before = model(ids).float()
        with mtq.set_quantizer_by_cfg_context(model, off):
            before_exact = model(ids).float()
    attn = model.get_submodule("model.layers.0.self_attn")
    mlp = model.get_submodule("model.layers.0.mlp")
    o_scale = attn.o_proj.input_quantizer._pre_quant_scale.detach().clone()
    d_scale = mlp.down_proj.input_quantizer._pre_quant_scale.detach().clone()
    v_w, up_w = attn.v_proj.weight.detach().clone(), mlp.up_proj.weight.detach().clone()

    fuse_prequant_to_linear(model, fuse_grouped_heads=True)

    for name in ("model.layers.0.self_attn.o_proj", "model.layers.0.mlp.down_proj",
                 "model.layers.1.self_attn.o_proj", "model.layers.1.mlp.down_proj"):
        lin = model.get_submodule(name)
        assert not hasattr(lin.input_quantizer, "_pre_quant_scale"), name
        assert lin.fused_with_prequant, name
    # the arithmetic of the fold
    kv, hd = heads[1], 64 // heads[0]
    want_scale = o_scale.view(kv, heads[0] // kv, hd).mean(dim=1).reshape(-1)
    assert torch.equal(attn.v_proj.weight.detach(), v_w * want_scale.view(-1, 1))
    assert torch.equal(mlp.up_proj.weight.detach(), up_w * d_scale.view(-1, 1))
    # and the weight amax of the scaled linears was taken again
    wq = mlp.up_proj.weight_quantizer
    if wq.amax.numel() == 1:
        assert_bits_equal(wq.amax.cpu().reshape(()), reduce.reduce_amax(mlp.up_proj.weight.detach().cpu()).reshape(()))
    with torch.no_grad():
        after = model(ids).float()
        with mtq.set_quantizer_by_cfg_context(model, off):
            after_exact = model(ids).float()
    assert torch.allclose(before, after, rtol=1e-1, atol=5e-1)
    # without quantization error only the rounding of the folded weights (and, for grouped
    # heads, of o_proj re-smoothed to the averaged scale) remains
    assert float((after_exact - before_exact).norm() / before_exact.norm()) < 0.03


def test_calibration_sweep_on_two_layers_of_the_8b_shape():
    """The calibration sweep configuration on a two-layer slice at the real layer shape (hidden 4096, FFN 14336,
    32 query / 8 KV heads; vocabulary cut to 1024): NVFP4 weight + input quantizers and FP8 K / V
    quantizers.  Every calibrated amax -- 14 weights, 14 linear inputs, 2 x (K, V) -- equals the
    oracle's reduce_amax over exactly the tensors that reached that quantizer on the device."""
    import dataclasses

    from modelopt_amd.testing.llama_decoder import LLAMA3_8B

    shape = dataclasses.replace(LLAMA3_8B, num_hidden_layers=2, vocab_size=1024)
    model = LlamaForCausalLM(shape, device=DEV, seed=9)
    g = torch.Generator().manual_seed(9)
    batches = [torch.randint(0, shape.vocab_size, (2, 512), generator=g) for _ in range(3)]
    cfg = mtq.utils.update_quant_cfg_with_kv_cache_quant(mtq.NVFP4_DEFAULT_CFG, mtq.FP8_KV_CFG["quant_cfg"])

    seen = {}   # quantizer name -> running oracle amax of what it was shown

    def watch(name):
        def hook(module, args):
            if module._if_calib:
                local = reduce.reduce_amax(args[0].detach().cpu())
                seen[name] = local if name not in seen else torch.maximum(seen[name], local)
        return hook

    def loop(m):
        handles = [q.register_forward_pre_hook(watch(n)) for n, q in m.named_modules()
                   if isinstance(q, TensorQuantizer)]
        for ids in batches:
            m(ids.to(DEV))
        for h in handles:
            h.remove()

    mtq.quantize(model, cfg, loop)
    enabled = {n: q for n, q in model.named_modules() if isinstance(q, TensorQuantizer) and q.is_enabled}
    assert len(enabled) == 2 * (7 * 2 + 2)
    kinds = {"weight_quantizer": 0, "input_quantizer": 0, "k_bmm_quantizer": 0, "v_bmm_quantizer": 0}
    for name, q in enabled.items():
        assert name in seen, name
        assert_bits_equal(q.amax.cpu().reshape(()), seen[name].reshape(()).to(q.amax.dtype), name)
        kinds[name.rsplit(".", 1)[1]] += 1
    assert kinds == {"weight_quantizer": 14, "input_quantizer": 14, "k_bmm_quantizer": 2, "v_bmm_quantizer": 2}
    assert model.get_submodule("model.layers.1.mlp.down_proj").weight.shape == (4096, 14336)
    k_seen = model.get_submodule("model.layers.0.self_attn.k_bmm_quantizer")
    assert k_seen.amax.numel() == 1 and float(k_seen.amax) > 0


def test_export_reports_a_scale_that_is_not_positive_in_the_getter_s_words(tmp_path):
    """The "scaling factor is positive" assertions of the per-layer getters (reference:
    qtensor/nvfp4_tensor.py:112-114, export/quant_utils.py:229) are made together when the export
    ends -- one host synchronisation instead of one per layer; a failure is an ``AssertionError``
    with the failing getter's own message.  Outside an export the getter asserts on the spot."""
    from modelopt_amd.torch.quantization.qtensor import NVFP4QTensor

    model, _ = _quantized(copy.deepcopy(mtq.NVFP4_DEFAULT_CFG))
    bad = model.get_submodule("model.layers.1.mlp.down_proj").input_quantizer
    bad.amax = torch.zeros_like(bad.amax)
    with pytest.raises(AssertionError, match="activation scaling factor .* not positive"):
        NVFP4QTensor.get_activation_scaling_factor(bad)
    with pytest.raises(AssertionError, match="activation scaling factor .* not positive"):
        export_hf_checkpoint(model, export_dir=tmp_path)
