"""Unified HF-layout export: packed weights + scales in safetensors, ``hf_quant_config.json``
and ``config.json["quantization_config"]``.

Reference: modelopt/torch/export/unified_export_hf.py:233-391 (``_export_quantized_weight``),
:394-553 (``_export_hf_checkpoint``), :556-620 (``export_hf_checkpoint``).  NVFP4 linears are
packed in ONE multi-tensor kernel launch over the whole model instead of module by module.
"""

import contextlib
import json
import warnings
from pathlib import Path
from typing import Any

import torch
from torch import nn

from ... import _hip
from ..quantization.nn import SequentialQuantizer, TensorQuantizer
from ..quantization import modes
from ..quantization.overflow import nvfp4_quantize_flags
from ..quantization.qtensor import NVFP4QTensor, QTensorWrapper
from ..quantization.utils import deferred_scale_checks, is_quantized_linear, true_divide
from .model_config import *  # noqa: F403
from .quant_utils import (fuse_prequant_layernorm, fuse_prequant_to_linear,
                          get_activation_scaling_factor, get_quant_config,
                          get_quantization_format,
                          get_weight_block_size, get_weight_scaling_factor,
                          get_weight_scaling_factor_2, postprocess_state_dict,
                          preprocess_linear_fusion, to_quantized_weight)

__all__ = ["export_hf_checkpoint", "convert_hf_quant_config_format",
           "requantize_resmooth_fused_llm_layers"]


def _register_input_scale(module, input_quantizer):
    # the reference asks `"disabled" not in repr(input_quantizer)`; a TensorQuantizer prints that word
    # exactly when it is disabled, and formatting the amax for the repr would wait for the device
    enabled = (not input_quantizer._disabled if isinstance(input_quantizer, TensorQuantizer)
               else "disabled" not in repr(input_quantizer)) if input_quantizer is not None else False
    if enabled and input_quantizer.amax is not None:
        module.register_buffer("input_scale", get_activation_scaling_factor(module).squeeze())


def _export_quantized_weight(module: nn.Module, dtype: torch.dtype):
    """Replace ``module.weight`` by its packed form and register ``weight_scale``,
    ``weight_scale_2`` and ``input_scale`` buffers."""
    fmt = get_quantization_format(module)
    if fmt == QUANTIZATION_NONE:
        return
    block = get_weight_block_size(module)
    wq, iq = module.weight_quantizer, getattr(module, "input_quantizer", None)
    weight = module.weight
    if fmt == QUANTIZATION_FP8:
        wq._amax = wq._amax.to(torch.float32)
        if wq._amax.dim() == 1:
            wsf = torch.tensor(wq.amax.item() / wq.maxbound)
        else:
            wsf = true_divide(wq.amax, wq.maxbound).clone().detach()
        module.register_buffer("weight_scale", wsf)
        if iq is not None and hasattr(iq, "_amax"):
            iq._amax = iq._amax.to(torch.float32)
            module.register_buffer("input_scale", get_activation_scaling_factor(module).squeeze())
    else:
        if fmt == QUANTIZATION_FP8_PB_REAL:
            # already packed by ``compress``: the scales live on the quantizer
            module.register_buffer("weight_scale", wq._scale.to(torch.float32))
            del wq._scale
        elif fmt not in (QUANTIZATION_NVFP4, QUANTIZATION_NVFP4_AWQ):
            module.register_buffer("weight_scale", get_weight_scaling_factor(module))
        _register_input_scale(module, iq)
    if fmt in (QUANTIZATION_NVFP4, QUANTIZATION_NVFP4_AWQ, QUANTIZATION_W4A8_AWQ,
               QUANTIZATION_W4A8_NVFP4_FP8):
        module.register_buffer("weight_scale_2", get_weight_scaling_factor_2(module).squeeze())

    weight_scale = getattr(module, "weight_scale", None)
    weight_scale_2 = getattr(module, "weight_scale_2", None)
    if isinstance(weight, QTensorWrapper):
        quantized = weight.data                 # packed by ``compress`` already
    elif fmt in (QUANTIZATION_NVFP4, QUANTIZATION_NVFP4_AWQ):
        # block scales and codes from one pass over the weight
        qt, weight_scale, _ = NVFP4QTensor.quantize(weight.data.to(dtype), block,
                                                    weights_scaling_factor_2=weight_scale_2)
        quantized = qt._quantized_data
    else:
        quantized = to_quantized_weight(weight.data.to(dtype), weight_scale, fmt, weight_scale_2, block)
    module.weight = nn.Parameter(quantized, requires_grad=False)
    if weight_scale is not None:
        module.register_buffer("weight_scale", weight_scale)


def _export_nvfp4_batched(modules: list[nn.Module], dtype: torch.dtype):
    """All NVFP4 linears of the model in one launch (bf16 weights, K % 16 == 0)."""
    weights = [m.weight.data for m in modules]
    amax = torch.stack([m.weight_quantizer._amax.reshape(()).float() for m in modules]).to(
        weights[0].device)
    # the kernel derives wsf2 = amax / (6 * 448)
    plan = _hip.Nvfp4QuantizePlan(weights, amax, flags=nvfp4_quantize_flags())
    packed, wsf, wsf2 = plan.run()
    for i, m in enumerate(modules):
        _register_input_scale(m, getattr(m, "input_quantizer", None))
        m.register_buffer("weight_scale_2", wsf2[i].clone())
        m.weight = nn.Parameter(packed[i], requires_grad=False)
        m.register_buffer("weight_scale", wsf[i])


def _fusable_groups(model: nn.Module):
    """(q, k, v) and (gate, up) projections that share an input."""
    for module in model.modules():
        for names in (("q_proj", "k_proj", "v_proj"), ("gate_proj", "up_proj")):
            group = [getattr(module, n, None) for n in names]
            if all(g is not None and is_quantized_linear(g) for g in group):
                yield group


def _is_layernorm(module: nn.Module) -> bool:
    return any(n in type(module).__name__ for n in ("LayerNorm", "RMSNorm"))


def _quantizer_on(q) -> bool:
    if isinstance(q, SequentialQuantizer):
        return any(m.is_enabled for m in q)
    return isinstance(q, TensorQuantizer) and q.is_enabled


_is_enabled_quantizer = _quantizer_on   # the reference's name for it (unified_export_hf.py:80-87)


@contextlib.contextmanager
def _every_quantizer_off(model: nn.Module):
    """What ``set_quantizer_by_cfg_context(model, {"*": {"enable": False}})`` does for the dummy
    forward below, without saving and restoring the whole state of several hundred quantizers:
    the enabled ones are switched off and back on."""
    switched = [m for m in model.modules() if isinstance(m, TensorQuantizer) and not m._disabled]
    for q in switched:
        q._disabled = True
    try:
        yield
    finally:
        for q in switched:
            q._disabled = False


def requantize_resmooth_fused_llm_layers(model: nn.Module):
    """Unify what an inference engine will fuse (reference: unified_export_hf.py:90-231).

    Quantised linears that read the same tensor (q/k/v, gate/up) are found with forward hooks
    during one two-token dummy forward with every quantizer switched off; each group gets one
    averaged ``pre_quant_scale`` (weights re-smoothed), one input amax and one per-tensor weight
    amax.  For AWQ formats, when the shared input is the output of a layernorm, the scale is
    folded into the layernorm weight.  A model that cannot run on token ids falls back to
    grouping by the usual projection names (no layernorm folding).
    """
    input_to_linear: dict = {}
    output_to_layernorm: dict = {}
    model_format = get_quantization_format(model)
    if model_format is not None and "nvfp4_awq" in model_format.lower():
        fuse_prequant_to_linear(model)      # o_proj's scale into v_proj, down_proj's into up_proj

    def linear_hook(module, args, output):
        input_to_linear.setdefault(args[0], []).append(module)

    def norm_hook(module, args, output):
        output_to_layernorm[output] = module

    handles = []
    for module in model.modules():
        if _is_layernorm(module):
            handles.append(module.register_forward_hook(norm_hook))
        elif is_quantized_linear(module) and (_quantizer_on(module.input_quantizer)
                                              or _quantizer_on(module.weight_quantizer)):
            handles.append(module.register_forward_hook(linear_hook))
    groups = None
    try:
        device = next(model.parameters()).device
        with torch.no_grad(), _every_quantizer_off(model):
            model(torch.ones([1, 2], dtype=torch.long, device=device))
        groups = list(input_to_linear.items())
    except Exception as err:  # noqa: BLE001 -- any failure of a foreign forward means "not an LLM"
        warnings.warn(f"dummy forward for layer fusion failed ({type(err).__name__}: {err}); "
                      "grouping q/k/v and gate/up projections by name")
    finally:
        for h in handles:
            h.remove()
    if groups is None:
        groups = [(None, g) for g in _fusable_groups(model)]
    for tensor, modules in groups:
        fmt = get_quantization_format(modules[0])
        if len(modules) > 1 and fmt not in (QUANTIZATION_FP8, QUANTIZATION_NONE,
                                            QUANTIZATION_FP8_PB_REAL):
            preprocess_linear_fusion(modules)
        if (fmt is not QUANTIZATION_NONE and fmt is not None and "awq" in fmt and tensor is not None
                and tensor in output_to_layernorm
                and modules[0].input_quantizer.pre_quant_scale is not None):
            fuse_prequant_layernorm(output_to_layernorm[tensor], modules)


def _export_hf_checkpoint(model: nn.Module, dtype: torch.dtype | None = None):
    # the "scaling factor is positive" assertions of the per-layer getters are one host
    # synchronisation each if made on the spot; they are made together when the export ends
    with deferred_scale_checks():
        return _export_hf_checkpoint_unchecked(model, dtype)


def _export_hf_checkpoint_unchecked(model: nn.Module, dtype: torch.dtype | None = None):
    if dtype is None:
        dtype = next(model.parameters()).dtype
    requantize_resmooth_fused_llm_layers(model)
    quant_config = get_quant_config(model)
    kv_format = quant_config["quantization"]["kv_cache_quant_algo"]
    kv_bound = {KV_CACHE_NVFP4: 6 * 448, KV_CACHE_FP8: 448}.get(kv_format, 0)

    linears = [m for m in model.modules()
               if is_quantized_linear(m) and get_quantization_format(m) != QUANTIZATION_NONE]
    batched = [m for m in linears
               if get_quantization_format(m) == QUANTIZATION_NVFP4 and m.weight.dtype == torch.bfloat16
               and dtype == torch.bfloat16 and m.weight.shape[-1] % 16 == 0 and m.weight.is_cuda
               and get_weight_block_size(m) == 16 and m.weight.is_contiguous()]
    if batched:
        _export_nvfp4_batched(batched, dtype)
    done = set(map(id, batched))
    for m in linears:
        if id(m) not in done:
            _export_quantized_weight(m, dtype)
    state = postprocess_state_dict(model.state_dict(), kv_bound, kv_format)
    if modes.one_launch_dynamic_quant() and _hip.fused_gave_up():
        warnings.warn("a one-launch quantize kernel could not run all its workgroups at once and "
                      "finished the slow way (same results); something else holds the device -- "
                      "consider set_one_launch_dynamic_quant(False)")
    return state, quant_config


def convert_hf_quant_config_format(input_config: dict[str, Any]) -> dict[str, Any]:
    """``hf_quant_config.json`` -> the ``quantization_config`` block written into config.json
    (reference: export/convert_hf_config.py:21-130)."""
    q = input_config.get("quantization", {})
    algo = q.get("quant_algo")
    out: dict[str, Any] = {}
    group = None
    if algo == "FP8":
        group = {"input_activations": {"dynamic": False, "num_bits": 8, "type": "float"},
                 "weights": {"dynamic": False, "num_bits": 8, "type": "float"}, "targets": ["Linear"]}
    elif algo == "NVFP4":
        gs = q.get("group_size", 16)
        group = {"input_activations": {"dynamic": False, "num_bits": 4, "type": "float", "group_size": gs},
                 "weights": {"dynamic": False, "num_bits": 4, "type": "float", "group_size": gs},
                 "targets": ["Linear"]}
    if group is not None:
        out["config_groups"] = {"group_0": group}
    out["ignore"] = q.get("exclude_modules") or []
    if algo:
        out["quant_algo"] = algo
    if q.get("kv_cache_quant_algo"):
        out["kv_cache_scheme"] = {"dynamic": False, "num_bits": 8, "type": "float"} if q[
            "kv_cache_quant_algo"] == "FP8" else q["kv_cache_quant_algo"]
    if input_config.get("producer"):
        out["producer"] = input_config["producer"]
    out["quant_method"] = "modelopt"
    return out


def export_hf_checkpoint(model: nn.Module, dtype: torch.dtype | None = None,
                         export_dir: Path | str = "/tmp", save_modelopt_state: bool = False):
    """Write ``model.safetensors``, ``hf_quant_config.json`` and ``config.json`` to
    ``export_dir``.  ``model.config`` (a dict or an object with ``to_dict``) is used for
    ``config.json`` when present."""
    from safetensors.torch import save_file

    export_dir = Path(export_dir)
    export_dir.mkdir(parents=True, exist_ok=True)
    state, hf_quant_config = _export_hf_checkpoint(model, dtype)
    with open(export_dir / "hf_quant_config.json", "w") as f:
        json.dump(hf_quant_config, f, indent=4)
    tensors = {k: v.detach().contiguous().cpu() for k, v in state.items() if isinstance(v, torch.Tensor)}
    save_file(tensors, str(export_dir / "model.safetensors"))
    cfg = getattr(model, "config", {})
    cfg = cfg.to_dict() if hasattr(cfg, "to_dict") else dict(cfg) if isinstance(cfg, dict) else {}
    cfg["quantization_config"] = convert_hf_quant_config_format(hf_quant_config)
    with open(export_dir / "config.json", "w") as f:
        json.dump(cfg, f, indent=4, default=str)
    return state, hf_quant_config
