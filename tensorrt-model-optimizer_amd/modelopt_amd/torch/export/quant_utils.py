"""Scaling factors, packed weights and state-dict post-processing for export.

Reference: modelopt/torch/export/quant_utils.py (:68-91, :214-320, :373-534, :602-738, :741-834,
:860-983, :1132-1185, :1190-1288).  The packing itself runs in the HIP kernels.
"""

import fnmatch
import warnings
from types import SimpleNamespace
from typing import Any

import torch
from torch import nn

from ... import __version__, _hip
from ..quantization.nn import SequentialQuantizer, TensorQuantizer
from ..quantization.qtensor import FP8QTensor, MXFP4QTensor, NVFP4QTensor, QTensorWrapper
from ..quantization.utils import (all_positive, quantizer_attr_names, reduce_block_amax, true_divide,
                                  weight_attr_names)
from .model_config import *  # noqa: F403

_NVFP4_FAMILY = (QUANTIZATION_NVFP4, QUANTIZATION_NVFP4_AWQ, QUANTIZATION_W4A8_NVFP4_FP8)
_MXFP4_FAMILY = (QUANTIZATION_MXFP4, QUANTIZATION_W4A8_MXFP4_FP8)

__all__ = [
    "get_scaling_factor_from_weight", "get_scaling_factor", "get_activation_scaling_factor",
    "get_weight_scaling_factor", "get_weight_scaling_factor_2", "get_prequant_scaling_factor",
    "get_kv_cache_dtype", "get_weight_block_size", "get_quantization_format",
    "process_layer_quant_config", "pack_int4_in_uint8", "to_quantized_weight",
    "postprocess_state_dict", "preprocess_linear_fusion", "fuse_prequant_layernorm",
    "fuse_prequant_to_linear",
    "get_quant_config", "all_items_same", "adjust_attn_amax_values", "get_kv_cache_scaling_factor",
    "from_quantized_weight",
]


def get_scaling_factor_from_weight(weight, group_size) -> torch.Tensor:
    """``max|w| / 7`` per group of ``group_size`` input channels (``/127`` per row when 0)."""
    n, k = weight.shape
    if group_size != 0:
        if k % group_size != 0:
            raise NotImplementedError("Weight shape is not divisible for block size for block quantization.")
        amax = reduce_block_amax(weight.contiguous(), {-1: group_size}).float()
        bound = 7.0
    else:
        acc = torch.zeros(n, dtype=torch.float32, device=weight.device)
        _hip.absmax_into(weight.contiguous(), acc, 1, n, k)
        amax, bound = acc, 127.0
    sf = true_divide(amax, bound)
    sf[sf == 0] = 1.0
    return sf


def maybe_transpose_expert_weight_dimensions(weight, weight_scale=None, is_bmm_expert_weight=True):
    """Swap the last two dims of a stacked expert weight (and of its scale) between the
    (experts, input, output) and (experts, output, input) layouts; anything else is returned as
    it is (reference: export/quant_utils.py:94-123)."""
    if not is_bmm_expert_weight or weight.dim() != 3:
        return weight, weight_scale
    return weight.transpose(-2, -1), None if weight_scale is None else weight_scale.transpose(-2, -1)


def resmooth_and_get_scale(merged_weights, pre_quant_scales, ranks, group_size, new_pre_quant_scale=None,
                           quantization=QUANTIZATION_NONE):
    """Bring the row chunks of ``merged_weights`` (one per rank, each smoothed with its own
    ``pre_quant_scale``) to one shared scale -- the mean unless given -- and recompute their block
    scales (reference: export/quant_utils.py:126-185).  Returns (weights, scales, shared scale).
    ``w * p / p_new`` is two tensor operations in the weight dtype, as in the reference."""
    if new_pre_quant_scale is None:
        new_pre_quant_scale = torch.stack(pre_quant_scales).mean(dim=0)
    assert len(pre_quant_scales) > 0 and new_pre_quant_scale.numel() == merged_weights.shape[1], (
        "Shape of pre_quant_scales and weights do not match.")
    chunks = torch.chunk(merged_weights, ranks, dim=0)
    weights, scales = [], []
    for chunk, own in zip(chunks, pre_quant_scales):
        weight = chunk * own.type(chunk.dtype) / new_pre_quant_scale.type(chunk.dtype)
        weights.append(weight)
        if quantization == QUANTIZATION_NVFP4_AWQ:
            # block scales travel as bytes so that they can be concatenated
            scales.append(NVFP4QTensor.get_weights_scaling_factor(weight, group_size)[0].view(torch.uint8))
        else:
            scales.append(get_scaling_factor_from_weight(weight, group_size))
    scales = torch.cat(scales, dim=0)
    if quantization == QUANTIZATION_NVFP4_AWQ:
        scales = scales.view(torch.float8_e4m3fn)
    return torch.cat(weights, dim=0), scales, new_pre_quant_scale


def get_scaling_factor(quantizer: TensorQuantizer) -> torch.Tensor | None:
    if not quantizer.is_enabled:
        return None
    amax = quantizer.export_amax()
    if amax is None:
        return None
    if quantizer.num_bits == (2, 1):
        sf = NVFP4QTensor.get_weights_scaling_factor_2_from_quantizer(quantizer)
    else:
        sf = true_divide(amax.float(), quantizer.maxbound)
    assert all_positive(sf, lambda: f"scaling factor {sf} not positive."), f"scaling factor {sf} not positive."
    return sf


def get_activation_scaling_factor(module: nn.Module, input_quantizer_name: str = "input_quantizer"):
    q = getattr(module, input_quantizer_name, None)
    if q is None:
        return None
    if get_quantization_format(module) in (QUANTIZATION_NVFP4, QUANTIZATION_NVFP4_AWQ):
        return NVFP4QTensor.get_activation_scaling_factor(q)
    return get_scaling_factor(q)


def get_weight_scaling_factor(module: nn.Module, weight_name: str = "weight"):
    weight = getattr(module, weight_name)
    wq = getattr(module, quantizer_attr_names(weight_name).weight_quantizer, None)
    if wq is None:
        return None
    if isinstance(wq, SequentialQuantizer):
        return get_scaling_factor(wq[0])
    fmt = get_quantization_format(module)
    if fmt in _NVFP4_FAMILY:
        if fmt == QUANTIZATION_W4A8_NVFP4_FP8:
            # the consumer dequantises the weight to FP8 (range 448), so the block scales are
            # laid out against amax / 448 rather than amax / (6 * 448)
            wsf2 = true_divide(wq._amax.float(), 448.0)
        else:
            wsf2 = NVFP4QTensor.get_weights_scaling_factor_2_from_quantizer(wq)
        return NVFP4QTensor.get_weights_scaling_factor(weight, wq.block_sizes[-1],
                                                       wsf2.to(weight.device))[0]
    if fmt in _MXFP4_FAMILY:
        return MXFP4QTensor.quantize(weight, block_size=wq.block_sizes[-1])[1].reshape(
            *weight.shape[:-1], -1)
    return get_scaling_factor(wq)


def get_weight_scaling_factor_2(module: nn.Module, weight_name: str = "weight"):
    wq = getattr(module, quantizer_attr_names(weight_name).weight_quantizer, None)
    if wq is None:
        return None
    fmt = get_quantization_format(module)
    if fmt in (QUANTIZATION_NVFP4, QUANTIZATION_NVFP4_AWQ):
        return NVFP4QTensor.get_weights_scaling_factor_2_from_quantizer(wq)
    if fmt == QUANTIZATION_W4A8_NVFP4_FP8:
        return true_divide(wq._amax.float(), 448.0)
    if not isinstance(wq, SequentialQuantizer) or not wq[-1].is_enabled:
        return None
    assert len(wq) == 2, "modelopt only supports 2 sequential quantization layers for now"
    return get_scaling_factor(wq[-1])


def get_prequant_scaling_factor(module: nn.Module):
    q = getattr(module, "input_quantizer", None)
    if q is not None and hasattr(q, "_pre_quant_scale"):
        return q._pre_quant_scale.squeeze()
    return None


def get_kv_cache_dtype(modules) -> str | None:
    if isinstance(modules, nn.Module):
        modules = [modules]
    bits = []
    for module in modules:
        for name in ("k_bmm_quantizer", "v_bmm_quantizer", "output_quantizer"):
            q = getattr(module, name, None)
            if q is not None and q.is_enabled:
                bits.append(q.num_bits)
    if (4, 3) in bits:
        return KV_CACHE_FP8
    if 8 in bits:
        return KV_CACHE_INT8
    if (2, 1) in bits:
        return KV_CACHE_NVFP4
    return QUANTIZATION_NONE


def get_weight_block_size(module: nn.Module, weight_name: str = "weight") -> int:
    wq = getattr(module, quantizer_attr_names(weight_name).weight_quantizer, None)
    if wq is None:
        return 0
    if isinstance(wq, SequentialQuantizer):
        wq = wq[0]
    if not wq.is_enabled:
        return 0
    return wq.block_sizes[-1] if wq.block_sizes else 0


def get_quantization_format(module) -> str | None:
    """Format string of the first quantised weight found in ``module`` or its children."""

    def of_layer(layer, names):
        wq = getattr(layer, names.weight_quantizer, None)
        iq = getattr(layer, names.input_quantizer, None)
        if wq is None or not wq.is_enabled:
            return QUANTIZATION_NONE
        if isinstance(wq, SequentialQuantizer):
            assert len(wq) == 2 and wq[0].num_bits == 4 and wq[1].num_bits == (4, 3), (
                "Unsupported SequentialQuantizer configuration")
            return QUANTIZATION_W4A8_AWQ
        if wq.num_bits == 4:
            assert wq.block_sizes and wq.block_sizes[-1] > 0, "Invalid block_sizes for INT4 quantizer"
            return QUANTIZATION_INT4_AWQ
        if wq.num_bits == 8:
            return QUANTIZATION_INT8_SQ if iq is not None and iq.is_enabled else QUANTIZATION_INT8_WO
        if wq.num_bits == (4, 3):
            if wq.block_sizes:
                assert wq.block_sizes[-1] > 0, "Invalid block_sizes for FP8 quantizer"
                return QUANTIZATION_FP8_PB_WO if wq.fake_quant else QUANTIZATION_FP8_PB_REAL
            return QUANTIZATION_FP8_PC_PT if wq.axis == 0 else QUANTIZATION_FP8
        if wq.num_bits == (2, 1):
            blocks = wq.block_sizes
            scale_bits = blocks.get("scale_bits")
            if iq is not None and hasattr(iq, "_pre_quant_scale"):
                return QUANTIZATION_NVFP4_AWQ
            if getattr(layer, "fused_with_prequant", False):
                return QUANTIZATION_NVFP4_AWQ
            assert iq is not None, f"input_quantizer is None for {names}"
            fp8_input = (blocks.get("type", "static") == "dynamic" and iq.is_enabled
                         and iq.num_bits == (4, 3) and iq.block_sizes is None)
            if fp8_input and scale_bits == (8, 0):
                return QUANTIZATION_W4A8_MXFP4_FP8
            if fp8_input and scale_bits == (4, 3):
                return QUANTIZATION_W4A8_NVFP4_FP8
            if scale_bits == (4, 3):
                return QUANTIZATION_NVFP4
            if scale_bits == (8, 0):
                return QUANTIZATION_MXFP4
        raise NotImplementedError(f"Unsupported quantizer with num_bits: {wq.num_bits}")

    for weight_name in weight_attr_names(module):
        fmt = of_layer(module, quantizer_attr_names(weight_name))
        if fmt != QUANTIZATION_NONE:
            return fmt
    for _, child in module.named_children():
        fmt = get_quantization_format(child)
        if fmt != QUANTIZATION_NONE:
            return fmt
    return QUANTIZATION_NONE


def _summarize_exclude_modules(unquantized, quantized):
    """Shortest dot-boundary prefix wildcards that cover every unquantised layer and no quantised
    one (``a.b.c`` -> ``a*`` if nothing quantised starts with ``a``, else ``{a.b, a.b.*}`` ...)."""
    quantized = list(quantized)

    def hits_quantized(pattern):
        return any(fnmatch.fnmatchcase(q, pattern) for q in quantized)

    result: set[str] = set()
    for layer in unquantized:
        chosen = [layer]
        for i, ch in enumerate(layer):
            if ch != ".":
                continue
            single = [layer[:i] + "*"]
            pair = [layer[:i], layer[:i] + ".*"]
            done = False
            for cand in (single, pair):
                if any(hits_quantized(p) for p in cand):
                    continue
                chosen, done = cand, True
                break
            if done:
                break
        if all(c in result for c in chosen):
            continue
        result.update(chosen)
    return result


_LAYER_CONFIGS = {
    "fp8": lambda b: {"quant_algo": "FP8"},
    "fp8_pc_pt": lambda b: {"quant_algo": "FP8_PER_CHANNEL_PER_TOKEN"},
    "int4_awq": lambda b: {"quant_algo": "W4A16_AWQ", "group_size": b, "has_zero_point": False,
                           "pre_quant_scale": True},
    "w4a8_awq": lambda b: {"quant_algo": "W4A8_AWQ", "group_size": b, "has_zero_point": False,
                           "pre_quant_scale": True},
    "int8_wo": lambda b: {"quant_algo": "W8A16"},
    "int8_sq": lambda b: {"quant_algo": "W8A8_SQ_PER_CHANNEL"},
    "nvfp4": lambda b: {"quant_algo": "NVFP4", "group_size": b},
    "nvfp4_awq": lambda b: {"quant_algo": "NVFP4_AWQ", "group_size": b, "has_zero_point": False,
                            "pre_quant_scale": True},
    "w4a8_nvfp4_fp8": lambda b: {"quant_algo": "W4A8_NVFP4_FP8", "group_size": b,
                                 "has_zero_point": False, "pre_quant_scale": True},
    "w4a8_mxfp4_fp8": lambda b: {"quant_algo": "W4A8_MXFP4_FP8", "group_size": b},
}


def process_layer_quant_config(layer_config_dict):
    """Per-layer ``{name.quantization, name.awq_block_size}`` entries -> the ``quantization``
    section of ``hf_quant_config.json``."""
    out: dict[str, Any] = {"quant_algo": None, "kv_cache_quant_algo": None, "quantized_layers": {}}
    formats, last, excluded = set(), None, []
    for key, fmt in layer_config_dict.items():
        if "awq_block_size" in key:
            continue
        prefix = ".".join(key.rsplit(".", 1)[:-1])
        block = layer_config_dict.get(prefix + ".awq_block_size", 0)
        cfg = _LAYER_CONFIGS[fmt](block) if fmt in _LAYER_CONFIGS else {"quant_algo": fmt}
        if cfg["quant_algo"] != QUANTIZATION_NONE:
            formats.add(str(cfg))
            last = cfg
            out["quantized_layers"][prefix] = cfg
        else:
            excluded.append(prefix)
    if len(formats) > 1:
        out["quant_algo"] = "MIXED_PRECISION"
    elif len(formats) == 1 and last is not None:
        out.update(last)
        out["exclude_modules"] = sorted(_summarize_exclude_modules(excluded, out["quantized_layers"].keys()))
        out.pop("quantized_layers")
    return out


def pack_int4_in_uint8(weight, weights_scaling_factor):
    """INT4-AWQ export pack: two's-complement nibbles, adjacent output rows share a byte;
    ``[.., N, K]`` -> uint8 ``[.., N / 2, K]``."""
    out_dim, in_dim = weight.shape[-2], weight.shape[-1]
    assert out_dim % 2 == 0, f"Cannot pack weight. Out dimension {out_dim} is not an even number."
    # the reference takes the block size to be in_dim // (number of scales per row) and indexes
    # the scales with column // block_size (export/quant_utils.py:701-706): when the blocks do
    # not tile the row (padded last block) that index runs past the last scale and it raises
    block_size = in_dim // weights_scaling_factor.shape[-1]
    if block_size == 0 or (in_dim - 1) // block_size >= weights_scaling_factor.shape[-1]:
        raise IndexError(
            f"cannot pack INT4 weight: {weights_scaling_factor.shape[-1]} scales per row do not tile "
            f"{in_dim} input channels (the last block is padded); the reference's pack fails the same way")
    # the quotient has the type tensor division gives it (export/quant_utils.py:704-706): fp32 with
    # the exporter's fp32 scales, the weight's own type when the scales share a 16-bit type with it
    via = torch.result_type(weight, weights_scaling_factor)
    if via not in (torch.float16, torch.bfloat16) or via != weight.dtype:
        via = torch.float32
    return _hip.int4_pack_rows(weight.contiguous(),
                               weights_scaling_factor.to(torch.float32).contiguous(), via)


def to_quantized_weight(weight, weights_scaling_factor, quantization: str,
                        weights_scaling_factor2=None, block_size=None):
    """Weight -> packed / cast storage for ``quantization``."""
    if weights_scaling_factor is not None:
        weights_scaling_factor = weights_scaling_factor.to(weight.device)
    if weights_scaling_factor2 is not None:
        weights_scaling_factor2 = weights_scaling_factor2.to(weight.device)
    if isinstance(weight, QTensorWrapper):
        return weight.data
    w = weight.contiguous()
    if quantization == QUANTIZATION_FP8:
        if weight.dtype == torch.float8_e4m3fn:
            return weight
        s = weights_scaling_factor
        if weight.dim() == 3:
            s = s.unsqueeze(-1)
        via = torch.result_type(w, s)  # 0-dim fp32 scale: the quotient is a tensor of w.dtype
        if s.numel() == 1:
            return _hip.real_quantize(w, s.reshape(1).contiguous(), 1, 1, w.numel(), via,
                                      _hip.MO_FMT_E4M3)
        return _hip.real_quantize(w, s.reshape(-1).contiguous(), 1, w.shape[0],
                                  w.numel() // w.shape[0], via, _hip.MO_FMT_E4M3)
    if quantization in (QUANTIZATION_INT8_SQ, QUANTIZATION_INT8_WO):
        s = weights_scaling_factor.reshape(-1).contiguous()
        return _hip.real_quantize(w, s, 1, w.shape[0], w.shape[1], torch.result_type(w, s[:, None]),
                                  _hip.MO_FMT_INT8)
    if quantization == QUANTIZATION_FP8_PB_WO:
        return FP8QTensor.quantize(weight, weights_scaling_factor.squeeze(),
                                   block_sizes={-1: block_size, -2: block_size})[0]._quantized_data
    if quantization == QUANTIZATION_FP8_PC_PT:
        if weight.dim() == 3:
            # stacked expert weights (export/quant_utils.py:780-810): one scale per expert, per
            # (expert, input channel) or per (expert, output channel), told apart by shape
            s = weights_scaling_factor
            experts, n, k = w.shape
            if s.dim() == 1:
                return _hip.real_quantize(w, s.contiguous(), 1, experts, n * k,
                                          torch.result_type(w, s[:, None, None]), _hip.MO_FMT_E4M3)
            if s.dim() == 2:
                if s.shape[0] != experts:
                    raise ValueError(
                        f"First dimension (num_experts) mismatch for FP8_PC_PT quantization. "
                        f"weight shape: {weight.shape}, scale shape: {s.shape}")
                if n == k:
                    raise ValueError(
                        f"Ambiguous scaling dimension for FP8_PC_PT quantization with square weight matrix. "
                        f"weight shape: {weight.shape}, scale shape: {s.shape}. "
                        f"Cannot determine if scaling should be applied to input_dim or output_dim.")
                via = torch.result_type(w, s.unsqueeze(-1))
                if s.shape[-1] == k:    # (experts, input_dim): the scale runs along the rows
                    return torch.stack([_hip.real_quantize(w[i], s[i].contiguous(), n, k, 1, via,
                                                           _hip.MO_FMT_E4M3) for i in range(experts)])
                if s.shape[-1] == n:    # (experts, output_dim)
                    return _hip.real_quantize(w, s.reshape(-1).contiguous(), 1, experts * n, k, via,
                                              _hip.MO_FMT_E4M3)
                raise ValueError(
                    f"Cannot determine correct unsqueeze dimension for FP8_PC_PT quantization. "
                    f"weight shape: {weight.shape}, scale shape: {s.shape}")
        s = weights_scaling_factor.reshape(-1).contiguous()
        return _hip.real_quantize(w, s, 1, w.shape[0], w.shape[1], torch.result_type(w, s[:, None]),
                                  _hip.MO_FMT_E4M3)
    if quantization in (QUANTIZATION_INT4_AWQ, QUANTIZATION_W4A8_AWQ):
        return pack_int4_in_uint8(weight, weights_scaling_factor)
    if quantization in _NVFP4_FAMILY:
        assert block_size is not None, "Block size not passed. Unable to quantize to NVFP4 format."
        assert weights_scaling_factor2 is not None, (
            "Weights scaling factor 2 not passed. Unable to quantize to NVFP4 format")
        # one global scale per expert of a stacked weight broadcasts over its matrix
        return NVFP4QTensor.quantize(
            weight, block_size, weights_scaling_factor,
            weights_scaling_factor2.view(-1, 1, 1) if weights_scaling_factor2.dim() != 0
            else weights_scaling_factor2)[0]._quantized_data
    if quantization in _MXFP4_FAMILY:
        return MXFP4QTensor.quantize(weight, block_size=block_size)[0]._quantized_data
    raise NotImplementedError(f"quantization format {quantization} not supported")


def postprocess_state_dict(state_dict: dict, maxbound: float, quantization: str | None) -> dict:
    """Drop quantizer internals, rename KV amax to ``k_proj.k_scale`` / ``v_proj.v_scale``
    (``amax / maxbound``, at least 1 for FP8) and input ``_pre_quant_scale`` to
    ``pre_quant_scale``."""
    replacements = {
        "k_bmm_quantizer._amax": "k_proj.k_scale",
        "v_bmm_quantizer._amax": "v_proj.v_scale",
        "input_quantizer._pre_quant_scale": "pre_quant_scale",
    }
    skip_keys = ["output_quantizer", "_amax", "_bias_value", "input_quantizer._pre_quant_scale"]
    out = {}
    for key, value in state_dict.items():
        if all(s not in key for s in skip_keys):
            out[key] = value
            continue
        for old, new in replacements.items():
            if key.endswith(old):
                prefix = key[: -len(old)]
                if "_amax" in key:
                    assert quantization in (KV_CACHE_FP8, KV_CACHE_NVFP4), "Invalid KV cache quantization format."
                    assert maxbound > 0, "Maxbound must be greater than zero."
                    value = true_divide(value.float(), maxbound)
                    if quantization == KV_CACHE_FP8:
                        value.clamp_(min=1.0)
                out[prefix + new] = value
                break
    for key, value in out.items():
        if "scale" in key and isinstance(value, torch.Tensor) and value.dim() == 3 and value.shape[0] == 1:
            out[key] = value.squeeze(0)
    drop = [k for k in out if any(k.endswith("weight_quantizer." + q)
                                  for q in ("_scale", "_double_scale", "_scale_zeros"))]
    seen = {}
    for key, value in out.items():
        if isinstance(value, torch.Tensor) and value.numel() > 0:
            ptr = value.data_ptr()
            if ptr in seen:
                drop.append(key)  # tied weight: keep the first name only
            else:
                seen[ptr] = key
    for key in drop:
        out.pop(key, None)
    return out


def all_items_same(items):
    return all(x == items[0] for x in items)


def _update_pre_quant_scale(module, new_pre_quant_scale):
    """Re-smooth one linear to a new input scale: ``W <- dtype(f32(W) * old / new)`` (fp32), then
    recalibrate the weight amax (reference: export/quant_utils.py:991-1008)."""
    old = module.input_quantizer._pre_quant_scale
    dtype, dev = module.weight.dtype, module.weight.device
    ratio_num = old.to(dtype=torch.float32, device=dev)
    ratio_den = new_pre_quant_scale.to(dtype=torch.float32, device=dev)
    module.weight = nn.Parameter((module.weight.to(torch.float32) * ratio_num / ratio_den).to(dtype),
                                 requires_grad=False)
    module.input_quantizer.pre_quant_scale = new_pre_quant_scale
    _recalibrate_weight(module)


def _recalibrate_weight(module):
    from ..quantization.model_calib import enable_stats_collection, finish_stats_collection

    module.weight_quantizer.reset_amax()
    enable_stats_collection(module.weight_quantizer)
    module.weight_quantizer(module.weight)
    finish_stats_collection(module.weight_quantizer)


# (classes whose name contains one of these, (linear that takes the scale, linear that gives it up))
PQS_FUSE_MODULE_MAPPING = [
    # attn @ (x @ Wv^T) * s == attn @ (x @ (s[:, None] * Wv)^T): o_proj's input scale moves into the
    # output rows of v_proj
    (["LlamaAttention", "Qwen3Attention", "Qwen3MoeAttention"], ("v_proj", "o_proj")),
    # (act(gate(x)) * up(x)) * s == act(gate(x)) * (x @ (s[:, None] * Wup)^T): down_proj's into up_proj
    (["LlamaMLP", "Qwen3MLP", "Qwen3MoeMLP"], ("up_proj", "down_proj")),
]


def fuse_prequant_to_linear(model: nn.Module, fuse_grouped_heads=False):
    """Fold the input ``pre_quant_scale`` of ``o_proj`` / ``down_proj`` into the output rows of the
    linear that produces their input (``v_proj`` / ``up_proj``), recalibrate that linear's weight
    amax and drop the scale (reference: export/quant_utils.py:1011-1101).

    With grouped-query attention ``o_proj`` has more input channels than ``v_proj`` has rows:
    skipped with a warning, unless ``fuse_grouped_heads``, in which case the scale is first
    averaged over the query heads of each KV head (and ``o_proj`` re-smoothed to that average).
    """
    for module in model.modules():
        for class_names, (into_name, from_name) in PQS_FUSE_MODULE_MAPPING:
            if not any(n in type(module).__name__ for n in class_names):
                continue
            into, source = module.get_submodule(into_name), module.get_submodule(from_name)
            if not hasattr(getattr(source, "input_quantizer", None), "_pre_quant_scale"):
                continue
            scale = source.input_quantizer._pre_quant_scale
            rows = into.weight.shape[-2]
            if scale.numel() != rows:
                if not fuse_grouped_heads or "attention" not in type(module).__name__.lower():
                    warnings.warn(f"Skipping pattern fuse prequant for {type(module).__name__}"
                                  f"pre_quant_scale dim {scale.numel()} != out_channel dim {rows}")
                    continue
                kv_heads = module.config.num_key_value_heads
                head_dim = rows // kv_heads
                n_rep = scale.numel() // kv_heads // head_dim
                averaged = scale.view(kv_heads, n_rep, head_dim).mean(dim=1)
                _update_pre_quant_scale(
                    source, averaged.unsqueeze(1).expand(kv_heads, n_rep, head_dim).reshape(-1))
                scale = averaged.reshape(-1)
            into.weight = nn.Parameter(into.weight * scale.view(-1, 1))
            if getattr(into, "bias", None) is not None:
                into.bias = nn.Parameter(into.bias * scale)
            _recalibrate_weight(into)
            delattr(source.input_quantizer, "_pre_quant_scale")
            source.fused_with_prequant = True


def preprocess_linear_fusion(modules: list[nn.Module], resmooth_only=False):
    """Give linears that an engine will fuse (q/k/v, gate/up) one shared input amax and one
    shared per-tensor weight amax."""
    assert all_items_same([get_quantization_format(m) for m in modules]), (
        "Modules have different quantization formats")
    first = modules[0]
    if hasattr(first, "input_quantizer"):
        if first.input_quantizer.pre_quant_scale is not None:
            avg = torch.mean(torch.stack([m.input_quantizer.pre_quant_scale for m in modules]), dim=0)
            for m in modules:
                if not torch.equal(m.input_quantizer.pre_quant_scale, avg):
                    _update_pre_quant_scale(m, avg)
        if resmooth_only:
            return
        if first.input_quantizer.is_enabled and first.input_quantizer.amax is not None:
            assert first.input_quantizer.amax.numel() == 1, "Only support scalar input quant amax"
            amax = torch.max(torch.stack([m.input_quantizer.amax for m in modules]))
            for m in modules:
                m.input_quantizer.amax = amax
    if hasattr(first, "weight_quantizer") and not isinstance(first.weight_quantizer, SequentialQuantizer):
        wq = first.weight_quantizer
        if wq.is_enabled and wq.amax is not None and wq.amax.numel() == 1:
            amax = torch.max(torch.stack([m.weight_quantizer.amax for m in modules]))
            for m in modules:
                m.weight_quantizer.amax = amax


def fuse_prequant_layernorm(layernorm_module: nn.Module, modules: list[nn.Module]):
    """Fold the (already shared) input ``pre_quant_scale`` of ``modules`` into the weight and bias
    of the layernorm that feeds them, and drop it from the modules so that it is not exported
    (reference: export/quant_utils.py:1104-1129):
    ``norm(x) * w * s == norm(x) * (w * s)``."""
    scale = modules[0].input_quantizer._pre_quant_scale
    layernorm_module.weight = nn.Parameter(layernorm_module.weight * scale)
    if getattr(layernorm_module, "bias", None) is not None:
        layernorm_module.bias = nn.Parameter(layernorm_module.bias * scale)
    for module in modules:
        delattr(module.input_quantizer, "_pre_quant_scale")
        module.fused_with_prequant = True


def get_quant_config(model: nn.Module) -> dict[str, Any]:
    """The ``hf_quant_config.json`` dictionary of a quantised model."""
    config: dict[str, Any] = {"producer": {"name": "modelopt", "version": __version__},
                              "quantization": {"quant_algo": None, "kv_cache_quant_algo": None}}
    layers = {}
    kv_format = QUANTIZATION_NONE
    off = SimpleNamespace(is_enabled=False)
    for name, module in dict(model.named_modules()).items():
        names = list(weight_attr_names(module))
        if any(hasattr(module, quantizer_attr_names(w).weight_quantizer) for w in names):
            layers[name + ".quantization"] = get_quantization_format(module)
            layers[name + ".awq_block_size"] = get_weight_block_size(module)
        if (getattr(module, "k_bmm_quantizer", off).is_enabled
                or getattr(module, "v_bmm_quantizer", off).is_enabled):
            fmt = get_kv_cache_dtype(module)
            assert kv_format in (QUANTIZATION_NONE, fmt), "Do not support mixed precision kv cache quantization"
            kv_format = fmt
    config["quantization"].update(process_layer_quant_config(layers))
    if kv_format is not None:
        config["quantization"]["kv_cache_quant_algo"] = kv_format
    return config


def adjust_attn_amax_values(module: nn.Module) -> None:
    """Give every direct child whose name contains ``q``, ``k`` or ``v`` and whose weight quantizer
    holds an amax the largest of those amax values, in place (reference: quant_utils.py:185-211).
    The maximum is taken and written on the device; no scalar comes back to the host."""
    layers = [child for name, child in module.named_children()
              if any(p in name for p in "qkv") and hasattr(child, "weight_quantizer")
              and getattr(child.weight_quantizer, "amax", None) is not None]
    if not layers:
        raise ValueError("No projection layers with the specified prefixes ('q', 'k', 'v') have amax attributes")
    top = torch.stack([layer.weight_quantizer.amax.float().max() for layer in layers]).max()
    assert top > 0, "max_amax must be positive."
    for layer in layers:
        amax = layer.weight_quantizer.amax
        amax.copy_(top.to(amax.dtype).expand_as(amax))


def get_kv_cache_scaling_factor(kv_module: nn.Module) -> list:
    """``[k_scale, v_scale]`` of an attention module's BMM quantizers, ``[None, None]`` without
    them; FP8 scales are raised to at least 1 (reference: quant_utils.py:348-370)."""
    if not hasattr(kv_module, "k_bmm_quantizer") or not hasattr(kv_module, "v_bmm_quantizer"):
        return [None, None]
    factors = [get_scaling_factor(getattr(kv_module, name)) for name in ("k_bmm_quantizer", "v_bmm_quantizer")]
    if get_kv_cache_dtype(kv_module) == KV_CACHE_FP8:
        for i, factor in enumerate(factors):
            if factor.item() > 0.5:
                warnings.warn(f"Warning: Large KV activation detected: {factor.item()}, "
                              "Quantized KV cache may lead to higher accuracy drop.")
            factors[i] = torch.clamp(factor.float().reshape(-1)[:1], min=1.0)
    return factors


def from_quantized_weight(weight, weights_scaling_factor, quantization: str, torch_dtype):
    """Back from the exported 8-bit storage to ``torch_dtype`` (reference: quant_utils.py:837-857):
    FP8 bytes times the per-tensor scale, INT8 rows times the per-row scale; wider tensors are
    only cast."""
    if weight.element_size() >= 2 or weights_scaling_factor is None or not quantization:
        return weight.to(torch_dtype)
    if quantization == QUANTIZATION_FP8:
        return weight.view(torch.float8_e4m3fn).to(torch_dtype) * weights_scaling_factor.to(torch_dtype)
    if quantization in (QUANTIZATION_INT8_SQ, QUANTIZATION_INT8_WO):
        return weight.to(torch_dtype) * weights_scaling_factor[:, None].to(torch_dtype)
    raise NotImplementedError(f"quantization format {quantization} not supported")
