"""User-facing API: ``quantize``, ``calibrate`` and helpers.

Reference: modelopt/torch/quantization/model_quant.py:53-118 (``calibrate``), :136-231
(``quantize``).  ``quantize(model, config, forward_loop)`` converts the model in place (module
swap + quantizer attributes) and runs the configured calibration algorithm; the reference's
mode registry / state manager (``apply_mode``) is not reproduced.
"""

import fnmatch
import inspect
import marshal
import warnings
from collections.abc import Callable

import torch
from torch import nn

from . import model_calib
from .config import QuantizeConfig, QuantizerAttributeConfig, normalize_algorithm
from .conversion import is_converted, replace_quant_module, set_quantizer_attribute, set_quantizer_by_cfg
from .nn import TensorQuantizer
from .utils import DeferredCheckError, deferred_scale_checks

__all__ = ["quantize", "calibrate", "disable_quantizer", "enable_quantizer", "print_quant_summary",
           "fold_weight", "postprocess_amax", "auto_quantize"]

ForwardLoop = Callable[[nn.Module], None]


def _full_attribute_cfg(cfg):
    """What pydantic validation of the reference's ``QuantizeConfig`` does to an attribute dict:
    it becomes a complete ``QuantizerAttributeConfig`` (unspecified fields take their defaults),
    so a later pattern replaces, rather than patches, what an earlier one set."""
    if isinstance(cfg, QuantizerAttributeConfig):
        return cfg
    if isinstance(cfg, (list, tuple)):
        return [_full_attribute_cfg(c) for c in cfg]
    if isinstance(cfg, dict):
        try:
            return QuantizerAttributeConfig(**cfg)
        except Exception:
            # class-scoped entry such as "nn.BatchNorm1d": {"*": {...}}
            if all(isinstance(v, (dict, list, QuantizerAttributeConfig)) for v in cfg.values()):
                return {k: _full_attribute_cfg(v) for k, v in cfg.items()}
            raise
    raise TypeError(f"unsupported quantizer config entry: {cfg!r}")


_VALIDATED = {}   # marshalled plain config -> (validated quant_cfg, marshalled algorithm); a handful of entries


def _content_key(config):
    """The content of a config made of plain values only (exact dicts, lists, tuples, strings,
    numbers, booleans, None -- every named config is) as bytes; None for anything else.
    ``marshal`` refuses every other type, subclasses of the plain ones included, and keeps the
    order of a dict's entries, which decides which pattern wins."""
    try:
        return marshal.dumps(config)
    except ValueError:
        return None


def _validated(config):
    """``(quant_cfg with every entry a complete QuantizerAttributeConfig, algorithm)``.  A config
    made of plain values only is validated once per distinct content: the validated entries are
    never handed out or written to -- a quantizer copies what it takes from them -- so calls
    with an equal config can share them."""
    key = _content_key(config) if type(config) is dict else None
    if key is not None:
        hit = _VALIDATED.get(key)
        if hit is not None:
            return dict(hit[0]), marshal.loads(hit[1])
    parsed = config if isinstance(config, QuantizeConfig) else QuantizeConfig(**dict(config))
    quant_cfg = {k: _full_attribute_cfg(v) for k, v in parsed.quant_cfg.items()}
    if key is not None:
        algorithm = _content_key(parsed.algorithm)
        if algorithm is not None:
            if len(_VALIDATED) >= 32:
                _VALIDATED.clear()
            _VALIDATED[key] = (dict(quant_cfg), algorithm)
    return quant_cfg, parsed.algorithm


def _takes_no_argument(fn) -> bool:
    """``len(inspect.signature(fn).parameters) == 0`` without building the signature for a plain
    function or lambda."""
    code = getattr(fn, "__code__", None)
    if code is not None and type(fn).__name__ == "function" and not hasattr(fn, "__wrapped__"):
        return code.co_argcount + code.co_kwonlyargcount == 0 and not code.co_flags & 0x0C  # no *args / **kwargs
    return len(inspect.signature(fn).parameters) == 0


def calibrate(model: nn.Module, algorithm="max", forward_loop: ForwardLoop | None = None) -> nn.Module:
    """Run a calibration algorithm (``"max"``, ``"smoothquant"``, ``"awq_lite"``, a dict with
    ``"method"``, or ``None``) on a converted model."""
    method, kwargs = normalize_algorithm(algorithm)
    if method is None:
        return model
    if forward_loop is not None and _takes_no_argument(forward_loop):
        # the pre-model-argument calling convention (reference: model_quant.py:81-96)
        warnings.warn("forward_loop should take model as argument, but got forward_loop without any"
                      " arguments. This usage will be deprecated in future versions.", DeprecationWarning)
        no_arg_loop = forward_loop

        def forward_loop(model):
            return no_arg_loop()
    training = model.training
    model.eval()
    try:
        # every "amax / scale is finite and non-negative" check of the algorithm and the final look at
        # what it left on the quantizers are one device reduction and one host synchronisation
        with deferred_scale_checks() as checks:
            if method == "max":
                model_calib.max_calibrate(model, forward_loop, kwargs.get("distributed_sync", True))
            elif method == "mse":
                model_calib.mse_calibrate(model, forward_loop, kwargs.get("distributed_sync", True),
                                          kwargs.get("num_steps", 10), kwargs.get("start_multiplier", 0.25),
                                          kwargs.get("stop_multiplier", 4.0))
            elif method == "smoothquant":
                model_calib.smoothquant(model, forward_loop, alpha=kwargs.get("alpha", 1.0))
            elif method in ("awq_clip", "awq_full"):
                model_calib.awq(model, forward_loop, method, **kwargs)
            elif method == "awq_lite":
                model_calib.awq(model, forward_loop, "awq_lite", alpha_step=kwargs.get("alpha_step", 0.1),
                                debug=kwargs.get("debug", False))
            quantizers = [(n, m) for n, m in model.named_modules() if isinstance(m, TensorQuantizer)]
            attrs = ("_amax", "_pre_quant_scale")
            checks.report = [t for _, m in quantizers for a in attrs
                             if isinstance(t := getattr(m, a, None), torch.Tensor)]
        # only a failure is walked through to name the culprit
        if not checks.report_ok:
            for name, module in quantizers:
                for attr in attrs:
                    module.validate_attr(attr_name=attr, warn_error=True, name=name)
    except DeferredCheckError:
        # a calibrator whose running maximum is bad says so in its own words (the reference's
        # per-collect assertions); anything else keeps the message of the deferred check
        for module in model.modules():
            cal = getattr(module, "_calibrator", None) if isinstance(module, TensorQuantizer) else None
            if getattr(cal, "_acc", None) is not None and hasattr(cal, "_validated"):
                cal._validated = False
                cal.compute_amax()
        raise
    finally:
        model.train(training)
    return model


def quantize(model: nn.Module, config, forward_loop: ForwardLoop | None = None) -> nn.Module:
    """Quantise and calibrate ``model`` in place and return it.

    ``config`` is ``{"quant_cfg": {wildcard: quantizer attributes, ...}, "algorithm": ...}`` (for
    instance ``NVFP4_DEFAULT_CFG``); ``forward_loop(model)`` feeds the calibration data.
    """
    quant_cfg, algorithm = _validated(config)
    if not is_converted(model):
        replace_quant_module(model)
    set_quantizer_by_cfg(model, quant_cfg)
    return calibrate(model, algorithm, forward_loop=forward_loop)


def disable_quantizer(model: nn.Module, wildcard_or_filter_func):
    set_quantizer_attribute(model, wildcard_or_filter_func, {"enable": False})


def enable_quantizer(model: nn.Module, wildcard_or_filter_func):
    set_quantizer_attribute(model, wildcard_or_filter_func, {"enable": True})


def auto_quantize(*args, **kwargs):
    """Per-layer format search (reference: model_quant.py:236-480, algorithms.py).  Not part of
    the path built here: it sits on the reference's searcher / mode machinery."""
    raise NotImplementedError(
        "auto_quantize (per-layer format search) is not part of this build; quantize with one of "
        "the named configs or a custom quant_cfg instead")


def print_quant_summary(model: nn.Module):
    count = 0
    for name, mod in model.named_modules():
        if isinstance(mod, TensorQuantizer):
            print(f"{name:80} {mod}")
            count += 1
    print(f"{count} TensorQuantizers found in model")


def fold_weight(model: nn.Module):
    for module in model.modules():
        if hasattr(module, "fold_weight") and hasattr(module, "weight_quantizer"):
            module.fold_weight()


def postprocess_amax(model: nn.Module, key: str, post_process_fn) -> None:
    """Apply ``post_process_fn`` to the amax of every quantizer whose name matches ``key``."""
    for name, module in model.named_modules():
        if isinstance(module, TensorQuantizer) and fnmatch.fnmatch(name, key) and module.amax is not None:
            module.amax = post_process_fn(module.amax)
