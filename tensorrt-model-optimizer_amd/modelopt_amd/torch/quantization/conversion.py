"""Model conversion: swap modules for their quantised versions and apply a ``quant_cfg``.

Reference: modelopt/torch/quantization/conversion.py:56-67 (``convert_to_quantized_model``),
:176 (``replace_quant_module``), :207 (``set_quantizer_by_cfg``), :241
(``set_quantizer_attribute``).  The mode / state-manager machinery of the reference is not
reproduced; conversion acts on the model in place.
"""

import fnmatch
import functools
import re
import warnings
from contextlib import contextmanager
from typing import Any

from torch import nn

from .config import QuantizeConfig, QuantizerAttributeConfig
from .nn import QuantModuleRegistry, SequentialQuantizer, TensorQuantizer

__all__ = ["replace_quant_module", "set_quantizer_by_cfg", "set_quantizer_attribute",
           "set_quantizer_by_cfg_context", "register", "unregister"]


def replace_quant_module(model: nn.Module):
    """Recursively convert every registered module type found in ``model`` (in place)."""
    assert not is_converted(model), "Model must not be quantized!"
    from .plugins import CUSTOM_MODEL_PLUGINS  # late: the plugins import the module registry

    for plugin in CUSTOM_MODEL_PLUGINS:
        plugin(model)
    for name, child in list(model.named_modules()):
        if type(child) in QuantModuleRegistry:
            QuantModuleRegistry.convert(child)
    return model


def is_converted(model: nn.Module) -> bool:
    return any(isinstance(m, TensorQuantizer) for m in model.modules())


def set_quantizer_by_cfg(quant_model: nn.Module, quant_cfg: dict | QuantizeConfig):
    """Apply ``{wildcard or filter: attributes}`` to the quantizers of ``quant_model``.

    ``"default"`` is applied first to every quantizer; then each pattern in insertion order, so
    later entries win.  Keys that name a ``nn`` class (``"nn.BatchNorm1d"``) hold a nested
    ``{pattern: attributes}`` dict applied only under modules of that class.
    """
    quant_cfg = dict(quant_cfg)
    index = _quantizer_index(quant_model)  # walked once, shared by every pattern below
    # When every entry is a complete attribute set (what validation makes of a dict), an entry
    # replaces whatever an earlier one set: each quantizer then takes the last entry that matches
    # it, once, instead of every matching entry in turn.
    order = [("*", quant_cfg["default"], None)] if "default" in quant_cfg else []
    for pattern, cfg in quant_cfg.items():
        if pattern == "default":
            continue
        if isinstance(pattern, str) and pattern.startswith("nn.") and isinstance(cfg, dict) and all(
                isinstance(v, (dict, list, QuantizerAttributeConfig)) for v in cfg.values()):
            cls = getattr(nn, pattern[3:], None)
            if cls is not None:
                order += [(k, v, cls) for k, v in cfg.items()]
        else:
            order.append((pattern, cfg, None))
    if all(isinstance(k, str) and isinstance(v, QuantizerAttributeConfig) for k, v, _ in order) \
            and not any(isinstance(e[1], SequentialQuantizer) for e in index):
        order.reverse()
        for name, module, parent, _ in index:
            for pattern, cfg, cls in order:
                if (cls is None or isinstance(parent, cls)) and _compiled(pattern)(name) is not None:
                    module.set_from_attribute_config(cfg)
                    break
        return
    if "default" in quant_cfg:
        set_quantizer_attribute(quant_model, "*", quant_cfg["default"], _index=index)
    for pattern, cfg in quant_cfg.items():
        if pattern == "default":
            continue
        if isinstance(pattern, str) and pattern.startswith("nn.") and isinstance(cfg, dict) and all(
                isinstance(v, (dict, list, QuantizerAttributeConfig)) for v in cfg.values()):
            cls = getattr(nn, pattern[3:], None)
            if cls is None:
                continue
            for sub_pattern, sub_cfg in cfg.items():
                set_quantizer_attribute(quant_model, sub_pattern, sub_cfg, parent_class=cls,
                                        _index=index)
            continue
        set_quantizer_attribute(quant_model, pattern, cfg, _index=index)


@functools.lru_cache(maxsize=512)
def _compiled(pattern: str):
    """``match(name)`` -> something that is not None when the wildcard matches.  The shapes almost
    every config uses (``*suffix``, ``*infix*``, ``prefix*``, a literal) become string methods;
    anything else is fnmatch's regular expression."""
    body = pattern.strip("*")
    if not any(c in body for c in "*?[]"):
        lead, trail = pattern.startswith("*"), pattern.endswith("*") and len(pattern) > 1
        stars = len(pattern) - len(body)
        if stars == int(lead) + int(trail):     # no doubled stars to think about
            if lead and trail:
                return lambda name: True if body in name else None
            if lead:
                return lambda name: True if name.endswith(body) else None
            if trail:
                return lambda name: True if name.startswith(body) else None
            return lambda name: True if name == body else None
    return re.compile(fnmatch.translate(pattern)).match


def _matches(name: str, wildcard_or_filter) -> bool:
    if isinstance(wildcard_or_filter, str):
        # fnmatch.fnmatch without its per-call normalisation (names are already in posix form)
        return _compiled(wildcard_or_filter)(name) is not None
    if callable(wildcard_or_filter):
        return bool(wildcard_or_filter(name))
    raise NotImplementedError(f"Unsupported type {type(wildcard_or_filter)}")


def _quantizer_index(quant_model: nn.Module):
    """[name, quantizer, parent module, attribute name] of every quantizer that is configured on
    its own (members of a ``SequentialQuantizer`` are configured through their container)."""
    index = []
    parents = dict(quant_model.named_modules())
    for name, module in parents.items():
        if not isinstance(module, (TensorQuantizer, SequentialQuantizer)):
            continue
        parent_name, _, leaf = name.rpartition(".")
        parent = parents[parent_name]
        if isinstance(parent, SequentialQuantizer):
            continue
        index.append([name, module, parent, leaf])
    return index


def set_quantizer_attribute(quant_model: nn.Module, wildcard_or_filter_func, attribute,
                            parent_class: type | None = None, _index=None):
    """Set attributes on every quantizer whose qualified name matches.  A list of attribute
    dicts turns the matched ``TensorQuantizer`` into a ``SequentialQuantizer``; a single dict on
    a ``SequentialQuantizer`` is applied to each of its members (reference: conversion.py
    :276-301)."""
    index = _quantizer_index(quant_model) if _index is None else _index
    many = isinstance(attribute, (list, tuple))
    cfg = [_as_cfg(a) for a in attribute] if many else _as_cfg(attribute)
    for entry in index:
        name, module, parent, leaf = entry
        if not _matches(name, wildcard_or_filter_func):
            continue
        if parent_class is not None and not isinstance(parent, parent_class):
            continue
        if many:
            if not isinstance(module, SequentialQuantizer):
                device = next((b.device for b in module.buffers()), None)
                module = SequentialQuantizer(*(TensorQuantizer() for _ in attribute))
                if device is not None:
                    module.to(device)
                setattr(parent, leaf, module)
                entry[1] = module
            elif len(attribute) != len(module):
                warnings.warn(f"The number of attributes ({len(attribute)}) does not match the number "
                              f"of quantizers of {module} leading to partial assignment.")
        # one dict on a SequentialQuantizer goes to every member
        module.set_from_attribute_config(cfg)


def _as_cfg(attribute):
    """Validate a user dict through ``QuantizerAttributeConfig`` but keep only the keys given,
    so a partial dict (``{"enable": False}``) leaves the other attributes alone."""
    if isinstance(attribute, QuantizerAttributeConfig):
        return attribute
    if set(attribute) == {"enable"}:
        # the "enable alone is not a config" rule is for user configs (checked when
        # ``mtq.quantize`` parses them); internally this is how a quantizer is switched on
        return {"enable": bool(attribute["enable"])}
    full = QuantizerAttributeConfig(**attribute)
    return {k: full[k] for k in attribute}


@contextmanager
def set_quantizer_by_cfg_context(quant_model: nn.Module, quant_cfg: dict[str, Any]):
    """Temporarily apply ``quant_cfg``; the previous python-side attributes come back on exit."""
    saved = {}
    for name, module in quant_model.named_modules():
        if isinstance(module, TensorQuantizer):
            saved[module] = module.get_modelopt_state(properties_only=True)
    set_quantizer_by_cfg(quant_model, quant_cfg)
    try:
        yield
    finally:
        for module, state in saved.items():
            module.set_from_modelopt_state(state, properties_only=True)


def register(original_cls: type, quantized_cls: type):
    """Register a user module class for conversion (reference: conversion.py:340-380)."""
    assert issubclass(original_cls, nn.Module) and issubclass(quantized_cls, nn.Module)
    QuantModuleRegistry.register({original_cls: original_cls.__name__})(quantized_cls)


def unregister(original_cls: type):
    QuantModuleRegistry.unregister(original_cls)
