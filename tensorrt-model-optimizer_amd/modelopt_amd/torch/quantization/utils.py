"""Quantization utilities with the reference's names (modelopt/torch/quantization/utils.py),
backed by the HIP abs-max kernels."""

import collections
import contextlib

import torch
import torch.nn.functional as F

from . import kernels

__all__ = [
    "true_divide", "convert_quantization_axis_to_reduce_axis", "reduce_amax", "reduce_block_amax",
    "reduce_block_padding", "is_quantized", "is_quantized_linear",
    "update_quant_cfg_with_kv_cache_quant", "quantizer_attr_names", "weight_attr_names",
    "enable_fake_quant", "enable_quant", "disable_calib", "reduce_sum",
    "all_positive", "all_valid_scales", "deferred_scale_checks",
]


def true_divide(t: torch.Tensor, divisor: float) -> torch.Tensor:
    """``t / divisor`` as one correctly rounded division.

    torch's GPU kernels evaluate ``tensor / python_scalar`` as ``tensor * (1 / scalar)`` (two
    roundings) while the CPU kernels divide; every scale the reference derives that way
    (``amax / 448``, ``amax / (6 * 448)``, ``amax / 7`` ...) is therefore computed here as a
    tensor / tensor division, which is a true division on both devices.
    """
    return torch.div(t, torch.full((), float(divisor), dtype=t.dtype, device=t.device))


def convert_quantization_axis_to_reduce_axis(input, axis):
    """Quantization axis -> dims to reduce (reference: utils.py:137-152)."""
    if axis is None:
        return None
    kept = list(axis) if isinstance(axis, (list, tuple)) else [axis]
    nd = input.dim()
    return [d for d in range(nd) if d not in kept and (d - nd) not in kept]


@torch.no_grad()
def reduce_amax(input, axis=None, keepdims=True, squeeze_scalar=True, *, reread=False):
    """Abs-max over ``axis`` (None = everything) in the input dtype (reference: utils.py:156-188).

    One kernel pass (the reference reads the tensor twice: max and min); NaN propagates.
    ``reread``: the caller reads ``input`` again right away (a dynamic quantizer's fake quant), so
    a per-tensor reduction leaves it in the memory-side cache.
    """
    if axis is None:
        return kernels.reduce_amax_gpu(input, None, reread=reread)
    out = kernels.reduce_amax_gpu(input, axis, keepdims=keepdims, reread=reread)
    if squeeze_scalar and out.numel() == 1:
        out = out.squeeze()
    return out


@torch.no_grad()
def reduce_block_padding(input, block_sizes: dict, pad_value: float = 0):
    """Right-pad the listed dims to multiples of their block (reference: utils.py:101-134)."""
    nd = input.dim()
    for dim, blk in block_sizes.items():
        d = dim if dim >= 0 else nd + dim
        rem = input.size(d) % blk
        if rem:
            spec = [0] * (2 * nd)
            spec[(nd - 1 - d) * 2 + 1] = blk - rem
            input = F.pad(input, spec, value=pad_value)
    return input


@torch.no_grad()
def reduce_block_amax(input_tensor, block_sizes: dict):
    """Blockwise abs-max, one listed dim at a time (reference: utils.py:52-98)."""
    out = input_tensor
    for dim, blk in block_sizes.items():
        d = dim if dim >= 0 else out.dim() + dim
        assert out.shape[d] % blk == 0, (
            f"Tensor dimension {out.shape[d]} is not divisible by {blk}")
        shape = list(out.shape)
        shape[d:d + 1] = [shape[d] // blk, blk]
        out = reduce_amax(out.reshape(shape), d + 1, keepdims=False, squeeze_scalar=False)
    return out


def is_quantized(module):
    from .nn import TensorQuantizer

    return any(isinstance(m, TensorQuantizer) for m in module.modules())


def is_quantized_linear(module):
    """A module with input/weight quantizers and a 2-D weight (reference: utils.py:222-232)."""
    from .nn import SequentialQuantizer, TensorQuantizer

    children = getattr(module, "__dict__", {}).get("_modules")
    if children is not None:
        # quantizers are child modules: looked up where nn.Module keeps them, since asking a
        # module for an attribute it does not have costs an exception
        input_quantizer, weight_quantizer = children.get("input_quantizer"), children.get("weight_quantizer")
        if input_quantizer is None or weight_quantizer is None:
            if "input_quantizer" not in module.__dict__ and "weight_quantizer" not in module.__dict__ \
                    and not hasattr(type(module), "input_quantizer"):
                return False
            input_quantizer = getattr(module, "input_quantizer", None)
            weight_quantizer = getattr(module, "weight_quantizer", None)
    else:
        input_quantizer = getattr(module, "input_quantizer", None)
        weight_quantizer = getattr(module, "weight_quantizer", None)
    if not (isinstance(input_quantizer, (TensorQuantizer, SequentialQuantizer))
            and isinstance(weight_quantizer, (TensorQuantizer, SequentialQuantizer))):
        return False
    weight = getattr(module, "weight", None)
    return weight is not None and weight.dim() == 2


# every quantizer-related attribute name that goes with one weight attribute (reference: utils.py:247-273)
QuantizerAttrNames = collections.namedtuple(
    "QuantizerAttrNames", ("weight_quantizer", "input_quantizer", "output_quantizer", "weight_scale",
                           "weight_scale_2", "input_scale", "output_scale"))


def quantizer_attr_names(weight_name="weight") -> QuantizerAttrNames:
    """The names for ``weight_name``: plain for ``"weight"``, prefixed ``<weight_name>_`` otherwise."""
    prefix = "" if weight_name == "weight" else weight_name + "_"
    return QuantizerAttrNames(*(prefix + field for field in QuantizerAttrNames._fields))


def is_pow2(n) -> bool:
    """True for 1, 2, 4, ... (reference: utils.py:377-379)."""
    return n != 0 and n & (n - 1) == 0


@contextlib.contextmanager
def replace_function(package, name, new_func):
    """Within the block ``package.name`` is ``new_func`` and the original is reachable as
    ``package._name`` (reference: utils.py:339-347)."""
    original = getattr(package, name)
    setattr(package, name, new_func)
    setattr(package, "_" + name, original)
    try:
        yield
    finally:
        setattr(package, name, original)
        delattr(package, "_" + name)


@contextlib.contextmanager
def multi_context(*managers):
    """Enter any number of context managers as one (reference: utils.py:350-354)."""
    with contextlib.ExitStack() as stack:
        yield [stack.enter_context(m) for m in managers]


EXPORT_MODE: bool = False


@contextlib.contextmanager
def export_torch_mode():
    """Marks the block as a ``torch.export`` trace (reference: utils.py:357-374)."""
    global EXPORT_MODE
    before, EXPORT_MODE = EXPORT_MODE, True
    try:
        yield
    finally:
        EXPORT_MODE = before


def is_torch_export_mode() -> bool:
    return EXPORT_MODE


@contextlib.contextmanager
def enable_weight_access_and_writeback(module, root_model):
    """The reference gathers a sharded or off-loaded weight here and writes it back afterwards
    (utils.py:466-486); weights of this build's modules are whole and resident, so the block runs
    as it is."""
    yield


def get_quantizer_state_dict(model):
    """``{quantizer name: its state_dict()}`` without calling ``model.state_dict()``
    (reference: utils.py:489-500)."""
    from .nn import TensorQuantizer

    return {name: module.state_dict() for name, module in model.named_modules()
            if isinstance(module, TensorQuantizer)}


def set_quantizer_state_dict(model, quantizer_state_dict: dict):
    """Load what ``get_quantizer_state_dict`` returned (reference: utils.py:503-511)."""
    from .nn import TensorQuantizer

    for name, module in model.named_modules():
        if isinstance(module, TensorQuantizer) and name in quantizer_state_dict:
            module.load_state_dict(quantizer_state_dict[name])


def weight_attr_names(module):
    if hasattr(module, "weight_quantizer") and getattr(module, "weight", None) is not None:
        yield "weight"


def update_quant_cfg_with_kv_cache_quant(quant_cfg: dict, kv_cache_quant_cfg: dict) -> dict:
    """Merge KV-cache quantizer entries into a config (reference: utils.py:769-781)."""
    import copy

    quant_cfg = copy.deepcopy(quant_cfg)
    inner = quant_cfg.get("quant_cfg", {"default": {"enable": False}})
    inner.update(kv_cache_quant_cfg)
    quant_cfg["quant_cfg"] = inner
    if not quant_cfg.get("algorithm"):
        quant_cfg["algorithm"] = "max"
    return quant_cfg


_DEFERRED_CHECKS = []   # innermost ``deferred_scale_checks`` block last


class DeferredCheckError(AssertionError):
    """A check recorded inside a ``deferred_scale_checks`` block failed when the block ended."""


class _DeferredChecks(list):
    """The tensors a ``deferred_scale_checks`` block has recorded: the list itself holds those
    that must be finite and non-negative, ``positive`` those that must be positive, ``report``
    those whose validity is only reported (``report_ok`` after the block)."""

    def __init__(self):
        super().__init__()
        self.positive = []
        self.positive_messages = []   # one per entry of ``positive``: text, callable or None
        self.report = []
        self.report_ok = True


def _validity_flags(tensors, strictly_positive=False):
    """What decides "every element is finite and non-negative (or positive)", one entry per
    (device, dtype) group of ``tensors``: the group's ``(min, max)`` as a 2-element device tensor
    from one ``aminmax`` over the concatenation (a NaN anywhere makes both NaN).  No host
    synchronisation."""
    groups = {}   # one concatenation per (device, dtype): no per-tensor conversion
    for t in tensors:
        if isinstance(t, torch.Tensor) and not t.is_meta and t.numel():
            t = t.detach()
            if not t.is_floating_point():
                t = t.to(torch.float32)
            groups.setdefault((t.device, t.dtype), []).append(t.reshape(-1))
    flags = []
    for group in groups.values():
        v = torch.cat(group) if len(group) > 1 else group[0]
        flags.append((torch.stack(torch.aminmax(v)).float(), strictly_positive))
    return flags


def _read_flags(flag_lists):
    """``[all(flags) for flags in flag_lists]`` with one host synchronisation per device."""
    by_device = {}
    for i, flags in enumerate(flag_lists):
        for pair, positive in flags:
            by_device.setdefault(pair.device, []).append((i, pair, positive))
    result = [True] * len(flag_lists)
    for entries in by_device.values():
        pairs = entries[0][1] if len(entries) == 1 else torch.cat([p for _, p, _ in entries])
        values = pairs.tolist()
        for n, (i, _, positive) in enumerate(entries):
            lo, hi = values[2 * n], values[2 * n + 1]
            # a NaN anywhere makes lo and hi NaN, and every comparison with it false
            ok = lo > 0 if positive else (lo >= 0 and hi < float("inf"))
            result[i] = result[i] and ok
    return result


def _checked(kinds):
    """``[ok, ...]`` for ``kinds`` = [(tensors, strictly_positive), ...]: whether every element of
    every tensor of a kind is finite and non-negative (or positive).  One launch and one host
    synchronisation for all kinds when the tensors are few and small (the calibrated values of a
    handful of layers); one reduction per kind and dtype otherwise."""
    from modelopt_amd import _hip

    lists = [[t.detach() for t in tensors if isinstance(t, torch.Tensor) and not t.is_meta and t.numel()]
             for tensors, _ in kinds]
    flat = [t for ts in lists for t in ts]
    ranges = _hip.value_ranges(flat) if flat else []
    if ranges is None:
        return _read_flags([_validity_flags(ts, positive) for ts, (_, positive) in zip(lists, kinds)])
    result, at = [], 0
    for ts, (_, positive) in zip(lists, kinds):
        ok = True
        for lo, hi, has_nan in ranges[at:at + len(ts)]:
            ok = ok and not has_nan and (lo > 0 if positive else (lo >= 0 and hi < float("inf")))
        at += len(ts)
        result.append(ok)
    return result


@contextlib.contextmanager
def deferred_scale_checks():
    """Within the block ``all_valid_scales`` and ``all_positive`` only record their tensors and
    report True; the real checks -- one device reduction per kind and ONE host synchronisation for
    all of them -- happen when the outermost block ends, which raises ``AssertionError`` if a
    recorded value is negative, infinite or NaN (not positive, for ``all_positive``) by then.  A
    nested block hands its tensors to the enclosing one.  Tensors appended to ``report`` of the
    yielded object are checked in the same synchronisation but only reported (``report_ok``).
    For loops over many layers whose per-layer checks would each wait for the device."""
    pending = _DeferredChecks()
    _DEFERRED_CHECKS.append(pending)
    try:
        yield pending
    finally:
        _DEFERRED_CHECKS.pop()
    if _DEFERRED_CHECKS:    # nested: the enclosing block checks
        outer = _DEFERRED_CHECKS[-1]
        outer.extend(pending)
        outer.positive.extend(pending.positive)
        outer.positive_messages.extend(pending.positive_messages)
        if pending.report:   # the block's owner wants an answer now
            pending.report_ok = _checked([(pending.report, False)])[0]
        return
    if not (pending or pending.positive or pending.report):
        return
    valid, positive, pending.report_ok = _checked([
        (pending, False), (pending.positive, True), (pending.report, False)])
    if not valid:
        raise DeferredCheckError("detected negative, inf or nan values in a calibrated amax or scale")
    if not positive:
        # only now, on the way to an error, look for the tensor that failed and its own words
        message = "pre_quant_scale should be positive"
        for tensor, own in zip(pending.positive, pending.positive_messages):
            if own is not None and not bool(torch.all(tensor > 0)):
                message = own() if callable(own) else own
                break
        raise DeferredCheckError(message)


def all_valid_scales(tensors) -> bool:
    """True when every element of every tensor is finite and non-negative -- one device
    reduction and one host synchronisation for the whole list."""
    if _DEFERRED_CHECKS:
        _DEFERRED_CHECKS[-1].extend(t for t in tensors if isinstance(t, torch.Tensor))
        return True
    return _checked([(list(tensors), False)])[0]


def all_positive(tensor, message=None) -> bool:
    """True when every element is positive; inside a ``deferred_scale_checks`` block the tensor is
    recorded and the answer comes when the block ends (``AssertionError`` with ``message`` -- a
    text, or a callable that builds it -- if this is the tensor that failed)."""
    if _DEFERRED_CHECKS:
        _DEFERRED_CHECKS[-1].positive.append(tensor)
        _DEFERRED_CHECKS[-1].positive_messages.append(message)
        return True
    return bool(torch.all(tensor > 0))


@contextlib.contextmanager
def enable_fake_quant(module):
    """Within the block every ``weight_quantizer`` under ``module`` fake-quantises, whatever its
    ``fake_quant`` setting (reference: utils.py:616-630).  A bare quantizer has no
    ``weight_quantizer`` child and is left as it is, as in the reference."""
    held = [m.weight_quantizer for m in module.modules() if hasattr(m, "weight_quantizer")]
    before = [q._fake_quant for q in held]
    for q in held:
        q._fake_quant = True
    try:
        yield
    finally:
        for q, was in zip(held, before):
            q._fake_quant = was


@contextlib.contextmanager
def enable_quant(quantizer):
    """Quantisation switched on for the block (reference: utils.py:633-646)."""
    was, quantizer._if_quant = quantizer._if_quant, True
    try:
        yield
    finally:
        quantizer._if_quant = was


@contextlib.contextmanager
def disable_calib(quantizer):
    """Statistics collection switched off for the block (reference: utils.py:649-662)."""
    was, quantizer._if_calib = quantizer._if_calib, False
    try:
        yield
    finally:
        quantizer._if_calib = was


def reduce_sum(input, axis=None, keepdims=True):
    """Sum over ``axis`` (None = everything) (reference: utils.py:192-218)."""
    if axis is None:
        return torch.sum(input)
    return torch.sum(input, dim=(axis,) if isinstance(axis, int) else tuple(axis), keepdim=keepdims)
