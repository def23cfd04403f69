"""Calibration algorithms: max, SmoothQuant and AWQ-lite.

Reference: modelopt/torch/quantization/model_calib.py:66-185 (``max_calibrate``), :272-306
(stats collection), :346-408 (pre-quant-scale folding), :412-496 (``smoothquant``), :530-786
(``awq_lite``).  Single GPU: every distributed synchronisation of the reference is a no-op here.
The per-element work (abs-max, scaling, quantize-dequantize, column statistics, squared error)
runs in the HIP kernels; the search GEMM is a plain library GEMM (``F.linear``).
"""

import functools
import math
import types
import warnings

import torch
import torch.nn.functional as F
from torch import nn

from ... import _hip
from . import calib
from .calib.max import MaxCalibrator
from .conversion import set_quantizer_by_cfg_context
from .nn import QuantModule, SequentialQuantizer, TensorQuantizer
from .nn.modules.quant_linear import _QuantLinear
from .nn.modules.tensor_quantizer import calibration_pass
from .utils import all_positive, all_valid_scales, deferred_scale_checks, is_quantized_linear

__all__ = ["max_calibrate", "smoothquant", "awq", "awq_lite", "enable_stats_collection",
           "finish_stats_collection", "apply_pre_quant_scale_and_smooth",
           "disable_pre_quant_scale_and_resmooth", "awq_clip", "mse_calibrate"]


# ----------------------------------------------------------------------------- max
def weight_only_quantize(model: nn.Module):
    """Show every weight to its quantizer once (no activations involved)."""
    seen = set()
    for module in model.modules():
        if module in seen:
            continue
        if isinstance(module, QuantModule) and hasattr(module, "weight_quantizer") and getattr(
                module, "weight", None) is not None:
            module.weight_quantizer(module.weight)
        seen.add(module)


def enable_stats_collection(model: nn.Module):
    """Switch every enabled quantizer to calibration (quantisation off, statistics on)."""
    for module in model.modules():
        if isinstance(module, TensorQuantizer) and not module._disabled:
            if module._calibrator is not None:
                module.disable_quant()
                module.enable_calib()
            else:
                module.disable()


def finish_stats_collection(model: nn.Module, method: str | None = None):
    """Load the collected amax into ``_amax`` and switch quantisation back on."""
    # the calibrators' deferred sanity checks, for all of them at once: one host synchronisation
    # instead of one per quantizer (a calibrator that fails is left to raise its own message)
    pending = [m._calibrator for m in model.modules()
               if isinstance(m, TensorQuantizer) and not m._disabled
               and getattr(m._calibrator, "_acc", None) is not None
               and not m._calibrator._validated]
    for c in pending:
        if hasattr(c, "_fold_pending"):
            c._fold_pending()   # tile maxima of reductions shared with another calibrator
    if pending and all_valid_scales([c._acc for c in pending]):
        for c in pending:
            c._validated = True
    for module in model.modules():
        if not isinstance(module, TensorQuantizer) or module._disabled:
            continue
        cal = getattr(module, "_calibrator", None)
        if cal and not getattr(module, "_dynamic", False):
            if type(cal) is MaxCalibrator:
                found = cal.has_amax()   # load_calib_amax computes it; not twice
            else:
                found = (cal.compute_amax() if method != "mse" or isinstance(cal, MaxCalibrator)
                         else cal.compute_amax(False)) is not None
            if found:
                module.load_calib_amax()
        module.enable_quant()
        module.disable_calib()


@torch.no_grad()
def max_calibrate(model: nn.Module, forward_loop=None, distributed_sync=True):
    """Max calibration: run ``forward_loop(model)`` with statistics collection on."""
    enable_stats_collection(model)
    if forward_loop is None:
        weight_only_quantize(model)
    else:
        with calibration_pass():
            forward_loop(model)
    finish_stats_collection(model)


@torch.no_grad()
def mse_calibrate(model: nn.Module, forward_loop=None, distributed_sync=True, num_steps: int = 10,
                  start_multiplier: float = 0.25, stop_multiplier: float = 4.0):
    """Max calibration first, then an amax search per quantizer that minimises the squared error
    between the tensors it sees and their fake-quantised versions (reference:
    model_calib.py:189-262)."""
    max_calibrate(model, forward_loop, distributed_sync)
    for name, module in model.named_modules():
        if not isinstance(module, TensorQuantizer) or module._disabled:
            continue
        if module.is_static_block_quant:
            raise ValueError("MSE calibration does not support static block quantization. "
                             f"Found static block quantization at {name}.")
        if module._calibrator is None or module._dynamic or not hasattr(module, "_amax"):
            continue
        initial_amax = module._amax.clone().detach()

        def quant_func(x, amax, quantizer=module):
            saved = quantizer._amax.clone() if hasattr(quantizer, "_amax") else None
            quantizer._amax = amax
            state = (quantizer._if_quant, quantizer._if_calib, quantizer._fake_quant)
            quantizer._if_quant, quantizer._if_calib, quantizer._fake_quant = True, False, True
            try:
                xq = quantizer(x)
            finally:
                quantizer._if_quant, quantizer._if_calib, quantizer._fake_quant = state
                if saved is not None:
                    quantizer._amax = saved
                else:
                    delattr(quantizer, "_amax")
            return xq

        module._calibrator = calib.MseCalibrator(
            amax=initial_amax, axis=module._calibrator._axis, num_steps=num_steps,
            start_multiplier=start_multiplier, stop_multiplier=stop_multiplier,
            quant_func=quant_func, quantizer=module)
    enable_stats_collection(model)
    if forward_loop is None:
        weight_only_quantize(model)
    else:
        forward_loop(model)
    finish_stats_collection(model, method="mse")


# ----------------------------------------------------------------------------- pre-quant scale
_ENABLE_FOLDING_PQS_TO_WEIGHTS = True


@torch.no_grad()
def _apply_weight_pre_quant_scale(linear, pre_quant_scale):
    """``W <- dtype(W * s[None, :])`` with an fp32 ``s`` (one product, one rounding), then
    recalibrate the weight amax."""
    if _ENABLE_FOLDING_PQS_TO_WEIGHTS:
        s = pre_quant_scale
        if not (s.dtype == torch.float32 and s.dim() == 1 and s.device == linear.weight.device
                and s.is_contiguous()):
            s = s.to(linear.weight.device).squeeze().to(torch.float32).contiguous()
        _hip.mul_cols(linear.weight.data, s, out=linear.weight.data)
    else:
        linear.weight_quantizer._enable_pre_quant_scale = True
        linear.weight_quantizer.pre_quant_scale = pre_quant_scale.squeeze()[None, :].to(
            linear.weight.dtype)
    linear.weight_quantizer.reset_amax()
    max_calibrate(linear, lambda lin: lin.weight_quantizer(lin.weight))


def _host_copy_later(t: torch.Tensor) -> torch.Tensor:
    """``t.cpu()`` without waiting for the device: a copy into pinned host memory queued on the
    current stream.  The host may read it once that stream has been synchronised -- the
    calibration algorithms end with a host synchronisation, so what they leave on the modules is
    complete when they return.  The device tensor rides along (``_device_twin``) for consumers
    that want the values back on the device."""
    if not t.is_cuda:
        return t
    host = torch.empty(t.shape, dtype=t.dtype, pin_memory=True)
    host.copy_(t, non_blocking=True)
    host._device_twin = t
    return host


def _on_device(t: torch.Tensor, device) -> torch.Tensor:
    """``t.to(device)``; a host copy made by ``_host_copy_later`` hands back the device tensor it
    was copied from."""
    twin = getattr(t, "_device_twin", None)
    if twin is not None and twin.device == torch.device(device):
        return twin
    return t.to(device)


@torch.no_grad()
def apply_pre_quant_scale_and_smooth(linear: nn.Module, pre_quant_scale: torch.Tensor | None = None, *,
                                     _rounded: torch.Tensor | None = None, _fold: torch.Tensor | None = None,
                                     _smoothed_amax: torch.Tensor | None = None):
    """Set the input ``pre_quant_scale`` and fold its inverse into the weight.  Inside a
    ``deferred_scale_checks`` block (a caller that loops over many layers) the positivity of the
    scale is checked when the block ends instead of here (a host synchronisation per layer).
    ``_rounded`` and ``_fold``: ``pre_quant_scale`` in the weight's dtype and ``1 / pre_quant_scale``
    in fp32, ``_smoothed_amax``: the input amax after smoothing, for a caller that has them
    already (bit for bit what is computed here otherwise)."""
    assert is_quantized_linear(linear), "Only quantized linear modules are supported"
    assert linear.input_quantizer.pre_quant_scale is None, "pre_quant_scale should be None first!"
    if pre_quant_scale is None:
        pre_quant_scale = getattr(linear.input_quantizer, "_pre_quant_scale", None)
    assert pre_quant_scale is not None, "pre_quant_scale should be provided or already set"
    assert all_positive(pre_quant_scale), "pre_quant_scale should be positive"
    pre_quant_scale = pre_quant_scale.to(torch.float32)  # fp32 keeps the scaling maths safe

    linear.input_quantizer._enable_pre_quant_scale = True
    linear.input_quantizer.pre_quant_scale = (_rounded if _rounded is not None
                                              else pre_quant_scale.to(linear.weight.dtype))
    _apply_weight_pre_quant_scale(linear, _fold if _fold is not None else 1.0 / pre_quant_scale)

    if linear.input_quantizer.amax is not None and _smoothed_amax is not None:
        assert hasattr(linear.input_quantizer, "_amax_for_smoothing")
        linear.input_quantizer.amax = _smoothed_amax
    elif linear.input_quantizer.amax is not None:
        assert hasattr(linear.input_quantizer, "_amax_for_smoothing")
        device, dtype = linear.weight.device, linear.weight.dtype
        smoothing = _on_device(linear.input_quantizer._amax_for_smoothing, device).to(dtype)
        # rounded to the weight's dtype, then widened again by hand (see smoothquant: no
        # mixed-dtype product)
        linear.input_quantizer.amax = (smoothing.float() * pre_quant_scale.to(device)).amax().to(dtype)


@torch.no_grad()
def disable_pre_quant_scale_and_resmooth(linear: nn.Module, delete_pre_quant_scale: bool = False):
    """Undo the smoothing of one linear: multiply the weight by the input ``pre_quant_scale``
    again, recalibrate the weight amax, switch the scale off (kept unless asked otherwise) and
    restore the un-smoothed input amax (reference: model_calib.py:309-339)."""
    assert is_quantized_linear(linear), "Only quantized linear modules are supported"
    assert linear.input_quantizer._enable_pre_quant_scale, "pre_quant_scale should be enabled first!"
    assert hasattr(linear.input_quantizer, "_pre_quant_scale"), "pre_quant_scale should be available"
    _apply_weight_pre_quant_scale(linear, linear.input_quantizer._pre_quant_scale.to(torch.float32))
    linear.input_quantizer._enable_pre_quant_scale = False
    if linear.input_quantizer.amax is not None:
        assert hasattr(linear.input_quantizer, "_amax_for_smoothing")
        device, dtype = linear.weight.device, linear.weight.dtype
        linear.input_quantizer.amax = linear.input_quantizer._amax_for_smoothing.amax().to(
            device=device, dtype=dtype)
    if delete_pre_quant_scale:
        delattr(linear.input_quantizer, "_pre_quant_scale")
        linear.input_quantizer._enable_pre_quant_scale = False


def _pow(t: torch.Tensor, exponent: float) -> torch.Tensor:
    """``t.pow(exponent)`` with the CPU result for the exponents the CPU evaluates exactly.

    torch's CPU kernel turns ``pow(x, 0.5)`` into a correctly rounded fp32 square root; the GPU
    kernel's square root is off by an ulp for about one input in six.  A double-precision root
    rounded to fp32 is the correctly rounded fp32 root, so that is what is used here; other
    exponents go through the device ``pow`` (within an ulp or two of the CPU's).
    """
    if exponent == 0.5:
        return t.double().sqrt().float().to(t.dtype)
    return t.pow(exponent)


# ----------------------------------------------------------------------------- SmoothQuant
@torch.no_grad()
def smoothquant(model: nn.Module, forward_loop=None, alpha=1.0):
    """SmoothQuant with per-channel weight scaling for INT8 linears."""
    assert forward_loop is not None, "forward_loop must be provided for smoothquant"
    for module in model.modules():
        if (is_quantized_linear(module) and module.input_quantizer.is_enabled
                and module.input_quantizer.axis is None):
            module.input_quantizer.axis = -1
    max_calibrate(model, forward_loop)

    def postprocess(module):
        act_amax = module.input_quantizer.amax.float()
        w = module.weight
        device, dtype = w.device, w.dtype
        col = torch.zeros(w.shape[1], dtype=torch.float32, device=device)
        _hip.absmax_into(w.data.contiguous(), col, w.shape[0], w.shape[1], 1)
        if (_SMOOTH_IN_ONE_LAUNCH and w.is_cuda and dtype in _hip._DTYPES and act_amax.device == device
                and act_amax.numel() == col.numel()):
            # the scale, its rounded copy, its inverse and both input amax values from one launch
            # (some twenty tensor operations otherwise, each a launch behind the layer's GEMM)
            pqs, pqs_t, fold, act_max, smoothed = _hip.smooth_scales(
                act_amax.contiguous().view(-1), col, float(alpha), dtype)
            module.input_quantizer._amax_for_smoothing = _host_copy_later(act_amax)
            module.input_quantizer.reset_amax()
            module.input_quantizer.axis = None
            module.input_quantizer.amax = act_max
            apply_pre_quant_scale_and_smooth(module, pqs, _rounded=pqs_t, _fold=fold, _smoothed_amax=smoothed)
            return
        weight_scale = col.to(dtype).reshape(1, -1)  # == w.abs().amax(dim=0, keepdim=True)
        # the 16-bit numerator is widened by hand: the same values as type promotion gives, but a
        # binary operation on two dtypes goes through the tensor library's casting kernel,
        # which takes 70 us for these 8192 values where a conversion and a division take 10
        scale_a = (_pow(weight_scale, 1 - alpha).float() / _pow(act_amax, alpha)).squeeze()
        module.input_quantizer._amax_for_smoothing = _host_copy_later(act_amax)
        module.input_quantizer.reset_amax()
        module.input_quantizer.axis = None
        module.input_quantizer.amax = act_amax.amax().to(dtype=dtype, device=device)
        eps = 1.0 / (1 << 31)
        # channels that never fired would make scale_a overflow: when the smallest scale is tiny
        # they are set to 1 -- selected on the device, the host does not wait for the answer
        dead = (scale_a.min() <= eps) & (act_amax.reshape(-1) <= eps)
        scale_a = torch.where(dead, torch.ones_like(scale_a), scale_a)
        scale_a = scale_a.clamp(min=1e-4, max=1e4)
        apply_pre_quant_scale_and_smooth(module, scale_a)

    smoothed = 0
    with deferred_scale_checks():   # one synchronisation for the checks of all layers
        for name, module in model.named_modules():
            if not is_quantized_linear(module):
                continue
            if not hasattr(module.input_quantizer, "_amax"):
                warnings.warn(f"{name} is not calibrated, skip smoothing")
                continue
            if module.input_quantizer.num_bits != 8 or module.weight_quantizer.num_bits != 8:
                warnings.warn(f"Only int8 smoothing is supported, skip {name}")
                continue
            if module.input_quantizer.axis != -1:
                warnings.warn(f"Only per-channel smoothing is supported, skip {name}")
                continue
            assert module.input_quantizer._amax.numel() > 1, f"Error: {name} has only one channel to smooth"
            postprocess(module)
            smoothed += 1
    print(f"Smoothed {smoothed} modules")


# ----------------------------------------------------------------------------- AWQ-clip
@functools.lru_cache(maxsize=16)
def _clip_ratios(min_clip_ratio: float, shrink_step: float) -> tuple:
    """The clip ratios of the search, smallest first, 1.0 last (reference: model_calib.py:818-821)."""
    return tuple(round(float(k), 2) for k in torch.arange(min_clip_ratio, 1.0, shrink_step)) + (1.0,)


@functools.lru_cache(maxsize=16)
def _ratio_column(ratios: tuple, device) -> torch.Tensor:
    """The ratios as an fp32 device vector (built once per ratio list and device)."""
    return torch.tensor(ratios, dtype=torch.float32).to(device)


def _best_clip(helper):
    """``(best_loss, best_clip_val)`` as the reference's loop over the ratios leaves them
    (model_calib.py:958-966: a ratio replaces the running best when its loss is strictly smaller,
    so the first smallest loss wins, a NaN never does, and a block for which no loss is below
    infinity keeps a clip value of zero) -- from the stacked losses in a handful of launches
    instead of three per ratio."""
    ratios = tuple(helper.loss)
    w_amax = helper.w_amax
    loss = helper.loss_all.view(len(ratios), *w_amax.shape)
    inf = torch.full((), float("inf"), dtype=loss.dtype, device=loss.device)
    best_loss, index = torch.where(torch.isnan(loss), inf, loss).min(dim=0)
    # amax * python float: one product in fp32, one rounding to the amax dtype
    clip = (w_amax.float() * _ratio_column(ratios, w_amax.device)[index]).to(w_amax.dtype)
    return best_loss, torch.where(best_loss < inf, clip, torch.zeros_like(clip))


class _AWQClipHelper:
    """Per-linear state of the clip search (reference: model_calib.py:810-850)."""

    def __init__(self, module, min_clip_ratio, shrink_step):
        self.num_tokens = 0
        self.block_size = _awq_block_size(module.weight, module.weight_quantizer)
        q = module.weight_quantizer
        q.reset_amax()
        max_calibrate(q, lambda quantizer: quantizer(module.weight))
        self.w_amax = q.amax.clone()
        co, ci = module.weight.shape
        ratios = list(_clip_ratios(float(min_clip_ratio), float(shrink_step)))
        dev = module.weight.device
        if self.is_per_tensor_clip(module):
            self.loss = {k: torch.tensor(0.0, device=dev) for k in ratios}
        else:
            # one tensor behind the per-ratio entries, so that the fused kernel can add to all
            # of them in one launch
            self.loss_all = torch.zeros((len(ratios), co, math.ceil(ci / self.block_size)), device=dev)
            self.loss = {k: self.loss_all[i] for i, k in enumerate(ratios)}
        self.best_clip_val = None
        self.best_loss = None
        self.is_input_quantized = module.input_quantizer.is_enabled
        q.disable()

    @staticmethod
    def is_per_tensor_clip(module):
        q = module.weight_quantizer
        dynamic_per_tensor = (q.block_sizes is not None and q.block_sizes.get("type") == "dynamic"
                              and q.axis is None)
        return dynamic_per_tensor or (q.axis is None and q.block_sizes is None)


def _fused_clip_search(helper, q, inputs, weight, bs):
    """Every ratio and every block in one kernel launch, when the weight quantizer is a plain
    integer fake quantizer with static blocks along the last axis that divide it (what
    ``INT4_AWQ_CFG`` / ``W4A8_AWQ_BETA_CFG`` set up).  False: not covered, nothing done."""
    blocks = q.block_sizes or {}
    plain = (isinstance(q, TensorQuantizer) and isinstance(q.num_bits, int) and q._fake_quant
             and not q._dynamic and blocks.get("type", "static") == "static"
             and blocks.get("scale_bits") is None and q.pre_quant_scale is None
             and not getattr(q, "_rotate", False) and getattr(q, "_bias", None) is None
             and {k for k in blocks if isinstance(k, int)} <= {-1, weight.dim() - 1}
             and weight.dim() == 2 and weight.shape[1] % bs == 0
             and inputs.dtype == weight.dtype and helper.w_amax.numel() == weight.numel() // bs)
    if not plain:
        return False
    return _hip.awq_clip_losses_into(inputs.contiguous(), weight.data.contiguous(),
                                     helper.w_amax.contiguous(), list(helper.loss), bs, q.num_bits,
                                     q._unsigned, q._narrow_range, helper.loss_all)


def _awq_clip_search(self, inputs, co_bsz, max_tokens):
    """Accumulate, for every clip ratio, the error the clipped and fake-quantised weight makes on
    the layer's partial (per input block) outputs (reference: model_calib.py:864-929).  The weight
    is quantised once per ratio by the block fake-quant kernel; the partial sums are torch ops."""
    helper, q = self.awq_clip, self.weight_quantizer
    weight = self.weight
    q.enable()
    if helper.is_per_tensor_clip(self):
        out_actual = inputs @ weight.T
        original = q.amax.clone()
        helper.num_tokens += inputs.shape[0]
        for shrink in helper.loss:
            q.amax = original * shrink
            out = inputs @ q(weight).T
            helper.loss[shrink] += (out - out_actual).float().pow(2).mean()
        return
    inputs = inputs.reshape(-1, inputs.shape[-1])
    inputs = inputs[0::max(1, inputs.shape[0] // max_tokens)]
    helper.num_tokens += inputs.shape[0]
    bs = helper.block_size
    co, ci = weight.shape
    if _fused_clip_search(helper, q, inputs, weight, bs):
        return
    pad = (bs - ci % bs) % bs
    if pad:
        weight = F.pad(weight, (0, pad), "constant", 0)
        inputs = F.pad(inputs, (0, pad), "constant", 0)
    w4 = weight.reshape(co, 1, -1, bs)
    x4 = inputs.reshape(1, inputs.shape[0], -1, bs)
    quantized = {}
    for shrink in helper.loss:           # one fake-quant pass over the weight per ratio
        q.amax = helper.w_amax * shrink
        wq = q(self.weight)
        quantized[shrink] = F.pad(wq, (0, pad), "constant", 0) if pad else wq
    for lo in range(0, co, co_bsz):
        hi = min(lo + co_bsz, co)
        org_out = (x4 * w4[lo:hi]).sum(dim=-1)
        for shrink, wq in quantized.items():
            cur_out = (x4 * wq[lo:hi].reshape(w4[lo:hi].shape)).sum(dim=-1)
            helper.loss[shrink][lo:hi] += (cur_out - org_out).float().pow(2).mean(dim=1)


def _awq_clip_forward(self, input, *args, **kwargs):
    helper = self.awq_clip
    if helper.is_input_quantized:
        self.input_quantizer.enable()
        max_calibrate(self.input_quantizer, lambda quantizer: quantizer(input))
        self.input_quantizer.disable()
    _awq_clip_search(self, self.input_quantizer(input), helper.max_co_batch_size,
                     helper.max_tokens_per_batch)
    self.weight_quantizer.disable()
    return self._forward_no_awq(input, *args, **kwargs)


@torch.no_grad()
def awq_clip(model: nn.Module, forward_loop, max_co_batch_size: int = 1024,
             max_tokens_per_batch: int = 64, min_clip_ratio: float = 0.5, shrink_step: float = 0.05,
             debug: bool = False, **kwargs):
    """AWQ clip: per weight block, the clipped amax (``ratio * block amax``) that minimises the
    error of the block's contribution to the layer output on the calibration tokens (reference:
    model_calib.py:789-997)."""
    assert forward_loop is not None, "forward_loop must be provided for awq_clip"
    patched = []
    for name, module in model.named_modules():
        if (is_quantized_linear(module) and module.weight_quantizer.is_enabled
                and module.weight_quantizer.block_sizes is not None):
            module._forward_no_awq = module.forward
            module.forward = types.MethodType(_awq_clip_forward, module)
            module.awq_clip = _AWQClipHelper(module, min_clip_ratio, shrink_step)
            module.awq_clip.max_co_batch_size = max_co_batch_size
            module.awq_clip.max_tokens_per_batch = max_tokens_per_batch
            patched.append(module)
    print("awq_clip: Estimating parameters...")
    enable_stats_collection(model)
    with calibration_pass():
        forward_loop(model)
    max_calibrate(model, lambda m: None)
    for module in patched:
        helper = module.awq_clip
        if helper.num_tokens > 0 and hasattr(helper, "loss_all"):
            helper.best_loss, helper.best_clip_val = _best_clip(helper)
        elif helper.num_tokens > 0:
            helper.best_loss = torch.ones_like(helper.w_amax) * float("inf")
            helper.best_clip_val = torch.zeros_like(helper.w_amax)
            for shrink, loss in helper.loss.items():
                loss = loss.view_as(helper.w_amax)
                better = loss < helper.best_loss
                helper.best_loss = torch.where(better, loss, helper.best_loss)
                helper.best_clip_val = torch.where(better, helper.w_amax * shrink, helper.best_clip_val)
        if helper.num_tokens > 0:
            module.weight_quantizer.amax = helper.best_clip_val
            module.weight_quantizer.enable()
            if helper.is_input_quantized:
                module.input_quantizer.enable()
        if not debug:
            delattr(module, "awq_clip")
        if "forward" in module.__dict__:
            del module.__dict__["forward"]
        if "_forward_no_awq" in module.__dict__:
            del module.__dict__["_forward_no_awq"]


# ----------------------------------------------------------------------------- AWQ-lite
def awq(model: nn.Module, forward_loop=None, algorithm: str = "awq_lite", **kwargs):
    with SequentialQuantizer.convert_to_single_quantizer(model):
        if algorithm in ("awq_full", "awq_lite"):
            awq_lite(model, forward_loop, **kwargs)
        if algorithm in ("awq_full", "awq_clip"):
            clip_args = {k: v for k, v in kwargs.items() if k in (
                "max_co_batch_size", "max_tokens_per_batch", "min_clip_ratio", "shrink_step", "debug")}
            awq_clip(model, forward_loop, **clip_args)
    for module in model.modules():
        if is_quantized_linear(module) and isinstance(module.weight_quantizer, SequentialQuantizer):
            max_calibrate(module, lambda lin: lin.weight_quantizer(lin.weight))


def _awq_block_size(weight, quantizer):
    if quantizer.block_sizes is None:
        return None
    return quantizer.block_sizes.get(-1) or quantizer.block_sizes.get(weight.dim() - 1)


def get_weight_scale(weight, block_size=None):
    """fp32 [K]: column mean of ``|w| / (block amax + tiny)``, every step rounded in the weight
    dtype like the reference's tensor expression."""
    n, k = weight.shape
    w = weight.data.contiguous()
    dev = w.device
    if block_size and k % block_size == 0:
        # block abs-max, quotient and column sum in one pass over the weight
        acc = torch.zeros(k, dtype=torch.float32, device=dev)
        if _hip.weight_scale_colsum_into(w, acc, block_size):
            return (acc / n).to(weight.dtype).to(torch.float32)
    if block_size:
        nb = -(-k // block_size)
        if k % block_size:
            w_blk = F.pad(w, (0, nb * block_size - k))
        else:
            w_blk = w
        blk_amax = torch.zeros(n * nb, dtype=torch.float32, device=dev)
        _hip.absmax_into(w_blk, blk_amax, 1, n * nb, block_size)
        bs = block_size
    else:
        blk_amax = torch.zeros(n, dtype=torch.float32, device=dev)
        _hip.absmax_into(w, blk_amax, 1, n, k)
        bs = k
    acc = torch.zeros(k, dtype=torch.float32, device=dev)
    _hip.abs_colsum_into(w, acc, blk_amax, bs)
    return (acc / n).to(weight.dtype).to(torch.float32)


def get_act_scale(x):
    """fp32 [K]: mean over tokens of ``|x|`` rounded in the activation dtype."""
    x2 = x.contiguous().view(-1, x.shape[-1])
    acc = torch.zeros(x2.shape[1], dtype=torch.float32, device=x.device)
    _hip.abs_colsum_into(x2, acc)
    return (acc / x2.shape[0]).to(x.dtype).to(torch.float32)


@functools.lru_cache(maxsize=64)
def _exponent_table_cached(alphas: tuple, device):
    """fp32 ``[4, A]`` on the device: alpha, 1 - alpha (the difference taken in double, as the
    scalar form of ``pow`` does before it narrows the exponent), and for each of the two how the
    power is evaluated -- 0 ``pow``; the exponents the scalar form of ``pow`` evaluates without
    calling it: 1 the constant one (exponent 0), 2 the base itself (exponent 1), 3 the correctly
    rounded square root (exponent 0.5, see ``_pow``)."""
    def mode(e):
        return {0.0: 1.0, 1.0: 2.0, 0.5: 3.0}.get(e, 0.0)
    a = [float(v) for v in alphas]
    b = [1 - v for v in a]
    return torch.tensor([a, b, [mode(v) for v in a], [mode(v) for v in b]], dtype=torch.float32).to(device)


def _exponent_table(alphas, device):
    """Built once per alpha grid and device."""
    return _exponent_table_cached(tuple(float(v) for v in alphas), torch.device(device))


def get_scales(x_max, w_max, alphas, table=None, dtype=None):
    """fp32 ``[len(alphas), K]``: row i is the AWQ scale ``x^a / w^(1-a)`` for ``a = alphas[i]``,
    clamped to [1e-4, 1e4] and normalised by ``sqrt(max * min)`` of its own row -- the whole
    search grid in one launch.  With ``dtype`` also the two rounded copies a search step
    multiplies with: ``(scales, dtype(scales), dtype(1 / scales))``."""
    dev = x_max.device
    table = table if table is not None else _exponent_table(alphas, dev)
    made = _hip.awq_scale_grid(x_max.float().contiguous().view(-1), w_max.to(dev).float().contiguous().view(-1),
                               table, dtype if dtype is not None else torch.float32)
    return made if dtype is not None else made[0]


def get_scale(x_max, w_max, alpha):
    """fp32 ``[K]``: the AWQ scale for one ``alpha`` (a one-row ``get_scales``, so the folded
    scale is bit for bit the one the search scored)."""
    return get_scales(x_max, w_max, [alpha])[0]


@functools.lru_cache(maxsize=16)
def _alpha_grid(alpha_step: float):
    """The alphas of the search grid as the reference builds them (model_calib.py:563: the fp32
    ``torch.arange`` values read back as Python floats), once per step size."""
    return tuple(k.item() for k in torch.arange(0, 1.0 + alpha_step, alpha_step))


class _AWQLiteHelper:
    cache_mode: bool = False

    def __init__(self, module, name, alpha_step):
        self.name = name
        self.act_scale = 0.0
        self.num_cache_steps = 0
        self.num_search_steps = 0
        self.block_size = _awq_block_size(module.weight, module.weight_quantizer)
        self.weight_scale = get_weight_scale(module.weight, self.block_size)
        dev = module.weight.device
        self.alphas = list(_alpha_grid(float(alpha_step)))
        self.sq_err_steps = []  # per search step: (float64 [n_alphas] sums of squared error, numel)
        self.loss = {a: 0.0 for a in self.alphas}
        self.best_scale = None
        self.best_alpha = None
        self.exponent_columns = None  # device table of the exponents, made on first search step
        self.scale_grid = None        # (fp32 scales [n_alphas, K], weight-dtype copy, inverse) of the search
        self.is_input_quantized = module.input_quantizer.is_enabled
        self.num_tokens = 0
        self.module = module
        self.is_enabled = True

    def setup(self):
        m = self.module
        # plain values: written past nn.Module.__setattr__, which would look through the
        # parameters, buffers and submodules for each
        m.__dict__["_forward_no_awq"] = m.forward
        m.__dict__["forward"] = types.MethodType(_awq_forward, m)
        if m.input_quantizer.is_enabled:
            m.input_quantizer.disable()
            if m.input_quantizer.axis not in (None, -1):
                self.is_enabled = False
                return
            m.input_quantizer.axis = -1

    def cleanup(self):
        m = self.module
        if hasattr(m, "_if_calib"):
            delattr(m, "_if_calib")
        if "forward" in m.__dict__:
            del m.__dict__["forward"]
        if hasattr(m, "_forward_no_awq"):
            del m.__dict__["_forward_no_awq"]


def _fused_weight_path(module):
    """True when the weight quantizer is a plain static last-axis INT block quantizer, so the
    per-alpha weight path can run as one fused kernel."""
    q = module.weight_quantizer
    if not isinstance(q, TensorQuantizer) or not isinstance(q._num_bits, int):
        return False
    bs = q.block_sizes
    if not bs or bs.get("type", "static") == "dynamic" or not q.fake_quant or hasattr(q, "_amax"):
        return False
    axes = {k: v for k, v in bs.items() if isinstance(k, int)}
    if list(axes) not in ([-1], [module.weight.dim() - 1]):
        return False
    b = next(iter(axes.values()))
    return b in (8, 16, 32, 64, 128, 256, 512) and module.weight.dtype in (
        torch.bfloat16, torch.float16, torch.float32)


_SEARCH_TOKENS = 512   # token rows one launch of the search kernel takes (mo_awq_search_losses)


def _one_launch_search(module, x, w, ref, x_scales, w_scales, block, sq_err) -> bool:
    """All alphas of a search step in one kernel launch per 512 tokens (weights quantised on the
    fly in front of the matrix cores, the loss reduced in the epilogue): used when the layer is a
    plain bf16 linear (with or without bias) whose input and output quantizers are switched off.  The loss
    is a sum over tokens, so a longer batch goes through in slices of 512 rows that add into the
    same ``sq_err`` (per-alpha launches with a library GEMM cost more at every batch size: they
    re-scale and re-quantise per alpha and pass over the activations three times).
    Returns False, with nothing launched and ``sq_err`` untouched, when the layer is not covered."""
    bias = module.bias
    if w.dtype != torch.bfloat16 or x.dtype != torch.bfloat16 or (bias is not None and bias.dtype != w.dtype):
        return False
    for name in ("input_quantizer", "output_quantizer"):
        quantizer = getattr(module, name, None)
        if not isinstance(quantizer, TensorQuantizer) or quantizer.is_enabled:
            return False
    n, k = w.shape
    tokens = x.numel() // k
    q = module.weight_quantizer
    # what mo_awq_search_losses takes, checked before the activations of every alpha are written
    # out for it (n_alpha x tokens x K values)
    if (tokens == 0 or k % 128 or n % 128 or block not in (32, 64, 128) or q._unsigned
            or any(t.data_ptr() % 16 for t in (x, w, w_scales, x_scales))):
        return False
    rows, outs = x.view(tokens, k), ref.view(tokens, -1)
    for t0 in range(0, tokens, _SEARCH_TOKENS):
        t1 = min(tokens, t0 + _SEARCH_TOKENS)
        xs = _hip.awq_scaled_activations(rows[t0:t1], x_scales)
        if not _hip.awq_search_losses_into(xs, w, w_scales, outs[t0:t1], block, q._num_bits, q._unsigned,
                                           q._narrow_range, sq_err,
                                           None if bias is None else bias.data.contiguous()):
            if t0:   # cannot happen: every slice has the shape the first one was accepted with
                raise RuntimeError("the search kernel refused a later slice of a batch it had started on")
            return False
    return True


def _awq_forward(self, input, *args, **kwargs):
    """Replacement ``forward`` of a quantised linear during AWQ-lite (cache pass, then search)."""
    helper = self.awq_lite
    self.weight_quantizer.disable()
    for q in (self.input_quantizer, self.weight_quantizer):
        if "_pre_quant_scale" in q._buffers or "_pre_quant_scale" in q.__dict__:
            delattr(q, "_pre_quant_scale")
    out_actual = self._forward_no_awq(input, *args, **kwargs)
    self.weight_quantizer.enable()
    if input.numel() == 0 or not helper.is_enabled:
        return out_actual

    if _AWQLiteHelper.cache_mode:
        helper.act_scale += get_act_scale(self.input_quantizer(input))
        helper.num_cache_steps += 1
        helper.num_tokens += input.numel() / input.shape[-1]
        if helper.is_input_quantized:
            with set_quantizer_by_cfg_context(self.input_quantizer, {"*": {"enable": True}}):
                max_calibrate(self.input_quantizer, lambda quantizer: quantizer(input), False)
        return out_actual

    ref = out_actual[0] if isinstance(out_actual, tuple) else out_actual
    ref = ref.contiguous()
    dtype = self.weight.dtype
    fused = _fused_weight_path(self) and not args and not kwargs
    sq_err = torch.zeros(len(helper.alphas), dtype=torch.float64, device=ref.device)
    if helper.exponent_columns is None or helper.exponent_columns.device != ref.device:
        helper.exponent_columns = _exponent_table(helper.alphas, ref.device)
    # the candidate scales depend on the cached statistics only: built at the first search step,
    # reused by the later ones, and the best row is folded when the search is over
    grid = helper.scale_grid
    if grid is None or grid[1].dtype != dtype or grid[0].device != ref.device:
        grid = helper.scale_grid = get_scales(helper.act_scale, helper.weight_scale, helper.alphas,
                                              helper.exponent_columns, dtype)
    _, w_scales, x_scales = grid
    if fused:
        q = self.weight_quantizer
        x_in = input.contiguous()
        w_in = self.weight.data.contiguous()
        block = _awq_block_size(self.weight, q)
        if _one_launch_search(self, x_in, w_in, ref, x_scales, w_scales, block, sq_err):
            helper.sq_err_steps.append((sq_err, ref.numel()))
            helper.num_search_steps += 1
            return out_actual
    # a plain quantised linear (``F.linear`` between its three quantizers) whose weight
    # quantizer is of another kind -- NVFP4, a sequential INT4 + FP8 pair -- still needs neither
    # the scale buffers on the quantizers nor the trip through the module's forward: a
    # quantizer multiplies by its pre-quant scale before anything else, in the tensor's dtype,
    # which is the column scaling below
    plain = (not fused and not args and not kwargs
             and getattr(self._forward_no_awq, "__func__", None) is _QuantLinear.forward
             and input.is_cuda and self.weight.dim() == 2)
    if plain:
        x_in = input.contiguous()
        w_in = self.weight.data.contiguous()
    for i in range(len(helper.alphas)):
        if fused:
            xs = self.input_quantizer(_hip.mul_cols(x_in, x_scales[i]))
            wq = _hip.scale_block_int_qdq(w_in, w_scales[i], block, q._num_bits, q._unsigned,
                                          q._narrow_range)
            out = self.output_quantizer(F.linear(xs, wq, self.bias))
        elif plain:
            xs = self.input_quantizer(_hip.mul_cols(x_in, x_scales[i]))
            wq = self.weight_quantizer(_hip.mul_cols(w_in, w_scales[i]))
            out = self.output_quantizer(F.linear(xs, wq, self.bias))
        else:
            self.input_quantizer.pre_quant_scale = x_scales[i]
            self.weight_quantizer.pre_quant_scale = w_scales[i]
            out = self._forward_no_awq(input, *args, **kwargs)
            out = out[0] if isinstance(out, tuple) else out
        _hip.sq_diff_sum_into(out.contiguous(), ref, sq_err[i:i + 1])
    helper.sq_err_steps.append((sq_err, ref.numel()))
    helper.num_search_steps += 1
    return out_actual


def _losses_on_device(helper):
    """float64 ``[n_alphas]`` on the device: loss[alpha] = sum over search steps of that step's mean
    squared error (the kernels leave per-step sums of squares there); None without search steps."""
    if not helper.sq_err_steps:
        return None
    # the element counts go in as scalars: a host tensor would have to be copied to the device,
    # which waits for everything queued on the stream
    total = None
    for sums, n in helper.sq_err_steps:
        mean = sums / float(n)
        total = mean if total is None else total + mean
    return total


_SMOOTH_IN_ONE_LAUNCH = True   # False: the tensor expressions of smoothquant's postprocess instead
_PICK_IN_ONE_LAUNCH = True   # False: the tensor expressions below instead (kept for tests that compare the two)


def _first_minimum(loss):
    """Index (0-dim int64 on the device) that ``min(dict, key=dict.get)`` would pick: the first
    smallest value; a NaN is never smaller than anything, and a NaN in front is never replaced."""
    key = torch.where(torch.isnan(loss), torch.full_like(loss, float("inf")), loss)
    idx = torch.argmin(key)
    return torch.where(torch.isnan(loss[0]), torch.zeros_like(idx), idx)


@torch.no_grad()
def awq_lite(model: nn.Module, forward_loop, alpha_step: float = 0.1, debug: bool = False, **kwargs):
    """AWQ-lite: per linear, search ``alpha`` of the scale ``s = act^alpha / w^(1-alpha)`` that
    minimises the output error of the quantised layer, then fold the best scale."""
    if forward_loop is None:
        warnings.warn("forward_loop must be provided for awq_lite; skipping awq_lite")
        return

    for name, module in model.named_modules():
        if is_quantized_linear(module) and module.weight_quantizer.is_enabled:
            helper = module.__dict__["awq_lite"] = _AWQLiteHelper(module, name, alpha_step)   # a plain attribute
            helper.setup()

    _AWQLiteHelper.cache_mode = True
    print("awq_lite: Caching activation statistics...")
    enable_stats_collection(model)
    with calibration_pass():
        forward_loop(model)
    max_calibrate(model, lambda model: None)

    cached = []
    for name, module in model.named_modules():
        if "awq_lite" in module.__dict__ and is_quantized_linear(module) and module.awq_lite.num_cache_steps > 0:
            module.__dict__["_if_calib"] = True
            h = module.awq_lite
            h.act_scale = h.act_scale / h.num_cache_steps
            cached.append(h)
    if cached:  # one host synchronisation for the NaN checks of all layers
        stats = [t for h in cached for t in (h.act_scale, h.weight_scale)]
        ranges = _hip.value_ranges(stats) if all(isinstance(t, torch.Tensor) for t in stats) else None
        if ranges is not None:   # a handful of layers: one launch as well
            flags = [ranges[2 * i][2] or ranges[2 * i + 1][2] for i in range(len(cached))]
        else:
            flags = torch.stack([torch.isnan(h.act_scale).any() | torch.isnan(h.weight_scale).any()
                                 for h in cached]).tolist()
        for h, bad in zip(cached, flags):
            if bad:
                h.is_enabled = False

    _AWQLiteHelper.cache_mode = False
    print("awq_lite: Searching parameters...")
    forward_loop(model)

    # The best alpha is picked on the device and the checks are collected, so that folding the
    # scales of one layer does not wait for the search kernels of the layers behind it: one host
    # synchronisation at the end instead of three per layer.
    searched = []

    def postprocess(module, name):
        h = module.awq_lite
        folded = None   # (1 / best_scale, the same in the weight's dtype, 1 / (1 / best_scale)) when made on the way
        if h.is_enabled:
            loss = _losses_on_device(h)
            if loss is None:
                h.loss = {a: 0.0 for a in h.alphas}
                h.best_alpha = min(h.loss, key=h.loss.get)
                h.best_scale = get_scale(h.act_scale, h.weight_scale, h.best_alpha)
            else:
                grid = h.scale_grid[0] if h.scale_grid is not None else get_scales(
                    h.act_scale, h.weight_scale, h.alphas, h.exponent_columns)
                if (_PICK_IN_ONE_LAUNCH and loss.is_cuda and loss.dtype == torch.float64
                        and grid.dtype == torch.float32 and module.weight.dtype in _hip._DTYPES):
                    # the row the search scored and what the folding makes of it, in one launch
                    best, h.best_scale, *folded = _hip.awq_pick_scale(
                        loss.contiguous(), grid.contiguous(), module.weight.dtype)
                else:
                    best = _first_minimum(loss)
                    h.best_scale = grid.index_select(0, best.reshape(1))[0]
                h.scale_grid = None
                searched.append((h, loss, best))
        for q in (module.weight_quantizer, module.input_quantizer):
            if hasattr(q, "_pre_quant_scale"):
                delattr(q, "_pre_quant_scale")
        if h.is_input_quantized and module.input_quantizer.amax is not None:
            act_amax = module.input_quantizer.amax
            module.input_quantizer._amax_for_smoothing = _host_copy_later(act_amax)
            module.input_quantizer.reset_amax()
            module.input_quantizer.axis = None
            module.input_quantizer.amax = act_amax.amax()
            module.input_quantizer.enable()
        if h.is_enabled:
            if folded:
                apply_pre_quant_scale_and_smooth(module, folded[0], _rounded=folded[1], _fold=folded[2])
            else:
                apply_pre_quant_scale_and_smooth(module, 1.0 / h.best_scale)
        else:
            warnings.warn(f"awq_lite: Disabling for {name}, quantizing with max calibration.")
            max_calibrate(module, lambda module: module.weight_quantizer(module.weight))

    kept = []
    with deferred_scale_checks():
        for name, module in model.named_modules():
            if hasattr(module, "awq_lite"):
                h = module.awq_lite
                if h.num_cache_steps == 0:
                    h.is_enabled = False
                elif h.num_search_steps == 0:
                    h.is_enabled = False
                    warnings.warn(
                        "awq_lite: Calling `forward_loop(model)` the second time did not forward data "
                        f"through the {name}. Please provide a valid `forward_loop` function that can "
                        "be used to forward data through the model many times.")
                postprocess(module, name)
                h.cleanup()
                if debug:
                    kept.append(h)
                else:
                    delattr(module, "awq_lite")
    if kept:  # the helpers stay on the modules: give them the numbers as Python values
        for h, loss, best in searched:
            h.loss = dict(zip(h.alphas, loss.tolist()))
            h.best_alpha = h.alphas[int(best)]
