"""``TensorQuantizer`` and ``SequentialQuantizer``.

Attribute names, buffers (``_amax``, ``_pre_quant_scale``, ``_scale``, ``_double_scale``,
``_scale_zeros``), the order of operations in ``forward`` and the exported amax shapes follow
the reference module (modelopt/torch/quantization/nn/modules/tensor_quantizer.py:65-1225); the
arithmetic runs in the HIP kernels.  Not built: affine bias, Hadamard rotation, ONNX export hooks.
"""

import contextlib
import math
import warnings
from typing import Any

import torch
import torch.nn.functional as F
from torch import nn
from torch.nn.modules import module as _module_hooks

from ... import calib, kernels, modes
from ... import utils as quant_utils
from ...config import QuantizerAttributeConfig
from ...qtensor import (BaseQuantizedTensor, FP8QTensor, INT4QTensor, INT8QTensor, MXFP4QTensor,
                        NF4QTensor, NVFP4QTensor, QTensorWrapper)
from ...overflow import get_fp8_overflow_behavior
from ...tensor_quant import dynamic_block_quant, fake_tensor_quant, scaled_e4m3

__all__ = ["SequentialQuantizer", "TensorQuantizer"]

_DEFAULT_CONFIG = []


def _default_config():
    """The all-defaults config, built (and validated) once: a model conversion creates three
    quantizers per layer and only reads it."""
    if not _DEFAULT_CONFIG:
        _DEFAULT_CONFIG.append(QuantizerAttributeConfig())
    return _DEFAULT_CONFIG[0]


# [id of the calibration pass in progress, or 0]; the weight abs-max cache is only valid inside one
_CALIBRATION_PASS = [0]
_PASS_COUNTER = [0]


@contextlib.contextmanager
def calibration_pass():
    """Marks one ``forward_loop`` run by the package's calibration drivers: within it a weight
    that has not changed is reduced once, not once per forward."""
    _PASS_COUNTER[0] += 1
    previous, _CALIBRATION_PASS[0] = _CALIBRATION_PASS[0], _PASS_COUNTER[0]
    shared, calib.max.SHARE_REDUCTIONS[0] = calib.max.SHARE_REDUCTIONS[0], True
    try:
        yield
    finally:
        _CALIBRATION_PASS[0] = previous
        calib.max.SHARE_REDUCTIONS[0] = shared
        calib.max.forget_last_reduction()


class TensorQuantizer(nn.Module):
    """Quantises (fake or real) and calibrates one tensor.

    Args:
        quant_attribute_cfg: a ``QuantizerAttributeConfig`` (defaults when None).
        if_quant: quantise in ``forward``.
        if_calib: collect calibration statistics in ``forward``.
        amax: initial amax (anything ``torch.tensor`` accepts).
    """

    _skip_properties_for_save_restore = {
        "_calibrator", "_bias_calibrator", "_original_shape", "_block_reshape_size", "_padding",
        "_is_hf_initialized",
    }

    def __init__(self, quant_attribute_cfg=None, if_quant=True, if_calib=False, amax=None):
        super().__init__()
        cfg = quant_attribute_cfg if quant_attribute_cfg is not None else _default_config()
        if amax is not None:
            self.amax = amax
        self.set_from_attribute_config(cfg)
        plain = object.__setattr__  # plain python values: skip nn.Module's attribute bookkeeping
        plain(self, "_if_quant", if_quant)
        plain(self, "_if_calib", if_calib)
        plain(self, "_enable_pre_quant_scale", True)
        plain(self, "_dequantize", False)
        plain(self, "_input_dtype", None)

    # Switches and settings (``_if_quant``, ``_disabled``, ``_axis`` ...) are plain python values
    # written thousands of times while a model is converted and calibrated; nn.Module's
    # ``__setattr__`` looks every value up as a parameter, module and buffer first.  A plain value
    # under a name that is none of those goes straight to the instance dict.
    _PLAIN_VALUE_TYPES = (bool, int, float, str, tuple, type(None))

    def __setattr__(self, name, value):
        if (type(value) in TensorQuantizer._PLAIN_VALUE_TYPES and name not in self._buffers
                and name not in self._parameters and name not in self._modules):
            object.__setattr__(self, name, value)
        else:
            super().__setattr__(name, value)

    # ------------------------------------------------------------------ configuration
    def set_from_attribute_config(self, attribute_cfg: QuantizerAttributeConfig | dict):
        """Copy config fields onto ``_<field>`` attributes (``enable`` -> ``_disabled``,
        ``type`` -> ``_dynamic``, ``calibrator`` -> a calibrator instance)."""
        if type(attribute_cfg) is QuantizerAttributeConfig:
            # a complete, validated config: its attribute set is built once per config object.
            # The values are plain python objects (never tensors or modules), so they go straight
            # into the instance dict, past nn.Module's attribute bookkeeping
            plain, calibrator = attribute_cfg.quantizer_attributes()
            own = self.__dict__
            own.update(plain)
            for name in ("_block_sizes", "_bias"):   # a quantizer owns its mutable settings
                if own[name] is not None:
                    own[name] = dict(own[name])
            own["_calibrator"] = self._make_calibrator(calibrator)
            if self.is_mx_format:
                self._pass_through_bwd = True
            return
        items = attribute_cfg.items()
        fields = QuantizerAttributeConfig.model_fields
        for name, val in items:
            assert name in fields, f"{name} is not a valid `TensorQuantizer` attribute"
        # the values are plain python objects (never tensors or modules), so they can skip
        # nn.Module's attribute bookkeeping
        plain = object.__setattr__
        for name, val in items:
            if name == "enable":
                plain(self, "_disabled", val is False)
            elif name == "type":
                plain(self, "_dynamic", val == "dynamic")
            elif name == "calibrator":
                continue
            else:
                plain(self, f"_{name}", val)
        for name, val in items:
            if name == "calibrator":
                plain(self, "_calibrator", self._make_calibrator(val))
        if self.is_mx_format:
            self._pass_through_bwd = True

    def _make_calibrator(self, spec):
        num_bits = getattr(self, "_num_bits", 8)
        axis = getattr(self, "_axis", None)
        unsigned = getattr(self, "_unsigned", False)
        if spec == "max":
            return calib.MaxCalibrator(num_bits, axis, unsigned)
        if spec == "histogram":
            raise NotImplementedError("the histogram calibrator is outside the hot path built here")
        if isinstance(spec, type):
            return spec(num_bits, axis, unsigned)
        if isinstance(spec, (tuple, list)):
            cls, *rest = spec
            args = rest[0] if len(rest) > 0 else ()
            kwargs = rest[1] if len(rest) > 1 else {}
            return cls(*args, **kwargs)
        raise ValueError(f"cannot build a calibrator from {spec!r}")

    # ------------------------------------------------------------------ properties
    @property
    def num_bits(self):
        return self._num_bits

    @num_bits.setter
    def num_bits(self, value):
        self._num_bits = value
        self._calibrator._num_bits = value

    @property
    def maxbound(self):
        """Largest representable magnitude of the target format."""
        if self._num_bits == (4, 3):
            return 448.0
        if self._num_bits == (2, 1) and self._block_sizes.get("scale_bits") == (4, 3):
            return 6.0
        return (1 << (self._num_bits - 1 + int(self._unsigned))) - 1

    @property
    def unsigned(self):
        return self._unsigned

    @unsigned.setter
    def unsigned(self, value):
        self._unsigned = value
        self._calibrator._unsigned = value

    @property
    def pre_quant_scale(self):
        if not hasattr(self, "_pre_quant_scale") or not self._enable_pre_quant_scale:
            return None
        return self._pre_quant_scale

    @pre_quant_scale.setter
    def pre_quant_scale(self, value):
        assert value is not None, "pre_quant_scale cannot be set to None."
        assert self._enable_pre_quant_scale, (
            "pre_quant_scale cannot be set when forward_with_pre_quant_scale is False.")
        if not isinstance(value, torch.Tensor):
            value = torch.tensor(value)
        if not hasattr(self, "_pre_quant_scale"):
            self.register_buffer("_pre_quant_scale", value.clone().detach())
        else:
            if self._pre_quant_scale.shape != value.shape:
                raise RuntimeError("Changing shape when setting pre_quant_scale is not allowed.")
            self._pre_quant_scale.data.copy_(value.clone().detach().to(self._pre_quant_scale.device))

    @property
    def amax(self):
        if not hasattr(self, "_amax") or self.is_mx_format:
            return None
        assert not self._dynamic, "Dynamic quantization does not have fixed amax"
        return self._amax

    @amax.setter
    def amax(self, value):
        assert value is not None, "amax cannot be set to None."
        if not isinstance(value, torch.Tensor):
            value = torch.tensor(value)
        if not hasattr(self, "_amax"):
            self.register_buffer("_amax", value.clone().detach())
        else:
            if self._amax.shape != value.shape:
                raise RuntimeError("Changing shape when setting amax is not allowed.")
            self._amax.data.copy_(value.clone().detach().to(self._amax.device))

    def reset_amax(self):
        if hasattr(self, "_amax"):
            delattr(self, "_amax")
        self._calibrator.reset()

    @property
    def step_size(self):
        if not hasattr(self, "_amax"):
            warnings.warn("step_size is undefined under dynamic amax mode!")
            return None
        assert isinstance(self._num_bits, int), "Step size is not defined for non-integer quantization."
        return quant_utils.true_divide(self._amax, 2.0 ** (self._num_bits - 1 + int(self._unsigned)) - 1.0)

    @property
    def axis(self):
        return self._axis

    @axis.setter
    def axis(self, value):
        self._axis = value
        self._calibrator._axis = value

    @property
    def block_sizes(self):
        return self._block_sizes

    @block_sizes.setter
    def block_sizes(self, value):
        self._axis = None
        self._block_sizes = value

    @property
    def bias(self):
        return None

    @property
    def fake_quant(self):
        return self._fake_quant

    @property
    def narrow_range(self):
        return self._narrow_range

    @narrow_range.setter
    def narrow_range(self, value):
        self._narrow_range = value

    @property
    def is_enabled(self):
        return not self._disabled

    def disable(self):
        """Bypass: no calibration, clipping or quantisation."""
        self._disabled = True

    def enable(self):
        self._disabled = False

    @property
    def trt_high_precision_dtype(self):
        return self._trt_high_precision_dtype

    @trt_high_precision_dtype.setter
    def trt_high_precision_dtype(self, value):
        self._trt_high_precision_dtype = value

    @property
    def is_mx_format(self):
        bs = self.block_sizes
        return bs is not None and bs.get("type") == "dynamic" and bs.get("scale_bits") == (8, 0)

    @property
    def is_static_block_quant(self):
        bs = self.block_sizes
        return bs is not None and bs.get("type") != "dynamic" and self._fake_quant

    def disable_calib(self):
        self._if_calib = False

    def enable_calib(self):
        if self._calibrator is None:
            raise ValueError("Calibrator was not created, cannot enable calibration.")
        if self._dynamic:  # dynamic quantisation has nothing to calibrate
            return
        self._if_calib = True

    def disable_quant(self):
        self._if_quant = False

    def enable_quant(self):
        self._if_quant = True

    # ------------------------------------------------------------------ calibration results
    def load_calib_amax(self, *args, **kwargs):
        """Create / update the ``_amax`` buffer from the calibrator."""
        assert not self._dynamic, "Dynamic quantization does not need calibration."
        strict = kwargs.pop("strict", True)
        if getattr(self, "_calibrator", None) is None:
            raise RuntimeError("Calibrator not created.")
        calib_amax = self._calibrator.compute_amax(*args, **kwargs)
        if calib_amax is None:
            msg = "Calibrator returned None. This usually happens when calibrator hasn't seen any tensor."
            if strict:
                raise RuntimeError(msg + " Passing 'strict=False' to `load_calib_amax()` will ignore the error.")
            warnings.warn(msg)
            warnings.warn("Set amax to NaN!")
            calib_amax = torch.tensor(math.nan)
        if type(self._calibrator) is calib.MaxCalibrator and calib_amax.device.type != "meta":
            fresh = calib_amax.detach()          # already a tensor of its own
        else:
            fresh = calib_amax.clone().detach()
        if not hasattr(self, "_amax"):
            self.register_buffer("_amax", fresh)
        else:
            self._amax.data.copy_(fresh)

    def _get_amax(self, inputs):
        """The calibrated ``_amax`` buffer, or the abs-max of ``inputs`` computed now."""
        if hasattr(self, "_amax"):
            if self._amax.device != inputs.device:  # e.g. an amax assigned from a CPU scalar
                self._amax = self._amax.to(inputs.device)
            return self._amax.data
        reduce_axis = quant_utils.convert_quantization_axis_to_reduce_axis(inputs, self._axis)
        # dynamic quantisation: the fake quant reads ``inputs`` again as soon as this returns
        return quant_utils.reduce_amax(inputs, axis=reduce_axis, keepdims=True,
                                       squeeze_scalar=True, reread=True).detach()

    def validate_attr(self, attr_value=None, attr_name="amax", raise_error=False, warn_error=False,
                      name=""):
        value = attr_value if attr_value is not None else getattr(self, attr_name, None)
        if value is None or (isinstance(value, torch.Tensor) and value.is_meta):
            return True
        ok = bool(torch.all(value >= 0) and not torch.any(torch.isinf(value))
                  and not torch.any(torch.isnan(value)))
        if ok:
            return True
        prefix = f"{name}." if name else ""
        msg = f"{prefix}{attr_name} contains invalid values: {value}"
        if warn_error:
            warnings.warn(msg)
        if raise_error:
            raise ValueError(msg)
        return False

    # ------------------------------------------------------------------ real quantisation
    def _is_real_quantize_support(self):
        return bool((self._num_bits == 4 and self._block_sizes)
                    or (self._num_bits == (2, 1) and self._block_sizes)
                    or self._num_bits in ((4, 3), 8))

    def dequantize(self, inputs):
        qtensor = inputs.get_qtensor() if isinstance(inputs, QTensorWrapper) else inputs
        assert isinstance(qtensor, BaseQuantizedTensor), "Expected input as real quantized tensors."
        return qtensor.dequantize(scale=self._scale, block_sizes=self.block_sizes,
                                  double_scale=getattr(self, "_double_scale", None),
                                  scale_zeros=getattr(self, "_scale_zeros", None))

    def _real_quantize(self, inputs):
        assert self._is_real_quantize_support(), "Real quantization not supported for this format."
        buffers = {}
        bs = self._block_sizes
        if self._num_bits == (4, 3):
            use_amax = self.amax is not None and not (bs and self.amax.numel() == 1)
            outputs, scale = FP8QTensor.quantize(inputs, axis=self._axis, block_sizes=bs,
                                                 scales=quant_utils.true_divide(self.amax, 448.0) if use_amax else None)
            buffers["_scale"] = scale
        elif self._num_bits == 8:
            outputs, scale = INT8QTensor.quantize(inputs, axis=self._axis, block_sizes=bs)
            buffers["_scale"] = scale
        elif bs.get("scale_bits", 0) == 8 and bs.get("scale_block_sizes"):
            sbs = bs["scale_block_sizes"][-1]
            outputs, scales = NF4QTensor.quantize(inputs, bs[-1], sbs)
            scale, double_scale, zeros = NF4QTensor.double_quantization(scales, sbs, bs["scale_bits"])
            buffers["_scale"], buffers["_double_scale"], buffers["_scale_zeros"] = scale, double_scale, zeros
        elif bs.get("scale_bits") == (8, 0) and bs.get("type") == "dynamic":
            if self._num_bits != (2, 1):
                raise NotImplementedError("of the MX formats only MXFP4 has a packed tensor class")
            outputs, scale = MXFP4QTensor.quantize(inputs, bs[-1])
            buffers["_scale"] = scale
        elif bs.get("scale_bits") == (4, 3):
            if self.amax is not None and self._amax.device != inputs.device:
                self._amax = self._amax.to(inputs.device)
            wsf2 = (quant_utils.true_divide(self.amax.float(), 448.0 * 6.0)
                    if self.amax is not None else None)
            outputs, wsf, wsf2 = NVFP4QTensor.quantize(inputs, bs[-1], weights_scaling_factor_2=wsf2)
            buffers["_scale"], buffers["_double_scale"] = wsf, wsf2
        else:
            outputs, scale = INT4QTensor.quantize(inputs, bs[-1])
            buffers["_scale"] = scale
        for k, v in buffers.items():
            self._set_buffer(k, v)
        self._dequantize = True  # later forwards on the packed tensor only dequantise
        return outputs

    # ------------------------------------------------------------------ fake quantisation
    def _fused_dynamic_per_tensor(self, inputs):
        """Dynamic per-tensor INT / FP8 fake quantisation (no calibrated ``_amax``, no axis, no
        blocks) outside autograd: abs-max and quantize-dequantize in one launch that reads the
        tensor once, when ``modes.set_one_launch_dynamic_quant(True)`` allows it.  None when that
        case does not apply or the tensor is too large for it."""
        if not modes.one_launch_dynamic_quant() or modes.strict_checks():
            return None
        if hasattr(self, "_amax") or self._axis is not None or self.block_sizes is not None:
            return None
        if not inputs.is_cuda or (inputs.requires_grad and torch.is_grad_enabled()):
            return None
        if getattr(self, "_bias_calibrator", None) is not None or self.is_mx_format:
            return None
        if isinstance(self._num_bits, tuple):
            if self._num_bits != (4, 3):
                return None
            # a per-tensor amax goes to the reference's clamping kernel unless "nan" is selected
            done = kernels._hip.fused_amax_qdq(inputs, "fp8", saturate=get_fp8_overflow_behavior() != "nan")
        else:
            done = kernels._hip.fused_amax_qdq(inputs, "int", self._num_bits, self._unsigned,
                                               self._narrow_range)
        return None if done is None else done[0]

    def _fake_quantize(self, inputs):
        fused = self._fused_dynamic_per_tensor(inputs)
        if fused is not None:
            return fused
        amax = None if self.is_mx_format else self._get_amax(inputs)
        bs = self.block_sizes
        if bs is not None and bs.get("type", "static") == "dynamic":
            block = bs.get(-1) or bs.get(inputs.dim() - 1)
            if block is None:
                raise ValueError("block size for dynamic quantization not found.")
            return dynamic_block_quant(inputs, block, amax, None, self._num_bits,
                                       bs.get("scale_bits"),
                                       getattr(self, "_trt_high_precision_dtype", None),
                                       getattr(self, "_onnx_quantizer_type", None),
                                       self._pass_through_bwd)
        if isinstance(self._num_bits, tuple):
            e, m = self._num_bits
            return scaled_e4m3(inputs, amax, None, e, m, self._trt_high_precision_dtype,
                               self._pass_through_bwd)
        return fake_tensor_quant(inputs, amax, None, self._num_bits, self._unsigned,
                                 self._narrow_range, self._trt_high_precision_dtype,
                                 self._pass_through_bwd, bs.get(-1) if bs else None,
                                 self.axis[0] if isinstance(self.axis, tuple) else self.axis)

    # ------------------------------------------------------------------ static block reshaping
    def _setup_for_blockquant(self, inputs: torch.Tensor):
        """Decide once how the input is padded and reshaped so that every block becomes a row
        (last-axis blocks) or its own dim (general case), and which dims carry the amax."""
        if hasattr(self, "_block_reshape_size"):
            return
        bs = self.block_sizes
        nd = inputs.dim()

        def axis_params(ax):
            key = ax if ax in bs else ax - nd
            size = bs.get(key)
            pad, sl = None, None
            if size is not None and inputs.shape[ax] % size != 0:
                pad = (size - inputs.shape[ax] % size, 0)
                sl = slice(inputs.shape[ax])
            return size, pad, sl

        def commit(axis, reshape, padding, slices, amax_shape=None):
            self._axis = tuple(axis)
            if hasattr(self, "_calibrator"):
                self._calibrator._axis = self._axis
            self._original_shape = inputs.shape
            self._block_reshape_size = torch.Size(reshape)
            if padding is not None:
                self._padding = tuple(padding)
                self._original_shape = F.pad(inputs, self._padding, "constant", 0).shape
            if slices is not None:
                self._slices = slices
            if amax_shape:
                self._amax_shape_for_export = amax_shape

        block_axes = QuantizerAttributeConfig._get_block_quant_axes_and_sizes(bs)
        if (bs.get(nd - 1) or bs.get(-1)) and len(block_axes) == 1:
            # blocks along the last axis only: flatten to rows of one block each
            size, pad, sl = axis_params(nd - 1)
            slices = None if sl is None else (*(slice(None),) * (nd - 1), sl)
            pad = pad if not pad else tuple(reversed(pad))
            commit((0,), (-1, size), pad, slices, (*inputs.shape[:-1], -1))
            return

        reshape, keep, pads, slices = [], [], [], []
        for ax in range(nd):
            size, pad, sl = axis_params(ax)
            pads.append(pad)
            slices.append(sl)
            if size is not None:
                reshape.extend([math.ceil(inputs.shape[ax] / size), size])
                keep.extend([True, False])
            else:
                reshape.append(inputs.shape[ax])
                keep.append(True)
        quant_axis = [i for i, k in enumerate(keep) if k]
        slices = None if all(s is None for s in slices) else [s if s else slice(None) for s in slices]
        if all(p is None for p in pads):
            padding = None
        else:
            flat = []
            for p in pads:
                if not (flat or p):
                    continue
                flat.extend(p if p else (0, 0))
            padding = tuple(reversed(flat))
        commit(quant_axis, reshape, padding, slices)

    def _process_for_blockquant(self, inputs: torch.Tensor):
        if hasattr(self, "_padding"):
            inputs = F.pad(inputs, self._padding, "constant", 0)
        if inputs.shape != self._original_shape:
            raise ValueError(f"Input shape has changed from {self._original_shape} to {inputs.shape}."
                             " Block-quantization requires a fixed input shape.")
        return inputs.reshape(self._block_reshape_size)

    def _reset_to_original_shape(self, outputs: torch.Tensor):
        outputs = outputs.reshape(self._original_shape)
        if hasattr(self, "_slices"):
            outputs = outputs[tuple(self._slices)]
        return outputs

    def _block_sizes_to_axis(self, x: torch.Tensor):
        """``block_sizes = {dim: None, ...}`` (whole-dim blocks) is per-channel quantisation in
        disguise: turn it into ``axis`` and drop ``block_sizes``."""
        bs = self._block_sizes
        if bs is None:
            return
        if all(v is None for k, v in bs.items() if isinstance(k, int)):
            assert self.axis is None, "Axis and block_sizes are both set."
            reduced = tuple(k if k >= 0 else k + x.dim() for k in bs if isinstance(k, int))
            self.axis = tuple(i for i in range(x.dim()) if i not in reduced) or None
            self._block_sizes = None

    def export_amax(self) -> torch.Tensor | None:
        """amax shaped for export: block amax reshaped to ``[..., K / block]``, zeros and NaNs
        replaced by ``maxbound``, clamped to the dtype's finite range."""
        if self.block_sizes is not None and self.block_sizes.get("type") == "dynamic":
            return self.amax
        if self.amax is None:
            return None
        amax = self.amax if not hasattr(self, "_amax_shape_for_export") else self.amax.reshape(
            self._amax_shape_for_export)
        amax[amax == 0] = self.maxbound
        amax = torch.nan_to_num(amax, nan=self.maxbound)
        info = torch.finfo(amax.dtype)
        amax = amax.clamp(min=info.tiny, max=info.max)
        self.validate_attr(attr_name="_amax", attr_value=amax)
        if self.block_sizes is None:
            if self.axis is None:
                amax = amax.unsqueeze(0)
            elif isinstance(self.axis, int) or (isinstance(self.axis, (list, tuple))
                                                and len(self.axis) == 1):
                amax = amax.squeeze()
        return amax

    # ------------------------------------------------------------------ forward
    def _apply_pre_quant_scale(self, inputs):
        pqs = self.pre_quant_scale
        if (inputs.is_cuda and pqs.dtype == inputs.dtype and pqs.numel() == inputs.shape[-1]
                and pqs.shape[-1] == inputs.shape[-1]):
            return kernels.mul_last_dim(inputs, pqs.to(inputs.device))
        return inputs * pqs  # other shapes / mixed dtypes: torch broadcasting and type promotion

    def forward(self, inputs):
        """Scale -> (calibrate) -> (quantise); returns a tensor of the input dtype for fake
        quantisation, a ``QTensorWrapper``-able packed tensor for real quantisation."""
        if isinstance(inputs, (BaseQuantizedTensor, QTensorWrapper)):
            assert self._dequantize, "No dequantization stats in the tensor quantizer."
            return self.dequantize(inputs)
        if inputs.numel() == 0:  # e.g. an MoE expert that saw no token
            return inputs
        source = inputs
        if self.pre_quant_scale is not None:
            inputs = self._apply_pre_quant_scale(inputs)
        if self._rotate:
            raise NotImplementedError("Hadamard rotation is outside the hot path built here")
        if self._disabled:
            self._input_dtype = inputs.dtype if hasattr(inputs, "dtype") else None
            return inputs
        if self.block_sizes is not None and self._fake_quant:
            self._block_sizes_to_axis(inputs)
        if self.is_static_block_quant:
            self._setup_for_blockquant(inputs)
            inputs = self._process_for_blockquant(inputs)
        outputs = inputs
        if self._if_calib and not self._dynamic:
            if self._calibrator is None:
                raise RuntimeError("Calibrator was not created.")
            if not self._seen_this_parameter(source):
                self.collect(inputs)
        if self._if_quant:
            if not inputs.is_contiguous():
                inputs = inputs.contiguous()
            if self.fake_quant:
                outputs = self._fake_quantize(inputs)
            elif not self._dequantize:
                outputs = self._real_quantize(inputs)
            else:
                raise ValueError("self._dequantize is True and self.fake_quant is False. "
                                 "This case should have been handled.")
        if self.is_static_block_quant:
            outputs = self._reset_to_original_shape(outputs)
        return outputs

    # A weight is shown to its quantizer on every forward of a calibration loop.  Inside one
    # ``forward_loop`` run by this package (``calibration_pass``) its abs-max cannot change while
    # the parameter is untouched, so a repeat of the same parameter (same storage, same version
    # counter, same scale) is not reduced again; the running maximum is idempotent, so the
    # calibrated amax is identical.  Outside such a pass -- a caller driving ``enable_calib`` and
    # forwards by hand, who may also write ``weight.data`` in place, which no version counter
    # sees -- every forward reduces again, as the reference does.  Calibrators other than the
    # plain MaxCalibrator (history tracking, user classes) always collect.
    cache_weight_amax = True

    def _seen_this_parameter(self, source) -> bool:
        if not (self.cache_weight_amax and _CALIBRATION_PASS[0] and isinstance(source, nn.Parameter)):
            return False
        cal = self._calibrator
        if type(cal) is not calib.MaxCalibrator or cal._track_amax:
            return False
        pqs = self.pre_quant_scale
        key = (_CALIBRATION_PASS[0], source.data_ptr(), source._version, tuple(source.shape),
               source.dtype, None if pqs is None else (pqs.data_ptr(), pqs._version))
        if getattr(cal, "_seen_parameter", None) == key and getattr(cal, "_acc", None) is not None:
            return True
        cal._seen_parameter = key
        return False

    def collect(self, inputs) -> None:
        if not self._if_calib or self._dynamic:
            return
        self._calibrator.collect(inputs)

    def _only_collects_per_tensor(self) -> bool:
        """``forward`` would do nothing but show the tensor to a per-tensor calibrator and hand
        it back (calibration phase of a plain per-tensor quantizer; no hooks that a direct call
        of the calibrator would skip)."""
        return (type(self) is TensorQuantizer and self._if_calib and not self._if_quant
                and not self._forward_pre_hooks and not self._forward_hooks
                and not _module_hooks._global_forward_pre_hooks and not _module_hooks._global_forward_hooks
                and not self._disabled and not self._dynamic and not self._rotate
                and self._block_sizes is None and self._axis is None
                and self.pre_quant_scale is None and self._calibrator is not None)

    @staticmethod
    def forward_pair(first, x0, second, x1):
        """``(first(x0), second(x1))``; while both quantizers only collect per-tensor statistics
        (calibration of the K / V cache quantizers) the two reductions share one launch."""
        if (first._only_collects_per_tensor() and second._only_collects_per_tensor()
                and isinstance(x0, torch.Tensor) and isinstance(x1, torch.Tensor)
                and x0.numel() and x1.numel()
                and calib.max.collect_pair(first._calibrator, x0, second._calibrator, x1)):
            return x0, x1
        return first(x0), second(x1)

    # ------------------------------------------------------------------ representation / state
    def _short_amax(self, fmt=".4f"):
        if self.is_mx_format:
            return "None"
        if not hasattr(self, "_amax"):
            return "dynamic"
        if self._amax is None:
            return "None"
        if self._amax.is_meta:
            return "meta"
        if self._amax.numel() == 1:
            return f"{self._amax.item():{fmt}}"
        return f"[{self._amax.min().item():{fmt}}, {self._amax.max().item():{fmt}}]({self._amax.numel()})"

    def extra_repr(self):
        if self._disabled:
            return "disabled"
        s = f"{'unsigned ' if self._unsigned else ''}{self._num_bits} bit"
        s += " narrow" if self._narrow_range else ""
        s += " fake" if self._fake_quant else ""
        if self.block_sizes is not None:
            s += f" block_sizes={self._block_sizes},"
        else:
            s += f" axis={self._axis}" if self._axis is not None else " per-tensor"
        s += f" amax={self._short_amax()}"
        s += " pre_quant_scale" if self.pre_quant_scale is not None else ""
        s += f" calibrator={self._calibrator.__class__.__name__}" if self._calibrator is not None else ""
        s += " quant" if self._if_quant else ""
        s += " calib" if self._if_calib else ""
        return s

    def _get_properties_for_modelopt_state(self):
        return self.__dict__.keys() - nn.Module().__dict__.keys() - self._skip_properties_for_save_restore

    def get_modelopt_state(self, properties_only: bool = False) -> dict[str, Any]:
        """Python-side attributes (and buffer shapes unless ``properties_only``) for a checkpoint."""
        state = {k: getattr(self, k) for k in self._get_properties_for_modelopt_state()}
        if properties_only:
            return state
        meta = {"params": {}, "buffers": {}}
        for k, v in self._buffers.items():
            if k not in self._non_persistent_buffers_set:
                meta["buffers"][k] = {"shape": v.shape, "dtype": v.dtype}
        state["_pytorch_state_metadata"] = meta
        return state

    def set_from_modelopt_state(self, modelopt_state, properties_only: bool = False):
        for key in modelopt_state.keys() - self._skip_properties_for_save_restore:
            if key != "_pytorch_state_metadata":
                setattr(self, key, modelopt_state[key])
        for key in ("_num_bits", "_axis", "_unsigned"):
            setattr(self._calibrator, key, getattr(self, key))
        if not properties_only:
            self._buffers.clear()
            self._non_persistent_buffers_set.clear()
            for k, v in modelopt_state.get("_pytorch_state_metadata", {}).get("buffers", {}).items():
                self.register_buffer(k, torch.empty(v["shape"], dtype=v.get("dtype")))

    def sync_amax_across_distributed_group(self, parallel_group=None):
        """Single-GPU build: nothing to synchronise."""
        return None

    @contextlib.contextmanager
    def disable_pre_quant_scale(self):
        was = self._enable_pre_quant_scale
        self._enable_pre_quant_scale = False
        try:
            yield
        finally:
            self._enable_pre_quant_scale = was

    def _set_buffer(self, key, value):
        if hasattr(self, key):
            setattr(self, key, value)
        else:
            self.register_buffer(key, value)


class SequentialQuantizer(nn.Sequential):
    """Applies several ``TensorQuantizer`` formats one after another (e.g. INT4 then FP8 for
    W4A8); ``fake_quant`` / ``is_enabled`` and the calibration methods fan out to all members."""

    _delegated_properties = ["fake_quant", "is_enabled"]
    _delegated_methods = ["reset_amax", "disable", "enable", "load_calib_amax", "load_calib_bias"]

    def __init__(self, *quantizers: TensorQuantizer):
        super().__init__(*quantizers)
        assert all(isinstance(q, TensorQuantizer) for q in self), "All quantizers must be a TensorQuantizer."

    def __getattr__(self, name):
        if name in self._delegated_properties:
            return getattr(self[0], name)
        if name in self._delegated_methods:
            def fan_out(*args, **kwargs):
                out = None
                for q in self:
                    out = getattr(q, name)(*args, **kwargs)
                return out
            return fan_out
        return super().__getattr__(name)

    def __setattr__(self, name, value):
        if name in self._delegated_properties:
            for q in self:
                setattr(q, name, value)
        else:
            super().__setattr__(name, value)

    def get_modelopt_state(self) -> dict[str, Any]:
        return {"num_quantizers": len(self), "is_sequential_quantizer": True}

    def set_from_attribute_config(self, attributes):
        if not isinstance(attributes, (list, tuple)):
            assert isinstance(attributes, (dict, QuantizerAttributeConfig)), "attributes must be a list or a dict."
            attributes = [attributes] * len(self)
        for attribute, q in zip(attributes, self):
            q.set_from_attribute_config(attribute)

    @staticmethod
    @contextlib.contextmanager
    def convert_to_single_quantizer(model, indx: int = 0):
        """Temporarily replace every ``SequentialQuantizer`` by its ``indx``-th member."""
        saved = []
        for name, module in list(model.named_modules()):
            if isinstance(module, SequentialQuantizer):
                assert len(module) > indx
                parent_name, _, leaf = name.rpartition(".")
                parent = model.get_submodule(parent_name)
                saved.append((parent, leaf, module))
                setattr(parent, leaf, module[indx])
        yield
        for parent, leaf, module in saved:
            setattr(parent, leaf, module)
