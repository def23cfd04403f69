"""Quantised module bases and the registry that maps ``nn`` classes to them.

Follows the structure of the reference (nn/modules/quant_module.py:37-195): a quantised module
is the original module with ``input_quantizer`` / ``output_quantizer`` (and ``weight_quantizer``)
children; ``weight`` is fake-quantised on every forward.  Conversion swaps the instance's class
in place (no copy of parameters), which stands in for the reference's ``DynamicModule``
machinery.
"""

import contextlib

import torch
from torch import nn

from ...config import QuantizerAttributeConfig
from .tensor_quantizer import SequentialQuantizer, TensorQuantizer

__all__ = ["QuantModule", "QuantInputBase", "QuantLinearConvBase", "QuantModuleRegistry"]


class _Registry:
    """original class -> quantised class (reference: ``QuantModuleRegistry``)."""

    def __init__(self):
        self._map: dict[type, type] = {}
        self._derived: dict[tuple[type, type], type] = {}   # (quantised base, original class) -> class

    def register(self, mapping: dict[type, str]):
        def deco(qcls):
            for orig in mapping:
                self._map[orig] = qcls
            return qcls
        return deco

    def unregister(self, orig):
        self._map.pop(orig, None)
        for key in [k for k in self._derived if k[1] is orig]:
            del self._derived[key]

    def get(self, orig):
        return self._map.get(orig)

    def __contains__(self, orig):
        return orig in self._map

    def convert(self, module: nn.Module):
        """Swap ``module`` to its quantised class in place and create its quantizers."""
        qcls = self._map[type(module)]
        if type(module) is not qcls:
            orig = type(module)
            object.__setattr__(module, "_original_cls", orig)
            derived = self._derived.get((qcls, orig))
            if derived is None:   # one class per pair, not one per converted instance
                derived = self._derived[(qcls, orig)] = type(f"Quant{orig.__name__}", (qcls, orig), {})
            module.__class__ = derived
        module._setup()
        return module


QuantModuleRegistry = _Registry()


class QuantModule(nn.Module):
    """Base of all quantised modules."""

    def _setup(self):
        raise NotImplementedError

    def modelopt_post_restore(self, prefix: str = ""):
        """Move quantizer buffers next to the module's own tensors after a restore."""
        ref = next(iter(self.parameters()), None)
        if ref is None:
            return
        for m in self.modules():
            if isinstance(m, TensorQuantizer):
                m.to(ref.device)

    def fold_weight(self):
        """Replace each weight by its fake-quantised value and disable its quantizer."""
        for name in ("weight",):
            q = getattr(self, "weight_quantizer", None)
            if q is None or not isinstance(q, TensorQuantizer) or not q.fake_quant:
                continue
            w = getattr(self, name)
            w.data.copy_(q(w.float()).to(w.dtype))
            q.disable()
            for attr in ("_pre_quant_scale", "_amax"):
                if hasattr(q, attr):
                    delattr(q, attr)


class QuantInputBase(QuantModule):
    """Quantises the input and (optionally) the output of the wrapped forward."""

    default_quant_desc_input = QuantizerAttributeConfig(num_bits=8)
    default_quant_desc_output = QuantizerAttributeConfig(num_bits=8)

    def forward(self, input, *args, **kwargs):
        input = self.input_quantizer(input)
        output = super().forward(input, *args, **kwargs)
        if isinstance(output, tuple):
            return (self.output_quantizer(output[0]), *output[1:])
        return self.output_quantizer(output)

    def _setup(self):
        # plain insertion: the names are fixed and the values are modules (add_module's checks
        # cost as much as building the quantizer)
        self._modules["input_quantizer"] = TensorQuantizer(self.default_quant_desc_input)
        out = self._modules["output_quantizer"] = TensorQuantizer(self.default_quant_desc_output)
        out.disable()


class QuantLinearConvBase(QuantInputBase):
    """Adds the weight quantizer; ``self.weight`` read inside ``forward`` is fake-quantised."""

    default_quant_desc_weight = QuantizerAttributeConfig(num_bits=8, axis=0)

    @contextlib.contextmanager
    def quantize_weight(self):
        self._enable_weight_quantization = True
        try:
            yield
        finally:
            self._enable_weight_quantization = False

    def _quantized_weight(self):
        w = self._parameters["weight"]
        if getattr(self, "_enable_weight_quantization", False):
            return self.weight_quantizer(w)
        return w

    def forward(self, input, *args, **kwargs):
        with self.quantize_weight():
            return super().forward(input, *args, **kwargs)

    def _setup(self):
        super()._setup()
        self._modules["weight_quantizer"] = TensorQuantizer(self.default_quant_desc_weight)
        object.__setattr__(self, "_enable_weight_quantization", False)
