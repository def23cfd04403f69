"""Quantised ``nn.Linear`` (reference: nn/modules/quant_linear.py:39-115)."""

import torch.nn.functional as F
from torch import nn

from ...config import QuantizerAttributeConfig
from ...qtensor.base_qtensor import QTensorWrapper
from .quant_module import QuantLinearConvBase, QuantModule, QuantModuleRegistry

__all__ = ["Linear", "QuantLinear", "RealQuantLinear"]


@QuantModuleRegistry.register({nn.Linear: "nn.Linear"})
class _QuantLinear(QuantLinearConvBase):
    """``y = F.linear(input_quantizer(x), weight_quantizer(W), b)`` then ``output_quantizer``."""

    default_quant_desc_weight = QuantizerAttributeConfig(num_bits=8, axis=0)

    def forward(self, input, *args, **kwargs):
        input = self.input_quantizer(input)
        weight = self.weight_quantizer(self.weight)
        output = F.linear(input, weight, self.bias)
        return self.output_quantizer(output)


class QuantLinear(_QuantLinear, nn.Linear):
    """``nn.Linear`` that is born quantised: ``QuantLinear(in_features, out_features)`` builds the
    linear layer and attaches its quantizers (reference: nn/modules/quant_linear.py:56-62 with
    the constructor of nn/modules/quant_module.py:172-196).  ``quant_desc_input`` /
    ``quant_desc_weight`` override the default quantizer configurations of this instance."""

    def __init__(self, *args, quant_desc_input=None, quant_desc_weight=None, **kwargs):
        nn.Linear.__init__(self, *args, **kwargs)
        if quant_desc_input is not None:
            self.default_quant_desc_input = quant_desc_input
        if quant_desc_weight is not None:
            self.default_quant_desc_weight = quant_desc_weight
        self._original_cls = nn.Linear
        self._setup()


Linear = QuantLinear


class RealQuantLinear(QuantModule):
    """Quantised linear whose weight is stored packed (reference: nn/modules/quant_linear.py
    :191-312).  ``forward`` is the fake-quant module's: the weight quantizer dequantises the
    ``QTensorWrapper`` on the fly (no real-quant GEMM backend is part of this build).  A
    high-precision weight assigned later (``module.weight = nn.Parameter(...)``, a checkpoint
    loader writing ``_parameters["weight"]``) is packed on assignment."""

    list_of_scale_tensors = ["_scale", "double_scale", "_scale_zeros"]
    allow_real_quant_gemm = False

    def forward(self, input, *args, **kwargs):
        return super().forward(input, *args, **kwargs)

    def _setup(self):
        class RealQuantParameterDict(dict):
            def __init__(self, weight_quantizer, *args, **kwargs):
                super().__init__(*args, **kwargs)
                self.weight_quantizer = weight_quantizer

            def __setitem__(self, key, value):
                q = self.weight_quantizer
                if (key == "weight" and q is not None and value is not None and q.is_enabled
                        and not q._fake_quant and not isinstance(value, QTensorWrapper)
                        and value.element_size() > 1):
                    q._dequantize = False       # a fresh weight: quantise, do not dequantise
                    value = QTensorWrapper(q(value))
                super().__setitem__(key, value)

        self._parameters = RealQuantParameterDict(self.weight_quantizer, self._parameters)

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        """Packed weights are copied as they are; everything else takes the stock path."""
        held = {}
        for name, param in self.named_parameters(recurse=False):
            key = prefix + name
            if key in state_dict and isinstance(param, QTensorWrapper):
                param.data.copy_(state_dict[key])
                held[key] = state_dict.pop(key)
        args = list(args)
        if len(args) > 1:
            args[1] = False                      # strict: the weight keys were taken out above
        super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)
        state_dict.update(held)
