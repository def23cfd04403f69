"""Quantised ``nn.Linear`` (reference: nn/modules/quant_linear.py:39-115)."""

import torch.nn.functional as F
from torch import nn

from ...config import QuantizerAttributeConfig
from .quant_module import QuantLinearConvBase, QuantModuleRegistry

__all__ = ["QuantLinear"]


@QuantModuleRegistry.register({nn.Linear: "nn.Linear"})
class _QuantLinear(QuantLinearConvBase):
    """``y = F.linear(input_quantizer(x), weight_quantizer(W), b)`` then ``output_quantizer``."""

    default_quant_desc_weight = QuantizerAttributeConfig(num_bits=8, axis=0)

    def forward(self, input, *args, **kwargs):
        input = self.input_quantizer(input)
        weight = self.weight_quantizer(self.weight)
        output = F.linear(input, weight, self.bias)
        return self.output_quantizer(output)


QuantLinear = _QuantLinear
