"""Quantised modules."""

from .modules.quant_linear import Linear, QuantLinear, RealQuantLinear
from .modules.quant_module import (QuantInputBase, QuantLinearConvBase, QuantModule,
                                   QuantModuleRegistry)
from .modules.tensor_quantizer import SequentialQuantizer, TensorQuantizer

__all__ = ["Linear", "QuantLinear", "RealQuantLinear", "QuantInputBase", "QuantLinearConvBase", "QuantModule",
           "QuantModuleRegistry", "SequentialQuantizer", "TensorQuantizer"]
