"""Quantised modules."""

from .modules.quant_linear import QuantLinear
from .modules.quant_module import (QuantInputBase, QuantLinearConvBase, QuantModule,
                                   QuantModuleRegistry)
from .modules.tensor_quantizer import SequentialQuantizer, TensorQuantizer

__all__ = ["QuantLinear", "QuantInputBase", "QuantLinearConvBase", "QuantModule",
           "QuantModuleRegistry", "SequentialQuantizer", "TensorQuantizer"]
