"""Real-quantised tensor containers."""

from .base_qtensor import BaseQuantizedTensor, QTensorWrapper, pack_real_quantize_weight
from .fp8_tensor import FP8QTensor
from .int4_tensor import INT4QTensor
from .int8_tensor import INT8QTensor
from .mxfp4_tensor import MXFP4QTensor
from .nf4_tensor import NF4QTensor
from .nvfp4_tensor import NVFP4QTensor

__all__ = ["BaseQuantizedTensor", "QTensorWrapper", "pack_real_quantize_weight", "FP8QTensor",
           "INT4QTensor", "INT8QTensor", "MXFP4QTensor", "NF4QTensor", "NVFP4QTensor"]
