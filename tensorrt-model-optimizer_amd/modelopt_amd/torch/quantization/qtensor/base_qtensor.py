"""Containers for real-quantised tensors (reference: qtensor/base_qtensor.py:39-137)."""

import torch

__all__ = ["BaseQuantizedTensor", "QTensorWrapper", "pack_real_quantize_weight"]


class BaseQuantizedTensor:
    """Packed data plus the shape and dtype of the tensor it was made from."""

    def __init__(self, original_shape, original_dtype, quantized_data: torch.Tensor):
        self.metadata = {"shape": original_shape, "dtype": original_dtype}
        self._quantized_data = quantized_data

    @classmethod
    def quantize(cls, input: torch.Tensor, block_size: int):
        raise NotImplementedError

    def dequantize(self, dtype: torch.dtype = None, **kwarg):
        raise NotImplementedError


class QTensorWrapper(torch.nn.Parameter):
    """``nn.Parameter`` that owns packed storage and remembers which QTensor class made it."""

    def __new__(cls, qtensor, metadata: dict | None = None):
        data = qtensor._quantized_data if isinstance(qtensor, BaseQuantizedTensor) else qtensor
        inst = super().__new__(cls, data, requires_grad=False)
        if metadata is None:
            inst.metadata = qtensor.metadata
            inst.metadata["qtensor_class"] = qtensor.__class__
        else:
            assert all(k in metadata for k in ("qtensor_class", "shape", "dtype")), f"metadata: {metadata}"
            inst.metadata = metadata
        return inst

    def dim(self):
        return len(self.metadata["shape"])

    def to(self, *args, **kwargs):
        device, dtype, *_ = torch._C._nn._parse_to(*args, **kwargs)
        if device:
            self.data = self.data.to(device=device)
        dtype = dtype if dtype else self.metadata["dtype"]
        return QTensorWrapper(self.metadata["qtensor_class"](self.metadata["shape"], dtype, self.data))

    def get_qtensor(self):
        return self.metadata["qtensor_class"](self.metadata["shape"], self.metadata["dtype"], self.data)

    def get_state(self):
        return {"metadata": self.metadata, "quantized_data.shape": self.data.shape,
                "quantized_data.dtype": self.data.dtype}


def pack_real_quantize_weight(module, force_quantize: bool = False):
    """Replace the weight of every sub-module whose weight quantizer is enabled and set to real
    quantisation by its packed form (a ``QTensorWrapper``).  Reference: qtensor/base_qtensor.py
    :196-229."""
    from ..nn import SequentialQuantizer  # circular at import time

    def compress(m):
        w = getattr(m, "weight", None)
        q = getattr(m, "weight_quantizer", None)
        if w is None or w.is_meta or q is None:
            return False
        if q.is_enabled and not q._fake_quant and w.element_size() > 1:
            if force_quantize:
                q._dequantize = False
            m.weight = QTensorWrapper(q(w))
            return True
        return False

    with SequentialQuantizer.convert_to_single_quantizer(module), torch.no_grad():
        for name, m in module.named_modules():
            if name != "":
                compress(m)
