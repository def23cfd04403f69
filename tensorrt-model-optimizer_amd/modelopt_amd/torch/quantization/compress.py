"""``mtq.compress``: store the weights of a quantised model in their packed format.

Reference: compress.py:52-227.  Every quantised linear becomes a ``RealQuantLinear``; the weight
quantizers selected by the pattern config are switched from fake to real quantisation and their
weights are packed once (NVFP4 / INT4 block / FP8 / INT8 kernels); forwards dequantise on the fly.
"""

import fnmatch
import warnings

from torch import nn

from .config import CompressConfig
from .conversion import set_quantizer_attribute
from .nn.modules.quant_linear import RealQuantLinear
from .qtensor import QTensorWrapper, pack_real_quantize_weight
from .utils import is_quantized_linear

__all__ = ["compress", "is_real_quantized"]


def _to_real_quant(module: nn.Module):
    """Class swap in place: ``RealQuantLinear`` in front of the module's current (quantised)
    class, so its forward still runs the quantizers of the module."""
    cls = type(module)
    if not issubclass(cls, RealQuantLinear):
        module.__class__ = type(f"RealQuant{getattr(module, '_original_cls', cls).__name__}",
                                (RealQuantLinear, cls), {})
        RealQuantLinear._setup(module)


def compress(model: nn.Module, config=None):
    """Compress the weights of a quantised model in place.

    ``config``: ``{pattern: bool}`` (or a ``CompressConfig``) -- ``"default"`` first, then the
    patterns in order, later entries winning; ``None`` compresses every supported layer.
    """
    if config is None:
        config = CompressConfig()
    elif isinstance(config, dict):
        patterns = config["compress"] if "compress" in config else config
        for to_compress in patterns.values():   # before pydantic coerces "yes" / 1 to True
            if not isinstance(to_compress, bool):
                raise ValueError(f"Invalid compression configuration: {to_compress}, expected a boolean as value.")
        config = CompressConfig(**config) if "compress" in config else CompressConfig(compress=config)
    for module in model.modules():
        if is_quantized_linear(module):
            _to_real_quant(module)
    cfg = config.compress
    if "default" in cfg and isinstance(cfg["default"], bool):
        set_quantizer_attribute(model, "*weight_quantizer*", {"fake_quant": not cfg["default"]})
    for pattern, to_compress in cfg.items():
        if pattern == "default":
            continue
        if not isinstance(to_compress, bool):
            raise ValueError(f"Invalid compression configuration: {to_compress}, expected a boolean as value.")
        set_quantizer_attribute(
            model, lambda name, p=pattern: fnmatch.fnmatch(name, p) and "weight_quantizer" in name,
            {"fake_quant": not to_compress})
    pack_real_quantize_weight(model)
    if any(isinstance(getattr(m, "weight", None), QTensorWrapper) for m in model.modules()):
        warnings.warn("Real quantization has been applied to the model. This feature is still "
                      "experimental, and some functionalities may not be supported.")
    return model


def is_real_quantized(model: nn.Module) -> bool:
    return any(isinstance(m, RealQuantLinear) for m in model.modules())
