"""Quantization configuration: ``QuantizerAttributeConfig``, ``QuantizeConfig`` and the named
format configs.

Field names, defaults, validation rules and the contents of the named configs follow the
reference (modelopt/torch/quantization/config.py:146-440, 661-955, 958-1190) so that a config
written for it is accepted unchanged.
"""

import weakref
from typing import Any, Literal

from pydantic import BaseModel, ConfigDict, ValidationInfo, field_validator, model_validator

__all__ = [
    "QuantizerAttributeConfig", "QuantizeConfig", "CompressConfig", "MaxCalibConfig", "MseCalibConfig", "SmoothQuantCalibConfig",
    "AWQLiteCalibConfig", "INT8_DEFAULT_CFG", "INT8_SMOOTHQUANT_CFG", "INT8_WEIGHT_ONLY_CFG",
    "FP8_DEFAULT_CFG", "INT4_BLOCKWISE_WEIGHT_ONLY_CFG", "INT4_AWQ_CFG", "W4A8_AWQ_BETA_CFG",
    "FP8_KV_CFG", "NVFP4_DEFAULT_CFG", "NVFP4_AWQ_LITE_CFG", "NVFP4_KV_CFG", "MXFP8_DEFAULT_CFG",
    "MXFP6_DEFAULT_CFG", "MXFP4_DEFAULT_CFG", "MXINT8_DEFAULT_CFG", "W4A8_MXFP4_FP8_CFG",
    "NVFP4_AWQ_CLIP_CFG", "NVFP4_AWQ_FULL_CFG", "FP8_PER_CHANNEL_PER_TOKEN_CFG",
    "FP8_2D_BLOCKWISE_WEIGHT_ONLY_CFG", "W4A8_NVFP4_FP8_CFG", "MXFP4_MLP_WEIGHT_ONLY_CFG",
    "NVFP4_MLP_WEIGHT_ONLY_CFG", "NVFP4_MLP_ONLY_CFG", "choices", "need_calibration",
]

_SPECIAL_BLOCK_KEYS = ("type", "scale_bits", "scale_block_sizes")
_FP_FORMATS = [(4, 3), (5, 2), (2, 1), (1, 2), (0, 3), (3, 0), (3, 2), (2, 3)]


class _MappingConfig(BaseModel):
    """pydantic model that also behaves like a read/write mapping over its fields."""

    model_config = ConfigDict(extra="forbid", validate_assignment=True, arbitrary_types_allowed=True)

    def __getitem__(self, key):
        if key not in type(self).model_fields:
            raise KeyError(key)
        return getattr(self, key)

    def __setitem__(self, key, value):
        setattr(self, key, value)

    def __contains__(self, key):
        return key in type(self).model_fields

    def __iter__(self):  # type: ignore[override]
        return iter(type(self).model_fields)

    def __len__(self):
        return len(type(self).model_fields)

    def keys(self):
        return type(self).model_fields.keys()

    def values(self):
        return [getattr(self, k) for k in self.keys()]

    def items(self):
        return [(k, getattr(self, k)) for k in self.keys()]

    def get(self, key, default=None):
        return getattr(self, key) if key in self else default


_QUANTIZER_ATTRIBUTES: dict = {}   # id(config) -> (weak reference to it, its quantizer_attributes())


class QuantizerAttributeConfig(_MappingConfig):
    """Attributes of one ``TensorQuantizer`` (reference: config.py:661-955)."""

    enable: bool = True
    num_bits: int | tuple[int, int] = 8
    axis: int | tuple[int, ...] | None = None
    fake_quant: bool = True
    unsigned: bool = False
    narrow_range: bool = False
    learn_amax: bool = False
    type: str = "static"
    block_sizes: dict[int | str, int | tuple[int, int] | str | dict[int, int] | None] | None = None
    bias: dict[int | str, Any] | None = None
    trt_high_precision_dtype: str = "Float"
    calibrator: Any = "max"
    rotate: bool = False
    pass_through_bwd: bool = False

    def __setattr__(self, name, value):
        super().__setattr__(name, value)
        _QUANTIZER_ATTRIBUTES.pop(id(self), None)   # a field changed

    def quantizer_attributes(self):
        """``({"_num_bits": ..., "_disabled": ..., "_dynamic": ...}, calibrator spec)``: the
        attribute names and values a ``TensorQuantizer`` takes from this config (``enable`` ->
        ``_disabled``, ``type`` -> ``_dynamic``, every other field ``_<field>``).  Kept until a
        field is assigned: a model conversion configures hundreds of quantizers from a handful
        of config objects."""
        entry = _QUANTIZER_ATTRIBUTES.get(id(self))
        if entry is not None and entry[0]() is self:
            return entry[1]
        plain = {}
        for name in type(self).model_fields:
            val = getattr(self, name)
            if name == "enable":
                plain["_disabled"] = val is False
            elif name == "type":
                plain["_dynamic"] = val == "dynamic"
            elif name != "calibrator":
                plain[f"_{name}"] = val
        made = (plain, self.calibrator)
        key = id(self)
        _QUANTIZER_ATTRIBUTES[key] = (weakref.ref(self, lambda _, key=key: _QUANTIZER_ATTRIBUTES.pop(key, None)),
                                      made)
        return made

    @model_validator(mode="before")
    @classmethod
    def _reject_bare_enable(cls, values):
        def walk(v):
            if isinstance(v, list):
                for item in v:
                    walk(item)
            elif isinstance(v, dict):
                if len(v) == 1 and v.get("enable") is True:
                    raise ValueError(
                        "Invalid quantizer config: Cannot specify only {'enable': True}. "
                        "Additional parameters are required when enabling quantization.")
                for item in v.values():
                    walk(item)

        walk(values)
        return values

    @field_validator("type")
    @classmethod
    def _check_type(cls, v):
        if v not in ("static", "dynamic"):
            raise ValueError("type must be 'static' or 'dynamic'")
        return v

    @field_validator("learn_amax")
    @classmethod
    def _check_learn_amax(cls, v):
        assert v is not True, "learn_amax is deprecated and reserved for backward compatibility."
        return v

    @staticmethod
    def _get_block_quant_axes_and_sizes(block_sizes):
        if block_sizes is None:
            return None
        return {k: v for k, v in block_sizes.items() if k not in _SPECIAL_BLOCK_KEYS}

    @field_validator("block_sizes")
    @classmethod
    def _check_block_sizes(cls, v, info: ValidationInfo):
        if v is None:
            return v
        assert info.data.get("axis") is None, "axis must be None when block_sizes is not None."
        if v.get("type") == "dynamic":
            assert len(cls._get_block_quant_axes_and_sizes(v)) == 1, (
                "Dynamic block quantization only supports quantization last axis.")
        for k, val in v.items():
            if isinstance(k, str):
                assert k in _SPECIAL_BLOCK_KEYS, f"unknown block_sizes key {k!r}"
            else:
                assert isinstance(k, int) and (val is None or isinstance(val, int))
        return v

    @field_validator("bias")
    @classmethod
    def _check_bias(cls, v):
        if v is None:
            return v
        if "type" in v and v["type"] not in ("static", "dynamic"):
            raise ValueError(f"Invalid bias type: {v['type']}, expected 'static' or 'dynamic'")
        if "method" in v and v["method"] not in ("mean", "max_min"):
            raise ValueError(f"Invalid bias method: {v['method']}, expected 'mean' or 'max_min'")
        axes = [k for k in v if k not in ("type", "method")]
        assert len(axes) > 0, "The axis for bias computation is not specified."
        for a in axes:
            if not isinstance(a, int):
                raise ValueError(f"Invalid axis type {type(a)}, expected int")
        return v

    @model_validator(mode="after")
    def _check_num_bits(self):
        nb = self.num_bits
        if isinstance(nb, int):
            if nb < 1:
                raise ValueError("num_bits must be a positive integer or a tuple of positive integers.")
            return self
        if not all(x > 0 for x in nb):
            raise ValueError("num_bits must be a positive integer or a tuple of positive integers.")
        if nb not in _FP_FORMATS:
            raise ValueError(
                "Supported FPx quantization formats: FP8 (E4M3, E5M2), FP6(E3M2, E2M3), FP4(E2M1).")
        if nb != (4, 3) and (self.block_sizes is None or self.block_sizes.get("type") != "dynamic"):
            raise ValueError("Only blockwise dynamic quantization is supported with this format.")
        return self


class MaxCalibConfig(_MappingConfig):
    method: Literal["max"] = "max"
    distributed_sync: bool | None = True


class SmoothQuantCalibConfig(_MappingConfig):
    method: Literal["smoothquant"] = "smoothquant"
    alpha: float | None = 1.0


class AWQLiteCalibConfig(_MappingConfig):
    method: Literal["awq_lite"] = "awq_lite"
    alpha_step: float | None = 0.1
    debug: bool | None = False


class AWQClipCalibConfig(_MappingConfig):
    """Reference: config.py:1069-1115."""

    method: Literal["awq_clip"] = "awq_clip"
    max_co_batch_size: int | None = 1024
    max_tokens_per_batch: int | None = 64
    min_clip_ratio: float | None = 0.5
    shrink_step: float | None = 0.05
    debug: bool | None = False


class AWQFullCalibConfig(_MappingConfig):
    """awq_lite followed by awq_clip (reference: config.py:1118-1135)."""

    method: Literal["awq_full"] = "awq_full"
    alpha_step: float | None = 0.1
    max_co_batch_size: int | None = 1024
    max_tokens_per_batch: int | None = 64
    min_clip_ratio: float | None = 0.5
    shrink_step: float | None = 0.05
    debug: bool | None = False


class MseCalibConfig(_MappingConfig):
    """amax search minimising the quantisation error (reference: config.py:984-1020)."""

    method: Literal["mse"] = "mse"
    num_steps: int | None = 10
    start_multiplier: float | None = 0.25
    stop_multiplier: float | None = 4.0
    distributed_sync: bool | None = True


_ALGO_CONFIGS = {"max": MaxCalibConfig, "smoothquant": SmoothQuantCalibConfig,
                 "awq_lite": AWQLiteCalibConfig, "mse": MseCalibConfig,
                 "awq_clip": AWQClipCalibConfig, "awq_full": AWQFullCalibConfig}


def normalize_algorithm(algorithm):
    """``None`` | name | dict -> (method name or None, keyword arguments).

    Accepts what the reference's ``QuantizeConfig.algorithm`` accepts for the methods built here
    (config.py:958-1150); other methods raise ``NotImplementedError``.
    """
    if algorithm is None:
        return None, {}
    if isinstance(algorithm, str):
        algorithm = {"method": algorithm}
    if isinstance(algorithm, _MappingConfig):
        algorithm = dict(algorithm.items())
    method = algorithm.get("method")
    if method is None:
        return None, {}
    if method not in _ALGO_CONFIGS:
        raise NotImplementedError(
            f"calibration algorithm {method!r} is outside the hot path built here "
            f"(supported: {sorted(_ALGO_CONFIGS)})")
    cfg = _ALGO_CONFIGS[method](**algorithm)
    kwargs = {k: v for k, v in cfg.items() if k != "method"}
    return method, kwargs


class QuantizeConfig(_MappingConfig):
    """``{"quant_cfg": {wildcard: attributes}, "algorithm": ...}`` (reference: config.py:1165)."""

    quant_cfg: dict[str, Any] = {"default": {"num_bits": 8, "axis": None}}
    algorithm: Any = "max"


class CompressConfig(_MappingConfig):
    """``compress``: pattern -> compress or not; ``quant_gemm`` is accepted for compatibility
    (no real-quant GEMM backend exists here).  Reference: config.py:1182-1195."""

    compress: dict[str, bool] = {"*": True}
    quant_gemm: bool = True


_default_disabled_quantizer_cfg = {
    "nn.BatchNorm1d": {"*": {"enable": False}},
    "nn.BatchNorm2d": {"*": {"enable": False}},
    "nn.BatchNorm3d": {"*": {"enable": False}},
    "nn.LeakyReLU": {"*": {"enable": False}},
    "*lm_head*": {"enable": False},
    "*proj_out.*": {"enable": False},
    "*block_sparse_moe.gate*": {"enable": False},
    "*router*": {"enable": False},
    "*mlp.gate.*": {"enable": False},
    "*mlp.shared_expert_gate.*": {"enable": False},
    "*linear_attn.conv1d*": {"enable": False},
    "*mixer.conv1d*": {"enable": False},
    "*output_layer*": {"enable": False},
    "output.*": {"enable": False},
    "default": {"enable": False},
}

_NVFP4 = {"num_bits": (2, 1), "block_sizes": {-1: 16, "type": "dynamic", "scale_bits": (4, 3)},
          "axis": None, "enable": True}

INT8_DEFAULT_CFG = {
    "quant_cfg": {"*weight_quantizer": {"num_bits": 8, "axis": 0},
                  "*input_quantizer": {"num_bits": 8, "axis": None},
                  **_default_disabled_quantizer_cfg},
    "algorithm": "max",
}
INT8_SMOOTHQUANT_CFG = {
    "quant_cfg": {"*weight_quantizer": {"num_bits": 8, "axis": 0},
                  "*input_quantizer": {"num_bits": 8, "axis": None},
                  **_default_disabled_quantizer_cfg},
    "algorithm": "smoothquant",
}
INT8_WEIGHT_ONLY_CFG = {
    "quant_cfg": {"*weight_quantizer": {"num_bits": 8, "axis": 0},
                  "*input_quantizer": {"enable": False},
                  **_default_disabled_quantizer_cfg},
    "algorithm": "max",
}
FP8_DEFAULT_CFG = {
    "quant_cfg": {"*weight_quantizer": {"num_bits": (4, 3), "axis": None},
                  "*input_quantizer": {"num_bits": (4, 3), "axis": None},
                  **_default_disabled_quantizer_cfg},
    "algorithm": "max",
}
INT4_BLOCKWISE_WEIGHT_ONLY_CFG = {
    "quant_cfg": {"*weight_quantizer": {"num_bits": 4, "block_sizes": {-1: 128}, "enable": True},
                  "*input_quantizer": {"enable": False},
                  **_default_disabled_quantizer_cfg},
    "algorithm": "max",
}
INT4_AWQ_CFG = {
    "quant_cfg": {"*weight_quantizer": {"num_bits": 4,
                                        "block_sizes": {-1: 128, "type": "static"},
                                        "enable": True},
                  "*input_quantizer": {"enable": False},
                  **_default_disabled_quantizer_cfg},
    "algorithm": {"method": "awq_lite", "alpha_step": 0.1},
}
W4A8_AWQ_BETA_CFG = {
    "quant_cfg": {"*weight_quantizer": [
                      {"num_bits": 4, "block_sizes": {-1: 128, "type": "static"}, "enable": True},
                      {"num_bits": (4, 3), "axis": None, "enable": True}],
                  "*input_quantizer": {"num_bits": (4, 3), "axis": None, "enable": True},
                  **_default_disabled_quantizer_cfg},
    "algorithm": "awq_lite",
}
FP8_KV_CFG = {
    "quant_cfg": {"*[kv]_bmm_quantizer": {"num_bits": (4, 3), "axis": None, "enable": True},
                  "default": {"enable": False}},
    "algorithm": "max",
}
NVFP4_KV_CFG = {
    "quant_cfg": {"*[kv]_bmm_quantizer": dict(_NVFP4), "default": {"enable": False}},
    "algorithm": "max",
}
NVFP4_DEFAULT_CFG = {
    "quant_cfg": {"*weight_quantizer": dict(_NVFP4), "*input_quantizer": dict(_NVFP4),
                  **_default_disabled_quantizer_cfg},
    "algorithm": "max",
}
NVFP4_AWQ_LITE_CFG = {
    "quant_cfg": {"*weight_quantizer": dict(_NVFP4), "*input_quantizer": dict(_NVFP4),
                  **_default_disabled_quantizer_cfg},
    "algorithm": "awq_lite",
}
# reference: config.py:410-447
NVFP4_AWQ_CLIP_CFG = {
    "quant_cfg": {"*weight_quantizer": dict(_NVFP4), "*input_quantizer": dict(_NVFP4),
                  **_default_disabled_quantizer_cfg},
    "algorithm": {"method": "awq_clip"},
}
NVFP4_AWQ_FULL_CFG = {
    "quant_cfg": {"*weight_quantizer": dict(_NVFP4), "*input_quantizer": dict(_NVFP4),
                  **_default_disabled_quantizer_cfg},
    "algorithm": {"method": "awq_full", "alpha_step": 0.1},
}
# reference: config.py:201-212 -- per-channel weights, per-token dynamic activations
FP8_PER_CHANNEL_PER_TOKEN_CFG = {
    "quant_cfg": {"*weight_quantizer": {"num_bits": (4, 3), "axis": 0},
                  "*input_quantizer": {"num_bits": (4, 3), "type": "dynamic",
                                       "block_sizes": {-1: None}},
                  **_default_disabled_quantizer_cfg},
    "algorithm": "max",
}
# reference: config.py:215-226 -- 128 x 128 weight tiles (DeepSeek style)
FP8_2D_BLOCKWISE_WEIGHT_ONLY_CFG = {
    "quant_cfg": {"*weight_quantizer": {"num_bits": (4, 3), "block_sizes": {-1: 128, -2: 128},
                                        "enable": True},
                  "*input_quantizer": {"enable": False},
                  **_default_disabled_quantizer_cfg},
    "algorithm": "max",
}
# reference: config.py:559-575 -- NVFP4 weights in 32-element blocks, FP8 per-tensor activations
W4A8_NVFP4_FP8_CFG = {
    "quant_cfg": {"*weight_quantizer": {"num_bits": (2, 1),
                                        "block_sizes": {-1: 32, "type": "dynamic",
                                                        "scale_bits": (4, 3)},
                                        "axis": None, "enable": True},
                  "*input_quantizer": {"num_bits": (4, 3), "axis": None, "enable": True},
                  **_default_disabled_quantizer_cfg},
    "algorithm": "max",
}
# reference: config.py:577-620 -- MLP layers only
MXFP4_MLP_WEIGHT_ONLY_CFG = {
    "quant_cfg": {"*mlp*weight_quantizer": {"num_bits": (2, 1),
                                            "block_sizes": {-1: 32, "type": "dynamic",
                                                            "scale_bits": (8, 0)},
                                            "enable": True, "pass_through_bwd": True},
                  **_default_disabled_quantizer_cfg},
    "algorithm": None,
}
NVFP4_MLP_WEIGHT_ONLY_CFG = {
    "quant_cfg": {"*mlp*weight_quantizer": {"num_bits": (2, 1),
                                            "block_sizes": {-1: 32, "type": "dynamic",
                                                            "scale_bits": (4, 3)},
                                            "enable": True, "pass_through_bwd": True},
                  **_default_disabled_quantizer_cfg},
    "algorithm": "max",
}
NVFP4_MLP_ONLY_CFG = {
    "quant_cfg": {"*mlp*weight_quantizer": {**_NVFP4, "pass_through_bwd": True},
                  "*mlp*input_quantizer": {**_NVFP4, "pass_through_bwd": True},
                  **_default_disabled_quantizer_cfg},
    "algorithm": "max",
}



def _mx_cfg(num_bits):
    q = {"num_bits": num_bits, "block_sizes": {-1: 32, "type": "dynamic", "scale_bits": (8, 0)},
         "enable": True}
    return {"quant_cfg": {"*weight_quantizer": dict(q), "*input_quantizer": dict(q),
                          **_default_disabled_quantizer_cfg},
            "algorithm": None}


# reference: config.py:266-345 -- 32-element blocks, shared power-of-two scale, no calibration
MXFP8_DEFAULT_CFG = _mx_cfg((4, 3))
MXFP6_DEFAULT_CFG = _mx_cfg((3, 2))
MXFP4_DEFAULT_CFG = _mx_cfg((2, 1))
MXINT8_DEFAULT_CFG = _mx_cfg(8)
W4A8_MXFP4_FP8_CFG = {
    "quant_cfg": {"*weight_quantizer": dict(_mx_cfg((2, 1))["quant_cfg"]["*weight_quantizer"]),
                  "*input_quantizer": {"num_bits": (4, 3), "axis": None},
                  **_default_disabled_quantizer_cfg},
    "algorithm": None,
}

choices = {
    "MXFP8_DEFAULT_CFG", "MXFP6_DEFAULT_CFG", "MXFP4_DEFAULT_CFG", "MXINT8_DEFAULT_CFG",
    "W4A8_MXFP4_FP8_CFG",
    "INT8_DEFAULT_CFG", "INT8_SMOOTHQUANT_CFG", "INT8_WEIGHT_ONLY_CFG", "FP8_DEFAULT_CFG",
    "INT4_BLOCKWISE_WEIGHT_ONLY_CFG", "INT4_AWQ_CFG", "W4A8_AWQ_BETA_CFG", "NVFP4_DEFAULT_CFG",
    "NVFP4_AWQ_LITE_CFG", "NVFP4_AWQ_CLIP_CFG", "NVFP4_AWQ_FULL_CFG", "FP8_PER_CHANNEL_PER_TOKEN_CFG",
    "FP8_2D_BLOCKWISE_WEIGHT_ONLY_CFG", "W4A8_NVFP4_FP8_CFG", "MXFP4_MLP_WEIGHT_ONLY_CFG",
    "NVFP4_MLP_WEIGHT_ONLY_CFG", "NVFP4_MLP_ONLY_CFG", "FP8_KV_CFG", "NVFP4_KV_CFG",
}


def need_calibration(config) -> bool:
    """Whether ``mtq.quantize`` needs a forward loop for ``config`` (reference: config.py:1205-1231):
    any algorithm other than plain max does; otherwise it is needed as soon as one enabled
    quantizer that is not a weight quantizer is static (``type`` other than ``"dynamic"`` at the top
    level of its entry; weights are calibrated from the weights themselves)."""
    if config["algorithm"] not in (None, "max"):
        return True

    def static_and_enabled(entry):
        return (entry.get("enable", True) and entry.get("type", "") != "dynamic"
                and entry.get("*", {}).get("enable", True))

    for pattern, entry in config.get("quant_cfg", {}).items():
        if "weight_quantizer" in pattern:
            continue
        entries = entry if isinstance(entry, list) else [entry]
        if any(static_and_enabled(e) for e in entries):
            return True
    return False
