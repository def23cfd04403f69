"""What happens to a value beyond the E4M3 range (a scaled magnitude above 464, i.e. data above
the calibrated amax) in FP8 fake quantisation, and to an NVFP4 block scale above 448.

The reference has both behaviours and picks by where it runs.  Its CUDA kernel, which is what it
dispatches to for a device tensor with a per-tensor or per-axis amax (tensor_quant.py:62-90),
casts through ``__nv_fp8_e4m3`` and saturates at +-448 (src/tensor_quant_gpu_fp8.cu:36-47); its
eager path -- amax ``None``, an amax with more than one non-unit dim, or any CPU tensor -- casts
with ``Tensor.to(float8_e4m3fn)``, which gives NaN (tensor_quant.py:45-59).  NVFP4 block scales
in real quantisation are cast with the non-saturating conversion on every device
(qtensor/nvfp4_tensor.py:84-91).

``"auto"`` (default) follows that dispatch, so a calibrated ``FP8_DEFAULT_CFG`` / ``FP8_KV_CFG``
model clamps an outlier like the reference does on a GPU.  ``"nan"`` is the CPU path everywhere
(what bit-for-bit comparisons against the CPU path use).  ``"saturate"`` clamps everywhere,
including NVFP4 block scales: since ``awq_clip`` shrinks the per-tensor amax of an NVFP4 weight
(model_calib.py:869-876), compress / export of such a model otherwise stores the NaN byte for
blocks above the clipped amax; with ``"saturate"`` it stores 448 and the packed model computes
what the fake-quantised one did.
"""

from ... import _hip

_MODES = ("auto", "nan", "saturate")
_mode = "auto"


def set_fp8_overflow_behavior(mode: str) -> str:
    """Select ``"auto"``, ``"nan"`` or ``"saturate"``; returns the previous mode."""
    global _mode
    if mode not in _MODES:
        raise ValueError(f"mode must be one of {_MODES}, got {mode!r}")
    previous, _mode = _mode, mode
    return previous


def get_fp8_overflow_behavior() -> str:
    return _mode


def fp8_saturates(amax) -> bool:
    """Whether FP8 fake quantisation with this ``amax`` clamps out-of-range values."""
    if _mode != "auto":
        return _mode == "saturate"
    return amax is not None and sum(1 for d in amax.shape if d != 1) <= 1


def nvfp4_quantize_flags() -> int:
    """Flag bits for the NVFP4 quantize + pack entry points."""
    return _hip.MO_FLAG_SATURATE_BLOCK_SCALE if _mode == "saturate" else 0
