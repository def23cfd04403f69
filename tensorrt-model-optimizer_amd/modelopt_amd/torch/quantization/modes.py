"""Process-wide switches of the Python layer that have no counterpart in the reference.

``set_one_launch_dynamic_quant`` -- dynamic per-tensor fake quantisation and ``NVFP4QTensor.quantize``
without given scales can run as ONE launch that reads the tensor once (``mo_fused_amax_qdq``,
``mo_nvfp4_quantize_fused``).  Those kernels want all their workgroups on the device at the same
time; when that cannot be had (another stream's kernel holds the compute units, a masked device)
they still return the right bits, but only after a bounded wait.  Off by default: the two-launch
path has no such dependence on what else the device is doing.

``set_strict_checks`` -- the reference's CPU path looks at the data on the host before it
quantises (``tensor_quant.py:577-587``: negative values with ``unsigned=True`` raise ``TypeError``,
a negative amax raises ``ValueError``) and ``MaxCalibrator.collect`` asserts on every batch
(``calib/max.py:69-77``).  Each of these is a device-to-host synchronisation per call, so by default
this package clamps like the reference's CUDA kernel and evaluates the calibrator's assertions once
in ``compute_amax``.  With strict checks on, the reference's errors are raised at the reference's
moment.
"""

_one_launch = False
_strict = False


def set_one_launch_dynamic_quant(enabled: bool) -> bool:
    """Allow the one-launch abs-max + quantize kernels; returns the previous setting."""
    global _one_launch
    previous, _one_launch = _one_launch, bool(enabled)
    return previous


def one_launch_dynamic_quant() -> bool:
    return _one_launch


def set_strict_checks(enabled: bool) -> bool:
    """Raise the reference's host-side errors at the reference's moment (one device
    synchronisation per checked call); returns the previous setting."""
    global _strict
    previous, _strict = _strict, bool(enabled)
    return previous


def strict_checks() -> bool:
    return _strict
