"""Max calibrator with a device-resident running maximum.

Same interface and result as the reference's ``MaxCalibrator`` (modelopt/torch/quantization/
calib/max.py:26-94).  ``collect`` is one kernel launch that folds |x| into a persistent fp32
accumulator with integer atomic max -- no temporaries and no host synchronisation.  The three
sanity checks the reference runs (and blocks on) at every ``collect`` -- non-negative, no inf, no
NaN -- are evaluated once, in ``compute_amax``; NaN and inf survive the running max, so nothing
is lost by deferring them.  ``modes.set_strict_checks(True)`` brings the reference's timing back:
every ``collect`` then reduces the batch on its own, asserts on it (one host synchronisation) and
only then folds it in.
"""

import torch

from .. import kernels, modes
from ..utils import convert_quantization_axis_to_reduce_axis

__all__ = ["MaxCalibrator"]

# Inside a calibration pass of this package (the flag is raised by ``calibration_pass``) one
# activation is often shown to several calibrators in a row -- the input of q_proj, k_proj and
# v_proj, of gate_proj and up_proj.  The first per-tensor reduction then also leaves the abs-max
# of every tile of the tensor behind, and a calibrator that is shown the *same tensor* next (same
# memory, shape, strides, dtype and version counter, the tensor object of the first reduction
# still alive so that its memory cannot have been handed out again) notes those words instead of
# reading the tensor again; it folds them into its running maximum when that is next looked at.
# Leaving the tile maxima behind costs the host a few microseconds per reduction, so it starts
# only once a pass has shown one tensor to two calibrators in a row (the first layer of a model
# with shared inputs does); a model whose quantizers never share an input pays nothing.
SHARE_REDUCTIONS = [False]
_last_reduction = [None]   # (key, the tensor itself, its tile maxima or None)
_sharing_seen = [False]


def forget_last_reduction():
    """Drop the reference to the last tensor reduced (end of a calibration pass)."""
    _last_reduction[0] = None
    _sharing_seen[0] = False


def _sharing_key(x):
    try:
        version = x._version
    except RuntimeError:   # inference tensors keep no version counter
        return None
    return (x.data_ptr(), version, tuple(x.shape), x.stride(), x.dtype, x.device.index,
            torch._C._cuda_getCurrentRawStream(x.device.index))


def collect_pair(cal0, x0, cal1, x1) -> bool:
    """``cal0.collect(x0); cal1.collect(x1)`` for two plain per-tensor ``MaxCalibrator``s in one
    kernel launch (the key and value states of an attention layer).  False, with nothing
    collected, when the pair is not covered; the caller then collects one by one."""
    if modes.strict_checks():
        return False
    flats = []
    for cal, x in ((cal0, x0), (cal1, x1)):
        if (type(cal) is not MaxCalibrator or cal._track_amax or cal._axis is not None
                or not x.is_cuda or x.numel() == 0 or (cal._acc is not None and cal._shape != torch.Size(()))):
            return False
        flat = x if x.is_contiguous() else kernels.dense_flat_view(x)   # order does not matter
        if flat is None:
            return False
        flats.append(flat)
    for cal, x in ((cal0, x0), (cal1, x1)):
        if cal._acc is None:
            cal._acc = torch.zeros(1, dtype=torch.float32, device=x.device)
            cal._shape, cal._dtype = torch.Size(()), x.dtype
    with torch.no_grad():
        if not kernels._hip.absmax_pair_into(flats[0], cal0._acc, flats[1], cal1._acc):
            return False
    cal0._validated = cal1._validated = False
    return True


class _Calibrator:
    def __init__(self, num_bits=8, axis=None, unsigned=False):
        self._num_bits = num_bits
        self._axis = axis
        self._unsigned = unsigned

    def collect(self, x):
        raise NotImplementedError

    def reset(self):
        raise NotImplementedError

    def compute_amax(self, *args, **kwargs):
        raise NotImplementedError

    def __repr__(self):
        return f"num_bits={self._num_bits} axis={self._axis} unsigned={self._unsigned}"


class MaxCalibrator(_Calibrator):
    """Tracks the running abs-max of every tensor it is shown."""

    def __init__(self, num_bits=8, axis=None, unsigned=False, track_amax=False):
        super().__init__(num_bits, axis, unsigned)
        self._track_amax = track_amax
        if track_amax:
            self._amaxs = []
        self._acc = None             # fp32 running max, one element per kept channel
        self._shape = None           # amax shape with the reduced dims kept as 1
        self._dtype = None
        self._meta_amax = None       # meta-device shortcut only
        self._validated = False
        self._seen_parameter = None  # identity of the last nn.Parameter folded in
        self._pending = []           # tile maxima of shared reductions not yet folded into _acc

    @property
    def amaxs(self):
        return self._amaxs

    @property
    def _calib_amax(self):
        """The running abs-max as the reference keeps it (calib/max.py:45, :86-93): a tensor of the
        collected dtype and amax shape, None before the first ``collect``.  Subclasses that
        override ``compute_amax`` read it (tests/unit/torch/quantization/test_quantize_cpu.py:73-75)."""
        if self._acc is None:
            return self._meta_amax
        self._fold_pending()
        return self._acc.to(self._dtype).reshape(self._shape)

    def _fold_pending(self):
        """Fold the tile maxima noted by shared reductions into the running maximum (the bit
        patterns of non-negative floats order like the values; a NaN pattern is the largest)."""
        if self._pending:
            words = self._pending[0] if len(self._pending) == 1 else torch.cat(self._pending)
            self._pending = []
            self._acc = torch.maximum(self._acc.view(torch.int32), words.max()).view(torch.float32)

    @staticmethod
    def _amax_shape(x, reduce_axis):
        if reduce_axis is None:
            return torch.Size(())
        shape = torch.Size(1 if d in reduce_axis else x.shape[d] for d in range(x.dim()))
        # the reference squeezes a one-element result to a scalar
        return torch.Size(()) if shape.numel() == 1 else shape

    def collect(self, x):
        """Fold the abs-max of ``x`` (over everything but ``axis``) into the running maximum.

        Raises ``RuntimeError`` when the amax shape differs from what was collected before.
        """
        if torch.is_grad_enabled():
            with torch.no_grad():
                return self._collect(x)
        return self._collect(x)

    def _collect(self, x):
        reduce_axis = convert_quantization_axis_to_reduce_axis(x, self._axis)
        shape = self._amax_shape(x, reduce_axis)
        if x.device.type == "meta":
            self._meta_amax = torch.empty(shape, dtype=x.dtype, device="meta")
            return
        keep = [] if reduce_axis is None else [d for d in range(x.dim()) if d not in reduce_axis]
        layout = kernels.amax_layout(tuple(x.shape), keep)
        if layout is None:  # kept dims apart (2-D blocks): reduce a copy with them in front
            x, _, layout = kernels.kept_dims_first(x, keep)
        if self._acc is None:
            self._acc = torch.zeros(layout[1], dtype=torch.float32, device=x.device)
            self._shape, self._dtype = shape, x.dtype
        elif shape != self._shape:
            raise RuntimeError("amax shape changed!")
        if modes.strict_checks():
            self._collect_checked(x, layout)
        elif not self._track_amax:
            if not (SHARE_REDUCTIONS[0] and layout[1] == 1 and x.is_cuda and x.is_contiguous()
                    and not isinstance(x, torch.nn.Parameter)) or not self._collect_shared(x):
                kernels.absmax_accumulate(x, self._acc, layout)
        else:
            local = torch.zeros_like(self._acc)
            kernels.absmax_accumulate(x, local, layout)
            self._acc = torch.maximum(self._acc, local)
            self._amaxs.append(local.reshape(shape).to(x.dtype).float().cpu().numpy())
        self._validated = False

    def _collect_checked(self, x, layout):
        """``collect`` as the reference runs it (calib/max.py:62-86): the abs-max of this batch
        alone, the three assertions on it -- one host synchronisation -- and only then the
        running maximum, so that a bad batch is reported when it is shown and leaves the
        calibrator as it was."""
        local = torch.zeros_like(self._acc)
        kernels.absmax_accumulate(x, local, layout)
        bad = torch.stack([(local < 0).any(), torch.isinf(local).any(),
                           torch.isnan(local).any()]).tolist()
        assert not bad[0], "detected negative values after abs, could be torch or cuda bug"
        assert not bad[1], ("detected inf values in amax. inf in original tensor: "
                            f"{torch.any(torch.isinf(x))}")
        assert not bad[2], ("detected nan values in amax. nan in original tensor: "
                            f"{torch.any(torch.isnan(x))}")
        self._acc = torch.maximum(self._acc, local)
        if self._track_amax:
            self._amaxs.append(local.reshape(self._shape).to(x.dtype).float().cpu().numpy())

    def _collect_shared(self, x) -> bool:
        """Per-tensor reduction inside a calibration pass: note the tile maxima of the previous
        reduction when it was of this very tensor, else reduce and leave the tile maxima for
        the next calibrator.  False when the tensor is not covered (the caller reduces it)."""
        key = _sharing_key(x)
        if key is None:
            return False
        last = _last_reduction[0]
        if last is not None and last[1] is x and last[0] == key:
            if last[2] is None:          # the same tensor twice in a row: share from now on
                _sharing_seen[0] = True
                return False
            self._pending.append(last[2])
            if len(self._pending) >= 64:
                self._fold_pending()
            return True
        parts = kernels._hip.absmax_tensor_parts_into(x, self._acc) if _sharing_seen[0] else None
        _last_reduction[0] = (key, x, parts)
        return parts is not None

    def reset(self):
        self._seen_parameter = None
        self._pending = []
        self._acc = None
        self._shape = None
        self._meta_amax = None
        self._validated = False

    def has_amax(self) -> bool:
        """Whether ``compute_amax`` would return something, without computing it."""
        return self._acc is not None or self._meta_amax is not None

    def compute_amax(self):
        """Running abs-max in the dtype of the collected tensors, or None if nothing was seen."""
        if self._acc is None:
            return self._meta_amax
        self._fold_pending()
        # always a tensor of its own (never a view of the accumulator)
        amax = self._acc.to(self._dtype, copy=True).reshape(self._shape)
        if not self._validated:
            bad = torch.stack([(self._acc < 0).any(), torch.isinf(self._acc).any(),
                               torch.isnan(self._acc).any()]).tolist()  # one host sync
            assert not bad[0], "detected negative values after abs, could be torch or cuda bug"
            assert not bad[1], "detected inf values in amax"
            assert not bad[2], "detected nan values in amax"
            self._validated = True
        return amax

    def __str__(self):
        return f"MaxCalibrator(track_amax={self._track_amax})"

    def __repr__(self):
        # the reference's fields in its order (calib/max.py:102-110)
        s = f"MaxCalibrator({super().__repr__()} calib_amax={self._calib_amax} track_amax={self._track_amax}"
        if self._track_amax:
            s += f" amaxs={self._amaxs}"
        return s + ")"
