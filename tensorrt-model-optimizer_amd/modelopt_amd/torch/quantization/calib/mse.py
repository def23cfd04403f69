"""MSE amax search (reference: calib/mse.py:28-177).

For every tensor shown to it, ``MseCalibrator`` scores ``num_steps`` candidate amax values
(``initial_amax * linspace(start, stop, num_steps)``) by the squared error between the fp32
tensor and its fake-quantised version; ``compute_amax`` returns, per tensor or per channel, the
candidate with the smallest accumulated error.

The reference evaluates one candidate at a time: quantise, subtract, square, sum.  When the
quantizer is a plain integer or FP8 one (per tensor, or per channel with contiguous rows) all
candidates are scored by one kernel that reads the tensor once (``mo_qdq_sq_err``); anything else
-- a custom ``error_func``, NVFP4, layouts the kernel does not cover -- takes the per-candidate
route through ``quant_func``.  The multipliers are generated and kept on the host so that every
device sees the candidate list the CPU computes.
"""

import torch
import torch.nn.functional as F

from .... import _hip
from .. import kernels
from ..overflow import fp8_saturates
from ..utils import convert_quantization_axis_to_reduce_axis
from .max import _Calibrator

__all__ = ["MseCalibrator"]


class MseCalibrator(_Calibrator):
    """Per-tensor and per-channel MSE amax search."""

    def __init__(self, amax: torch.Tensor, axis=None, num_steps: int = 10,
                 start_multiplier: float = 0.25, stop_multiplier: float = 4.0, quant_func=None,
                 error_func=None, quantizer=None):
        """``quant_func(x, amax) -> xq`` and ``error_func(x, xq) -> error`` as in the reference;
        ``quantizer`` (optional) names the ``TensorQuantizer`` behind ``quant_func`` so that the
        fused kernel can be used when its format allows."""
        super().__init__(num_bits=None, axis=axis, unsigned=None)
        self._initial_amax = amax
        self._num_steps = num_steps
        self._start_multiplier = start_multiplier
        self._stop_multiplier = stop_multiplier
        self._quant_func = quant_func
        self._error_func = error_func
        self._quantizer = quantizer
        self._losses_sum = [None] * num_steps
        self._candidate_amaxs = [None] * num_steps
        self._amax = None

    def _candidates(self, device):
        # The multipliers stay 0-dim host tensors: a device kernel then receives them as fp32
        # scalars, exactly as the CPU evaluates ``amax * multiplier`` (a 0-dim *device* tensor
        # would first be rounded to the amax dtype, e.g. bf16).  A 0-dim amax times a 0-dim fp32
        # multiplier is fp32, an amax with dims keeps its own dtype.
        multipliers = torch.linspace(self._start_multiplier, self._stop_multiplier,
                                     steps=self._num_steps)
        return [self._initial_amax * m for m in multipliers]

    def _fused_spec(self):
        """Arguments of the fused kernel for the quantizer's format, or None."""
        q = self._quantizer
        if q is None or self._error_func is not None or q.block_sizes is not None:
            return None
        if q.pre_quant_scale is not None or getattr(q, "_rotate", False) or not q.fake_quant:
            return None
        if isinstance(q._num_bits, int):
            return {"kind": "int", "num_bits": q._num_bits, "unsigned": q._unsigned,
                    "narrow_range": q._narrow_range}
        if q._num_bits == (4, 3):
            return {"kind": "fp8", "saturate": None}  # decided per call from the candidates' shape
        return None

    @torch.no_grad()
    def collect(self, x: torch.Tensor):
        if self._quant_func is None:
            raise RuntimeError("Quantization function not set. Msecalibrator requires a quant_func to be provided.")
        x = x.detach()
        cands = self._candidates(x.device)
        for step in range(self._num_steps):
            if self._candidate_amaxs[step] is None:
                self._candidate_amaxs[step] = cands[step]
        reduce_axis = convert_quantization_axis_to_reduce_axis(x, self._axis)
        spec = self._fused_spec()
        if spec is not None and x.is_cuda and self._collect_fused(x, cands, reduce_axis, spec):
            return
        x = x.to(dtype=torch.float32)
        for step, cand in enumerate(cands):
            xq = self._quant_func(x, cand)
            error = self._error_func(x, xq) if self._error_func is not None else F.mse_loss(
                x, xq, reduction="none")
            loss = torch.sum(error) if reduce_axis is None else torch.sum(error, dim=reduce_axis,
                                                                          keepdim=False)
            self._losses_sum[step] = loss.clone() if self._losses_sum[step] is None else \
                self._losses_sum[step] + loss

    def _collect_fused(self, x, cands, reduce_axis, spec) -> bool:
        keep = [] if reduce_axis is None else [d for d in range(x.dim()) if d not in reduce_axis]
        layout = kernels.amax_layout(tuple(x.shape), keep)
        if layout is None:
            return False
        outer, axis, inner = layout
        x = x if x.is_contiguous() else x.contiguous()
        cand = torch.stack([c.to(torch.float32).reshape(-1).expand(axis) for c in cands]).contiguous()
        loss = torch.zeros_like(cand)
        if spec.get("saturate", False) is None:
            spec = dict(spec, saturate=fp8_saturates(cands[0]))
        if not _hip.qdq_sq_err_into(x, cand, loss, outer, axis, inner, **spec):
            return False
        for step in range(self._num_steps):
            step_loss = loss[step].reshape(()) if reduce_axis is None else loss[step]
            self._losses_sum[step] = step_loss if self._losses_sum[step] is None else \
                self._losses_sum[step] + step_loss
        return True

    def reset(self):
        self._losses_sum = [None] * self._num_steps
        self._candidate_amaxs = [None] * self._num_steps
        self._amax = None

    @torch.no_grad()
    def compute_amax(self, verbose: bool = False):
        """The candidate with the smallest accumulated error (per tensor or per channel), or
        None when nothing was collected."""
        seen = [l for l in self._losses_sum if l is not None]
        if not seen:
            return None
        first = seen[0]
        losses = torch.stack([l if l is not None else torch.full_like(first, float("inf"))
                              for l in self._losses_sum])
        best = torch.argmin(losses, dim=0)
        if first.ndim == 0:
            self._amax = self._candidate_amaxs[best.item()]
        else:
            stacked = torch.stack([c.reshape(-1) for c in self._candidate_amaxs])
            n = best.shape[0]
            self._amax = stacked[best, torch.arange(n, device=best.device)].reshape(
                self._initial_amax.shape)
        if verbose:
            ratio = self._amax / self._initial_amax
            if ratio.ndim == 0:
                print(f"MSE Calibrator: best_amax/initial_amax ratio = {ratio.item():.4f}")
            else:
                print(f"MSE Calibrator: best_amax/initial_amax ratio - mean: {ratio.mean().item():.4f}, "
                      f"min: {ratio.min().item():.4f}, max: {ratio.max().item():.4f}")
        return self._amax
