"""Oracle: MSE amax search (test infrastructure).

Restates ``MseCalibrator.collect`` / ``compute_amax`` (TQ/calib/mse.py:69-177) one candidate at a
time with torch CPU ops: fake-quantise the fp32 tensor with ``initial_amax * multiplier``,
``F.mse_loss(reduction="none")``, ``torch.sum`` over the reduced dims, accumulate over batches,
``argmin`` per tensor or per channel.
"""

import torch
import torch.nn.functional as F

from .reduce import quant_axis_to_reduce_dims


def candidates(initial_amax: torch.Tensor, num_steps=10, start=0.25, stop=4.0):
    """``initial_amax * m`` for the fp32 multipliers of ``torch.linspace`` (0-dim tensors, so a
    0-dim amax is promoted to fp32 and an amax with dims keeps its dtype), :84-92."""
    return [initial_amax * m for m in torch.linspace(start, stop, steps=num_steps)]


def mse_search(batches, initial_amax: torch.Tensor, axis, quant_func, num_steps=10, start=0.25,
               stop=4.0):
    """Returns (losses stacked [num_steps] or [num_steps, channels], best amax)."""
    cands = candidates(initial_amax, num_steps, start, stop)
    sums = [None] * num_steps
    for x in batches:
        x = x.detach().to(torch.float32)
        dims = quant_axis_to_reduce_dims(x, axis)
        for k, cand in enumerate(cands):
            err = F.mse_loss(x, quant_func(x, cand), reduction="none")
            loss = torch.sum(err) if dims is None else torch.sum(err, dim=dims, keepdim=False)
            sums[k] = loss.clone() if sums[k] is None else sums[k] + loss
    losses = torch.stack(sums)
    best = torch.argmin(losses, dim=0)
    if losses.dim() == 1:
        amax = cands[best.item()]
    else:
        stacked = torch.stack([c.reshape(-1) for c in cands])
        amax = stacked[best, torch.arange(best.shape[0])].reshape(initial_amax.shape)
    return losses, amax
