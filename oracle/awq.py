"""Oracle: AWQ-lite scale search and SmoothQuant for one linear layer (test infrastructure).

Functional restatement (one ``[N, K]`` weight, a list of ``[T, K]`` activation batches) of what
the reference does module by module through patched forwards.
"""

import torch
import torch.nn.functional as F

from .fake_quant import static_block_fake_quant, tensor_quant
from .reduce import reduce_amax


def pow_ref(t: torch.Tensor, exponent: float):
    """``t.pow(exponent)`` as the reference writes it, with one host dependence removed: torch's
    CPU kernel evaluates ``pow(x, 0.5)`` as an fp32 square root, which is correctly rounded on
    some hosts and one ulp off for about one input in six on others (seen between two x86 hosts
    with the same torch build).  The oracle pins the correctly rounded root -- a double-precision
    root rounded to fp32, then to ``t.dtype`` -- so that it gives one answer everywhere."""
    if exponent == 0.5:
        return t.double().sqrt().float().to(t.dtype)
    return t.pow(exponent)


def awq_weight_scale(w: torch.Tensor, block_size: int | None):
    """mean over rows of |w| / (block amax + tiny), in the weight dtype, then fp32 ``[K]``.
    Follows TQ/model_calib.py:588-603."""
    shape = w.shape
    keep = None
    if block_size:
        if shape[-1] % block_size:
            keep = slice(shape[-1])
            w = F.pad(w, (0, block_size - shape[-1] % block_size), "constant", 0)
            shape = w.shape
        w = w.contiguous().view(-1, block_size)
    peak = w.abs().amax(dim=1, keepdim=True)
    s = (w.abs() / (peak + torch.finfo(w.dtype).tiny)).view(shape)
    if keep is not None:
        s = s[..., keep]
    return s.mean(0).to(torch.float32)


def awq_act_scale(x: torch.Tensor):
    """mean over tokens of |x| in the activation dtype, then fp32 ``[K]``.
    Follows TQ/model_calib.py:605-606."""
    return x.abs().contiguous().view(-1, x.shape[-1]).mean(0).to(torch.float32)


def awq_get_scale(x_max: torch.Tensor, w_max: torch.Tensor, alpha: float):
    """s = clamp(x^a / (w^(1-a) + tiny), 1e-4, 1e4); s /= sqrt(max(s) * min(s)).
    Follows TQ/model_calib.py:608-621."""
    s = (pow_ref(x_max, alpha) / (pow_ref(w_max, 1 - alpha) + torch.finfo(torch.float32).tiny)).clamp(
        min=1e-4, max=1e4).view(-1)
    return (s / (s.max() * s.min()).sqrt()).view(-1)


def awq_alphas(alpha_step: float):
    """Keys of the loss table: fp32 ``arange`` items.  Follows TQ/model_calib.py:562-565."""
    return [k.item() for k in torch.arange(0, 1.0 + alpha_step, alpha_step)]


def int4_block_qdq(w: torch.Tensor, block_size: int):
    """INT4 static-block QDQ of a weight as the weight quantizer of ``INT4_AWQ_CFG`` does it:
    4 bit, ``narrow_range`` False (range [-8, 7]), block amax computed on the fly."""
    return static_block_fake_quant(
        w, block_size, lambda x2, amax: tensor_quant(x2, amax, 4, False, False))


@torch.no_grad()
def awq_lite_search(w: torch.Tensor, batches, alpha_step: float = 0.1, block_size: int = 128,
                    bias=None):
    """Follows TQ/model_calib.py:530-786 for one weight-only INT4 linear.

    Pass 1 averages ``awq_act_scale`` over batches; pass 2 accumulates, per alpha,
    ``mean(f32(bf16(out - out_actual))**2)`` where ``out = (x * bf16(1/s)) @ QDQ(w * bf16(s))^T``.
    Returns (losses dict alpha->float, best_alpha, best_scale fp32 [K], act_scale, weight_scale).
    """
    weight_scale = awq_weight_scale(w, block_size)
    act_scale = 0.0
    for x in batches:
        act_scale = act_scale + awq_act_scale(x)
    act_scale = act_scale / len(batches)
    losses = {a: torch.zeros((), dtype=torch.float32) for a in awq_alphas(alpha_step)}
    for x in batches:
        ref_out = F.linear(x, w, bias)
        for a in losses:
            s = awq_get_scale(act_scale, weight_scale, a)
            xs = x * (1 / s).to(w.dtype)
            ws = w * s.to(w.dtype)
            out = F.linear(xs, int4_block_qdq(ws, block_size), bias)
            losses[a] += (out - ref_out).float().pow(2).mean()
    losses = {a: float(v) for a, v in losses.items()}
    best_alpha = min(losses, key=losses.get)
    best_scale = awq_get_scale(act_scale, weight_scale, best_alpha)
    return losses, best_alpha, best_scale, act_scale, weight_scale


@torch.no_grad()
def fold_pre_quant_scale(w: torch.Tensor, pre_quant_scale: torch.Tensor):
    """Follows TQ/model_calib.py:346-393: input scale ``bf16(p)``; weight
    ``w <- dtype(w * (1.0 / f32(p))[None, :])`` (bf16 tensor times fp32 row -> fp32 product)."""
    p = pre_quant_scale.to(torch.float32)
    inv = 1.0 / p
    w_new = (w * inv.squeeze()[None, :]).to(w.dtype)
    return p.to(w.dtype), w_new


@torch.no_grad()
def smoothquant_linear(w: torch.Tensor, act_amax: torch.Tensor, alpha: float = 1.0):
    """SmoothQuant post-processing of one INT8 linear.  Follows TQ/model_calib.py:447-473 and
    :365-408.  ``act_amax`` is the calibrated per-channel input amax ``[K]`` (input dtype).

    Returns (input pre_quant_scale [K] in w.dtype, smoothed weight, new per-tensor input amax,
    new per-row weight amax [N, 1]).
    """
    a = act_amax.float()
    wcol = w.abs().amax(dim=0, keepdim=True)
    scale_a = (pow_ref(wcol, 1 - alpha) / pow_ref(a, alpha)).squeeze()
    eps = 1.0 / (1 << 31)
    if scale_a.min() <= eps:
        scale_a[a.reshape(-1) <= eps] = 1
    scale_a = scale_a.clamp(min=1e-4, max=1e4)
    pqs, w_new = fold_pre_quant_scale(w, scale_a)
    smoothing = a.to(w.dtype)
    in_amax = (smoothing * scale_a.to(torch.float32)).amax().to(w.dtype)
    w_amax = reduce_amax(w_new, axis=[1], keepdims=True)
    return pqs, w_new, in_amax, w_amax


@torch.no_grad()
def awq_clip_search(w: torch.Tensor, batches, block_size: int = 128, num_bits: int = 4,
                    max_co_batch_size: int = 1024, max_tokens_per_batch: int = 64,
                    min_clip_ratio: float = 0.5, shrink_step: float = 0.05):
    """AWQ clip for one ``[N, K]`` weight with static last-axis INT blocks.  Follows
    TQ/model_calib.py:810-929,852-862: per clip ratio the weight is fake-quantised with
    ``ratio * block amax``; the error is measured on the per-block partial outputs of up to
    ``max_tokens_per_batch`` strided tokens of every batch, all elementwise arithmetic in the
    weight dtype as the reference writes it.  Returns (losses {ratio: [N, K/bs]}, best clip amax
    [N * K/bs, 1])."""
    co, ci = w.shape
    assert ci % block_size == 0
    w_amax = reduce_amax(w.reshape(-1, block_size), axis=[1], keepdims=True)
    ratios = [round(float(k), 2) for k in torch.arange(min_clip_ratio, 1.0, shrink_step)] + [1.0]
    losses = {k: torch.zeros((co, ci // block_size)) for k in ratios}
    w4 = w.reshape(co, 1, -1, block_size)
    for x in batches:
        x = x.reshape(-1, x.shape[-1])
        x = x[0::max(1, x.shape[0] // max_tokens_per_batch)]
        x4 = x.reshape(1, x.shape[0], -1, block_size)
        for lo in range(0, co, max_co_batch_size):
            hi = min(lo + max_co_batch_size, co)
            org_out = (x4 * w4[lo:hi]).sum(dim=-1)
            for shrink in ratios:
                amax = w_amax * shrink
                wq = tensor_quant(w.reshape(-1, block_size), amax, num_bits, False, False).reshape(w.shape)
                cur_out = (x4 * wq[lo:hi].reshape(w4[lo:hi].shape)).sum(dim=-1)
                losses[shrink][lo:hi] += (cur_out - org_out).float().pow(2).mean(dim=1)
    best_loss = torch.ones_like(w_amax) * float("inf")
    best = torch.zeros_like(w_amax)
    for shrink, loss in losses.items():
        loss = loss.view_as(w_amax)
        better = loss < best_loss
        best_loss = torch.where(better, loss, best_loss)
        best = torch.where(better, w_amax * shrink, best)
    return losses, best
