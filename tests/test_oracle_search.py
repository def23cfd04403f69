"""Pins the search oracles (``oracle.awq``: AWQ-lite, AWQ clip, SmoothQuant; ``oracle.mse``) on
the CPU against formulations that share no code with them: numpy float64, written from the
mathematics (per-column statistics, a closed-form block quantizer, explicit sums over the block
/ token / candidate axes), on the case the reference's own tests use -- the 16-32-16-16 MLP of
tests/unit/torch/quantization/test_calib.py:33-52 under seed 0 with one ``randn(2, 64, 16)``
batch and INT4 blocks of 8 (:170-186), which the reference checks against its own independent
implementations (:72-167) with ``allclose`` -- and on the known-answer properties of
tests/unit/torch/quantization/test_mse_calibrator.py:40-186.  A dropped term, a wrong axis, a
transposed operand or a wrong candidate order in the oracle fails here."""

import numpy as np
import pytest
import torch

from oracle import awq as oawq
from oracle import mse as omse
from oracle.fake_quant import tensor_quant


# ----------------------------------------------------------------------------- independent pieces
def _int_qdq64(w, amax, bits=4):
    """round-half-even(w * bound / amax) clamped to [-bound - 1, bound], times amax / bound"""
    bound = 2.0 ** (bits - 1) - 1
    scale = bound / amax
    return np.clip(np.rint(w * scale), -bound - 1, bound) / scale


def _block_qdq64(w, block, ratio=1.0):
    n, k = w.shape
    blocks = w.reshape(n, k // block, block)
    amax = np.abs(blocks).max(axis=2, keepdims=True) * ratio
    return _int_qdq64(blocks, amax).reshape(n, k)


def _mlp_case():
    """the reference test's layers and the activations each of them sees"""
    torch.manual_seed(0)
    dims = [(16, 32), (32, 16), (16, 16)]
    weights = [torch.nn.Linear(i, o, bias=False).weight.detach().clone() for i, o in dims]
    x = torch.randn(2, 64, 16)
    acts = []
    for w in weights:
        acts.append(x.reshape(-1, x.shape[-1]).clone())
        x = torch.relu(x @ w.T)
    return weights, acts


# ----------------------------------------------------------------------------- AWQ-lite
def _awq_lite64(w, x, block, alphas):
    w, x = w.double().numpy(), x.double().numpy()
    n, k = w.shape
    peak = np.abs(w.reshape(n, k // block, block)).max(axis=2, keepdims=True)
    w_stat = (np.abs(w.reshape(n, k // block, block)) / peak).reshape(n, k).mean(axis=0)
    x_stat = np.abs(x).mean(axis=0)
    ref = x @ w.T
    losses, scales = [], []
    for a in alphas:
        s = np.clip(x_stat ** a / w_stat ** (1 - a), 1e-4, 1e4)
        s = s / np.sqrt(s.max() * s.min())
        out = (x / s) @ _block_qdq64(w * s, block).T
        losses.append(((out - ref) ** 2).mean())
        scales.append(s)
    best = int(np.argmin(losses))
    return np.array(losses), best, scales[best], x_stat, w_stat


@pytest.mark.parametrize("layer", [0, 1, 2])
def test_awq_lite_oracle_against_float64_formulation(layer):
    weights, acts = _mlp_case()
    w, x = weights[layer], acts[layer]
    losses, best_alpha, best_scale, act_scale, weight_scale = oawq.awq_lite_search(w, [x], 0.1, 8)
    alphas = list(losses)
    want_losses, want_best, want_scale, x_stat, w_stat = _awq_lite64(w, x, 8, alphas)
    assert np.allclose(act_scale.numpy(), x_stat, rtol=1e-5)
    assert np.allclose(weight_scale.numpy(), w_stat, rtol=1e-5)
    got = np.array([losses[a] for a in alphas])
    # fp32 against float64: a rounding tie in the 4-bit grid can move single weights
    assert np.allclose(got, want_losses, rtol=2e-2), (got, want_losses)
    assert alphas[want_best] == pytest.approx(best_alpha) or abs(
        want_losses[want_best] - want_losses[alphas.index(best_alpha)]) < 1e-3 * want_losses[want_best]
    assert np.allclose(oawq.awq_get_scale(act_scale, weight_scale, alphas[want_best]).numpy(), want_scale,
                       rtol=1e-4)


def test_awq_scale_special_cases():
    """alpha = 0: the scale depends on the weights only; alpha = 1: on the activations only;
    the normalisation makes max * min = 1; a uniform statistic gives the all-ones scale."""
    g = torch.Generator().manual_seed(1)
    x_stat, w_stat = torch.rand(64, generator=g) + 0.1, torch.rand(64, generator=g) + 0.1
    s0 = oawq.awq_get_scale(x_stat, w_stat, 0.0)
    s1 = oawq.awq_get_scale(x_stat, w_stat, 1.0)
    want0 = 1 / w_stat
    want1 = x_stat
    assert torch.allclose(s0, want0 / (want0.max() * want0.min()).sqrt(), rtol=1e-5)
    assert torch.allclose(s1, want1 / (want1.max() * want1.min()).sqrt(), rtol=1e-5)
    for s in (s0, s1, oawq.awq_get_scale(x_stat, w_stat, 0.35)):
        assert float(s.max() * s.min()) == pytest.approx(1.0, rel=1e-5)
    ones = oawq.awq_get_scale(torch.full((8,), 0.3), torch.full((8,), 0.7), 0.6)
    assert torch.allclose(ones, torch.ones(8), rtol=1e-6)


# ----------------------------------------------------------------------------- AWQ clip
def _awq_clip64(w, x, block, ratios, max_tokens):
    w, x = w.double().numpy(), x.double().numpy()
    x = x[0::max(1, x.shape[0] // max_tokens)]
    n, k = w.shape
    nblk = k // block
    losses = np.zeros((len(ratios), n, nblk))
    for r, ratio in enumerate(ratios):
        err = _block_qdq64(w, block, ratio) - w                       # [n, k]
        for b in range(nblk):
            cols = slice(b * block, (b + 1) * block)
            partial = x[:, cols] @ err[:, cols].T                     # [tokens, n]
            losses[r, :, b] = (partial ** 2).mean(axis=0)
    amax = np.abs(w.reshape(n, nblk, block)).max(axis=2)
    best = amax * np.array(ratios)[np.argmin(losses, axis=0)]
    return losses, best


@pytest.mark.parametrize("layer", [0, 1, 2])
def test_awq_clip_oracle_against_float64_formulation(layer):
    weights, acts = _mlp_case()
    w, x = weights[layer], acts[layer]
    losses, best = oawq.awq_clip_search(w, [x], 8, 4, max_tokens_per_batch=64)
    ratios = list(losses)
    assert ratios == [0.5, 0.55, 0.6, 0.65, 0.7, 0.75, 0.8, 0.85, 0.9, 0.95, 1.0]
    want_losses, want_best = _awq_clip64(w, x, 8, ratios, 64)
    for r, ratio in enumerate(ratios):
        got = losses[ratio].numpy()
        close = np.isclose(got, want_losses[r], rtol=1e-3, atol=1e-9)
        assert close.mean() > 0.98, (ratio, close.mean())       # the rest: 4-bit rounding ties
        assert abs(got.sum() - want_losses[r].sum()) < 2e-3 * want_losses[r].sum()
    same = np.isclose(best.numpy().reshape(want_best.shape), want_best, rtol=1e-6)
    assert same.mean() > 0.97, same.mean()


def test_awq_clip_oracle_token_subsampling_and_batches():
    """every (tokens // max_tokens)-th token of each batch is used; batches add up"""
    g = torch.Generator().manual_seed(4)
    w = torch.randn(8, 32, generator=g)
    xa, xb = torch.randn(96, 32, generator=g), torch.randn(40, 32, generator=g)
    losses, _ = oawq.awq_clip_search(w, [xa, xb], 16, 4, max_tokens_per_batch=32)
    la, _ = _awq_clip64(w, xa, 16, list(losses), 32)      # 96 // 32 = 3: tokens 0, 3, 6, ...
    lb, _ = _awq_clip64(w, xb, 16, list(losses), 32)      # 40 // 32 = 1: all 40 tokens
    for r, ratio in enumerate(losses):
        got, want = losses[ratio].numpy(), la[r] + lb[r]
        assert abs(got.sum() - want.sum()) < 2e-3 * want.sum()
        assert np.isclose(got, want, rtol=1e-3, atol=1e-9).mean() > 0.95


# ----------------------------------------------------------------------------- SmoothQuant
def test_smoothquant_oracle_against_float64_formulation():
    """s = w_col^(1 - a) / x^a; the smoothed layer computes the same function; the new input
    amax is max(x_amax * s) and the weight amax the row maxima of w / s."""
    g = torch.Generator().manual_seed(2)
    w = torch.randn(24, 48, generator=g)
    act_amax = torch.rand(48, generator=g) * 5 + 0.1
    for alpha in (0.5, 0.8, 1.0):
        pqs, w_new, in_amax, w_amax = oawq.smoothquant_linear(w, act_amax, alpha)
        wcol = np.abs(w.double().numpy()).max(axis=0)
        s = np.clip(wcol ** (1 - alpha) / act_amax.double().numpy() ** alpha, 1e-4, 1e4)
        assert np.allclose(pqs.numpy(), s, rtol=1e-5)
        assert np.allclose(w_new.numpy(), w.double().numpy() / s, rtol=1e-5)
        assert float(in_amax) == pytest.approx((act_amax.double().numpy() * s).max(), rel=1e-5)
        assert np.allclose(w_amax.numpy().reshape(-1), np.abs(w.double().numpy() / s).max(axis=1), rtol=1e-5)
        x = torch.randn(5, 48, generator=g)
        assert torch.allclose((x * pqs) @ w_new.T, x @ w.T, rtol=1e-4, atol=1e-4)


# ----------------------------------------------------------------------------- MSE search
def _mse64(x, amax0, multipliers, bits, unsigned=False, axis=None):
    x = x.double().numpy()
    losses = []
    for m in multipliers:
        amax = amax0 * m
        bound = 2.0 ** (bits - 1 + int(unsigned)) - 1
        lo = 0.0 if unsigned else -bound            # narrow range, the TensorQuantizer default
        scale = bound / amax
        q = np.clip(np.rint(x * scale), lo, bound) / scale
        err = (x - q) ** 2
        losses.append(err.sum() if axis is None else err.sum(axis=tuple(i for i in range(x.ndim) if i != axis)))
    return np.array(losses)


def _quant(bits, unsigned):
    return lambda x, amax: tensor_quant(x, amax, bits, unsigned, True)


def test_mse_oracle_outlier_cases():
    """test_mse_calibrator.py:40-186: a single outlier (1024 ones and a 10, its negative twin, an
    unsigned variant) -- the search must settle on an amax that beats both the initial one and
    1.0; here additionally the whole loss curve equals the float64 one."""
    for sign, unsigned in ((1.0, False), (-1.0, False), (1.0, True)):
        x = torch.ones(1024)
        x[0] = 10.0 * sign
        if unsigned:
            x = x.abs()
        amax0 = x.abs().max()
        losses, best = omse.mse_search([x], amax0, None, _quant(8, unsigned), 20, 0.1, 1.5)
        mult = np.linspace(0.1, 1.5, 20)
        want = _mse64(x, float(amax0), mult, 8, unsigned)
        assert np.allclose(losses.numpy(), want, rtol=1e-4, atol=1e-6)
        assert float(best) == pytest.approx(float(amax0) * mult[int(np.argmin(want))], rel=1e-6)
        assert 0 < float(best) <= float(amax0) * 1.5 + 1e-6
        at_best = _mse64(x, float(best), [1.0], 8, unsigned)[0]
        assert at_best <= _mse64(x, 1.0, [1.0], 8, unsigned)[0] + 1e-6
        assert at_best <= _mse64(x, float(amax0), [1.0], 8, unsigned)[0] + 1e-6


def test_mse_oracle_accumulates_batches_and_optimises_channels_independently():
    """:187-232, :321-479: losses of several collections add; with a per-channel amax every
    channel picks its own multiplier"""
    g = torch.Generator().manual_seed(0)
    xa, xb = torch.rand(4096, generator=g) * 2 - 1, torch.rand(4096, generator=g) * 2 - 1
    amax0 = torch.tensor(1.0)
    both, best = omse.mse_search([xa, xb], amax0, None, _quant(8, False), 12, 0.5, 1.5)
    mult = np.linspace(0.5, 1.5, 12)
    want = _mse64(xa, 1.0, mult, 8) + _mse64(xb, 1.0, mult, 8)
    assert np.allclose(both.numpy(), want, rtol=1e-4)
    assert float(best) == pytest.approx(mult[int(np.argmin(want))], rel=1e-6)

    x = torch.randn(6, 512, generator=g) * torch.tensor([0.1, 1.0, 3.0, 0.5, 2.0, 8.0])[:, None]
    x[2, 0], x[5, 7] = 60.0, -200.0                         # outliers in two channels only
    amax0 = x.abs().amax(dim=1, keepdim=True)
    losses, best = omse.mse_search([x], amax0, 0, _quant(4, False), 10, 0.25, 4.0)
    mult = np.linspace(0.25, 4.0, 10)
    assert losses.shape == (10, 6)
    for c in range(6):
        want = _mse64(x[c], float(amax0[c]), mult, 4)
        assert np.allclose(losses[:, c].numpy(), want, rtol=1e-4)
        assert float(best[c]) == pytest.approx(float(amax0[c]) * mult[int(np.argmin(want))], rel=1e-6)
    picked = (best / amax0).reshape(-1)
    assert float(picked[2]) < 1.0 and float(picked[5]) < 1.0       # the outlier channels clip


# ----------------------------------------------------------------------------- small helpers
def test_fold_pre_quant_scale_keeps_the_layer_function():
    """the folded weight with the scaled input computes what the layer computed"""
    g = torch.Generator().manual_seed(6)
    w, x = torch.randn(12, 20, generator=g), torch.randn(7, 20, generator=g)
    p = torch.rand(20, generator=g) + 0.5
    pqs, w_new = oawq.fold_pre_quant_scale(w, p)
    assert torch.allclose(pqs, p) and torch.allclose(w_new, w / p[None, :], rtol=1e-6)
    assert torch.allclose((x * pqs) @ w_new.T, x @ w.T, rtol=1e-4, atol=1e-5)


def test_int8_export_cast_and_block_fake_quant_closed_forms():
    from oracle import export as oexport
    from oracle.fake_quant import static_block_fake_quant

    g = torch.Generator().manual_seed(7)
    w = torch.randn(10, 24, generator=g) * 3
    s = w.abs().amax(dim=1) / 127.0
    want = np.clip(np.rint(w.double().numpy() / s.double().numpy()[:, None]), -128, 127)
    got = oexport.int8_export_cast(w, s).numpy()
    assert (got != want).mean() < 0.01 and np.abs(got - want).max() <= 1   # fp32 vs float64 quotient at a tie
    got = static_block_fake_quant(w, 8, lambda x2, amax: tensor_quant(x2, amax, 4, False, False))
    assert np.allclose(got.numpy(), _block_qdq64(w.double().numpy(), 8), rtol=1e-5, atol=1e-6)
