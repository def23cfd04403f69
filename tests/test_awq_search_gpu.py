"""The one-launch AWQ-lite search kernel (matrix-core GEMM with the weight quantised on the fly)
against (i) the same step done with separate kernels and a library GEMM on the device and (ii)
the CPU restatement of the reference's search loop.  Losses are sums over a GEMM whose
accumulation order differs between implementations, so they are compared to 1e-3 relative
(the figure the selected alpha is required to be stable at); typical agreement is ~1e-5."""

import pytest
import torch
import torch.nn.functional as F

from modelopt_amd import _hip
from oracle import awq as oawq

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _problem(tokens, n, k, n_alpha, seed):
    g = torch.Generator().manual_seed(seed)
    w = (0.02 * torch.randn(n, k, generator=g)).to(torch.bfloat16)
    c = torch.exp(torch.randn(k, generator=g))
    x = (torch.randn(tokens, k, generator=g) * c).to(torch.bfloat16)
    s = torch.exp(0.5 * torch.randn(n_alpha, k, generator=g)).to(torch.bfloat16)
    s[0] = 1.0
    return x, w, s


def _unfused_losses(x, w, s, ref, block, bits, unsigned, narrow):
    out = torch.zeros(s.shape[0], dtype=torch.float64, device=DEV)
    for i in range(s.shape[0]):
        xs = _hip.mul_cols(x, (1 / s[i].float()).to(torch.bfloat16))
        wq = _hip.scale_block_int_qdq(w, s[i].contiguous(), block, bits, unsigned, narrow)
        _hip.sq_diff_sum_into(F.linear(xs, wq).contiguous(), ref, out[i:i + 1])
    return out


def _fused_losses(x, w, s, ref, block, bits, unsigned, narrow):
    xs = _hip.awq_scaled_activations(x, (1 / s.float()).to(torch.bfloat16))
    out = torch.zeros(s.shape[0], dtype=torch.float64, device=DEV)
    assert _hip.awq_search_losses_into(xs, w, s.contiguous(), ref, block, bits, unsigned, narrow, out)
    return out


@pytest.mark.parametrize("tokens,n,k", [(512, 256, 512), (128, 128, 128), (100, 128, 256),
                                        (300, 384, 384), (1, 128, 128), (257, 256, 256),
                                        (512, 4096, 4096)])
@pytest.mark.parametrize("block,bits,unsigned,narrow", [(128, 4, False, False), (64, 4, False, True),
                                                         (32, 8, False, False)])
def test_matches_unfused_device_path(tokens, n, k, block, bits, unsigned, narrow):
    x, w, s = (t.to(DEV) for t in _problem(tokens, n, k, 5, tokens + n))
    ref = F.linear(x, w).contiguous()
    got = _fused_losses(x, w, s, ref, block, bits, unsigned, narrow)
    want = _unfused_losses(x, w, s, ref, block, bits, unsigned, narrow)
    assert torch.allclose(got, want, rtol=1e-3, atol=0), (got, want)
    assert (got > 0).all()


@pytest.mark.parametrize("tokens,n,k,n_alpha", [(300, 2048, 256, 21), (96, 1536, 128, 11),
                                                (512, 2560, 256, 21), (512, 4096, 4096, 21)])
def test_column_tiles_of_two_widths(tokens, n, k, n_alpha):
    """Launches whose 128-wide column tiles would leave the chip's last round part empty (more
    than 256 tiles, one per compute unit at a time) cut some of every alpha's columns into
    96-wide tiles: 16 of 20, all 16, 12 of 29 and 12 of 35 tiles per alpha in these cases."""
    x, w, s = (t.to(DEV) for t in _problem(tokens, n, k, n_alpha, tokens + n))
    ref = F.linear(x, w).contiguous()
    got = _fused_losses(x, w, s, ref, 128, 4, False, False)
    want = _unfused_losses(x, w, s, ref, 128, 4, False, False)
    assert torch.allclose(got, want, rtol=1e-3, atol=0), (got, want)
    assert int(got.argmin()) == int(want.argmin())


@pytest.mark.parametrize("tokens,n,k", [(96, 128, 256), (512, 384, 512), (300, 1536, 128)])
def test_layer_with_a_bias(tokens, n, k):
    """``bf16(sum + bias)`` in the epilogue: against the same step with a library GEMM that adds
    the bias on the device, and against the CPU restatement of the loop body with ``F.linear(xs,
    wq, bias)``."""
    x, w, s = _problem(tokens, n, k, 4, tokens + k)
    bias = (0.3 * torch.randn(n, generator=torch.Generator().manual_seed(n))).to(torch.bfloat16)
    ref = F.linear(x, w, bias)
    want_cpu = []
    for i in range(s.shape[0]):
        xs = x * (1 / s[i].float()).to(torch.bfloat16)
        out = F.linear(xs, oawq.int4_block_qdq(w * s[i], 128), bias)
        want_cpu.append((out - ref).float().pow(2).sum().double())
    want_cpu = torch.stack(want_cpu)
    xd, wd, sd, bd = (t.to(DEV) for t in (x, w, s, bias))
    ref_d = ref.to(DEV).contiguous()
    xs = _hip.awq_scaled_activations(xd, (1 / sd.float()).to(torch.bfloat16))
    got = torch.zeros(s.shape[0], dtype=torch.float64, device=DEV)
    assert _hip.awq_search_losses_into(xs, wd, sd.contiguous(), ref_d, 128, 4, False, False, got, bd)
    want_dev = torch.zeros(s.shape[0], dtype=torch.float64, device=DEV)
    for i in range(s.shape[0]):
        xi = _hip.mul_cols(xd, (1 / sd[i].float()).to(torch.bfloat16))
        wq = _hip.scale_block_int_qdq(wd, sd[i].contiguous(), 128, 4, False, False)
        _hip.sq_diff_sum_into(F.linear(xi, wq, bd).contiguous(), ref_d, want_dev[i:i + 1])
    assert torch.allclose(got, want_dev, rtol=1e-3, atol=0), (got, want_dev)
    assert torch.allclose(got.cpu(), want_cpu, rtol=1e-3, atol=0), (got, want_cpu)
    without = torch.zeros(s.shape[0], dtype=torch.float64, device=DEV)
    assert _hip.awq_search_losses_into(xs, wd, sd.contiguous(), ref_d, 128, 4, False, False, without)
    assert (without > 1.3 * got).all(), "the bias must matter in this case"


def test_accumulates_and_rejects_uncovered_shapes():
    x, w, s = (t.to(DEV) for t in _problem(64, 128, 128, 2, 3))
    ref = F.linear(x, w).contiguous()
    first = _fused_losses(x, w, s, ref, 128, 4, False, False)
    xs = _hip.awq_scaled_activations(x, (1 / s.float()).to(torch.bfloat16))
    acc = first.clone()
    assert _hip.awq_search_losses_into(xs, w, s, ref, 128, 4, False, False, acc)
    assert torch.allclose(acc, 2 * first, rtol=1e-12)
    # block size, feature count, token count outside the kernel's set: nothing is launched
    assert not _hip.awq_search_losses_into(xs, w, s, ref, 256, 4, False, False, acc)
    assert not _hip.awq_search_losses_into(xs[:, :8].contiguous(), w[:, :64].contiguous(),
                                           s[:, :64].contiguous(), ref, 32, 4, False, False, acc)
    assert not _hip.awq_search_losses_into(xs, w[:64].contiguous(), s, ref[:, :64].contiguous(), 128, 4,
                                           False, False, acc)   # 64 output features
    big = torch.zeros(2, 16, 513, 8, dtype=torch.bfloat16, device=DEV)
    assert not _hip.awq_search_losses_into(big, w, s, torch.zeros(513, 128, dtype=torch.bfloat16, device=DEV),
                                           128, 4, False, False, acc)
    assert torch.allclose(acc, 2 * first, rtol=1e-12)


def test_matches_cpu_restatement_of_the_search_loop():
    """losses of the reference's loop body (x * bf16(1/s)) @ QDQ(w * bf16(s))^T on the CPU"""
    x, w, s = _problem(96, 128, 256, 4, 11)
    ref = F.linear(x, w)
    want = []
    for i in range(s.shape[0]):
        xs = x * (1 / s[i].float()).to(torch.bfloat16)
        out = F.linear(xs, oawq.int4_block_qdq(w * s[i], 128))
        want.append((out - ref).float().pow(2).sum().double())
    want = torch.stack(want)
    got = _fused_losses(x.to(DEV), w.to(DEV), s.to(DEV), ref.to(DEV).contiguous(), 128, 4, False, False)
    assert torch.allclose(got.cpu(), want, rtol=1e-3), (got, want)


def _cpu_search_losses(x, w, s, block):
    """The reference's per-alpha loop body (model_calib.py:645-690 with the weight quantizer of
    INT4_AWQ_CFG, tensor_quant.py:574-612) on the CPU: sum of f32(bf16(out - ref))^2."""
    ref = F.linear(x, w)
    want = []
    for i in range(s.shape[0]):
        xs = x * (1 / s[i].float()).to(torch.bfloat16)
        out = F.linear(xs, oawq.int4_block_qdq(w * s[i], block))
        want.append((out - ref).float().pow(2).sum().double())
    return ref, torch.stack(want)


@pytest.mark.parametrize("tokens,n,k,n_alpha", [(512, 14336, 4096, 5), (512, 4096, 14336, 5),
                                                (200, 4096, 4096, 3)])
def test_llama_8b_layer_shapes_against_the_cpu_restatement(tokens, n, k, n_alpha):
    """gate / up (14336 x 4096) and down (4096 x 14336) of the 8B shape -- the layers the sweep
    spends its time on, 112 and 32 column tiles per alpha over 32 and 112 k blocks -- scored by
    the one-launch kernel and by the CPU restatement: every loss within 1e-3, same best alpha."""
    x, w, s = _problem(tokens, n, k, n_alpha, n + k)
    ref, want = _cpu_search_losses(x, w, s, 128)
    got = _fused_losses(x.to(DEV), w.to(DEV), s.to(DEV), ref.to(DEV).contiguous(), 128, 4, False, False)
    assert torch.allclose(got.cpu(), want, rtol=1e-3, atol=0), (got, want)
    assert int(got.argmin()) == int(want.argmin())


@pytest.mark.parametrize("tokens,k,n_alpha", [(512, 4096, 21), (100, 256, 3), (1, 8, 1), (65, 1032, 2)])
def test_scaled_activations_layout_and_rounding(tokens, k, n_alpha):
    """``bf16(x * inv_s[a])`` for every alpha, chunk-major: bit for bit the tensor expression
    (the reference multiplies the input by the bf16 pre-quant scale, tensor_quantizer.py:881-882)."""
    g = torch.Generator().manual_seed(tokens + k)
    x = (torch.randn(tokens, k, generator=g) * torch.exp(torch.randn(k, generator=g))).to(torch.bfloat16)
    inv_s = torch.exp(0.5 * torch.randn(n_alpha, k, generator=g)).to(torch.bfloat16)
    got = _hip.awq_scaled_activations(x.to(DEV), inv_s.to(DEV)).cpu()
    want = (x[None] * inv_s[:, None, :]).view(n_alpha, tokens, k // 8, 8).transpose(1, 2).contiguous()
    assert got.shape == want.shape and torch.equal(got.view(torch.int16), want.view(torch.int16))
