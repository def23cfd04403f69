"""Seeded random cases -- shapes, magnitudes from 1e-9 to 1e5, heavy tails, zeros, a few special
values -- through the main kernels, each against the CPU oracle bit for bit.  Small tensors, many
of them: the fixed-shape tests cover the layouts, these cover the value space around them."""

import pytest
import torch

from conftest import assert_bits_equal
from modelopt_amd import _hip
from oracle import fake_quant, qtensor, reduce

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _case(seed, dtype, last_multiple=1):
    g = torch.Generator().manual_seed(seed)
    rows = int(torch.randint(1, 97, (1,), generator=g))
    k = int(torch.randint(1, 40, (1,), generator=g)) * last_multiple
    scale = 10.0 ** float(torch.empty(1).uniform_(-9, 5, generator=g))
    x = torch.randn(rows, k, generator=g)
    kind = seed % 5
    if kind == 1:    # heavy tail
        x = x * torch.exp(2.5 * torch.randn(rows, k, generator=g))
    elif kind == 2:  # sparse
        x = x * (torch.rand(rows, k, generator=g) < 0.15)
    elif kind == 3:  # a few huge outliers
        x.view(-1)[torch.randint(0, x.numel(), (3,), generator=g)] *= 1e4
    elif kind == 4:  # whole rows of zeros and negative zeros
        x[::3] = 0.0
        x[1::7] = -0.0
    return (x * scale).to(dtype)


@pytest.mark.parametrize("seed", range(40))
def test_nvfp4_quantize_pack_and_dequantize(seed):
    dtype = (torch.bfloat16, torch.float16, torch.float32)[seed % 3]
    x = _case(seed, dtype, 16)
    if dtype == torch.float16:
        x = x.clamp(-6e4, 6e4)
    po, wo, w2o = qtensor.nvfp4_quantize(x, 16)
    amax = reduce.reduce_amax(x).float()
    packed, wsf, wsf2 = _hip.nvfp4_quantize(x.to(DEV), amax.to(DEV), 16)
    assert_bits_equal(wsf2.cpu().reshape(()), w2o.reshape(()), f"global scale, seed {seed}")
    assert_bits_equal(wsf.cpu(), wo, f"block scales, seed {seed}")
    assert_bits_equal(packed.cpu(), po, f"codes, seed {seed}")
    y = _hip.nvfp4_dequantize(packed, wsf, wsf2, 16, dtype)
    assert_bits_equal(y.cpu(), qtensor.nvfp4_dequantize(po, wo, w2o, 16, x.shape, dtype), f"dequantised, seed {seed}")


@pytest.mark.parametrize("seed", range(40))
def test_fp8_and_int_fake_quant(seed, cpu_fp8_overflow):
    dtype = (torch.bfloat16, torch.float16, torch.float32)[seed % 3]
    x = _case(seed + 100, dtype, 8 if seed % 2 else 1)
    if dtype == torch.float16:
        x = x.clamp(-6e4, 6e4)
    xd = x.to(DEV)
    amax = reduce.reduce_amax(x)
    clip = amax * (0.5 if seed % 4 == 0 else 1.0)      # every fourth case clips
    got = _hip.fp8_qdq(xd, clip.to(DEV), 1, 1, x.numel()).cpu()
    assert_bits_equal(got, fake_quant.fp8_eager(x, clip), f"fp8 per tensor, seed {seed}")
    bits = (8, 4, 3, 5, 7, 11)[seed % 6]
    unsigned = seed % 7 == 3
    xi = x.abs() if unsigned else x
    got = _hip.int_qdq(xi.to(DEV), clip.to(DEV), 1, 1, x.numel(), bits, unsigned, seed % 2 == 0).cpu()
    assert_bits_equal(got, fake_quant.tensor_quant(xi, clip, bits, unsigned, seed % 2 == 0), f"int{bits}, seed {seed}")
    # per row
    a_row = reduce.reduce_amax(x, axis=[1], keepdims=True)
    got = _hip.int_qdq(xd, a_row.reshape(-1).to(DEV), 1, x.shape[0], x.shape[1], bits, False, False).cpu()
    assert_bits_equal(got, fake_quant.tensor_quant(x, a_row, bits, False, False), f"int{bits} per row, seed {seed}")
    got = _hip.fp8_qdq(xd, a_row.reshape(-1).to(DEV), 1, x.shape[0], x.shape[1]).cpu()
    assert_bits_equal(got, fake_quant.fp8_eager(x, a_row), f"fp8 per row, seed {seed}")


@pytest.mark.parametrize("seed", range(24))
def test_abs_max_reductions(seed):
    dtype = (torch.bfloat16, torch.float16, torch.float32)[seed % 3]
    x = _case(seed + 200, dtype)
    if dtype == torch.float16:
        x = x.clamp(-6e4, 6e4)
    xd = x.to(DEV)
    rows, k = x.shape
    for outer, axis, inner, want in ((1, 1, x.numel(), reduce.reduce_amax(x).reshape(1)),
                                     (1, rows, k, reduce.reduce_amax(x, axis=[1]).reshape(-1)),
                                     (rows, k, 1, reduce.reduce_amax(x, axis=[0]).reshape(-1))):
        acc = torch.zeros(axis, dtype=torch.float32, device=DEV)
        _hip.absmax_into(xd, acc, outer, axis, inner)
        assert_bits_equal(acc.cpu().to(dtype), want, f"abs-max [{outer}, {axis}, {inner}], seed {seed}")


def _wide_case(seed, dtype, last_multiple):
    """Like ``_case`` with shapes up to a few hundred thousand elements, so that the tiled kernels
    run with several workgroups and ragged last tiles."""
    g = torch.Generator().manual_seed(seed)
    rows = int(torch.randint(1, 700, (1,), generator=g))
    k = int(torch.randint(1, 40, (1,), generator=g)) * last_multiple
    while rows * k > 400_000:
        rows = max(1, rows // 2)
    scale = 10.0 ** float(torch.empty(1).uniform_(-6, 3, generator=g))
    x = torch.randn(rows, k, generator=g)
    kind = seed % 5
    if kind == 1:
        x = x * torch.exp(2.0 * torch.randn(rows, k, generator=g))
    elif kind == 2:
        x = x * (torch.rand(rows, k, generator=g) < 0.15)
    elif kind == 3:
        x.view(-1)[torch.randint(0, x.numel(), (3,), generator=g)] *= 1e3
    elif kind == 4:
        x[::3] = 0.0
        x[1::7] = -0.0
    x = (x * scale).to(dtype)
    return x.clamp(-6e4, 6e4) if dtype == torch.float16 else x


@pytest.mark.parametrize("seed", range(24))
def test_int4_export_pack_with_both_scale_types(seed):
    from oracle import export

    dtype = (torch.bfloat16, torch.float16, torch.float32)[seed % 3]
    bs = (8, 16, 64, 128, 12)[seed % 5]
    w = _wide_case(seed + 300, dtype, bs)
    if w.shape[0] % 2:
        w = torch.cat([w, w[:1]])
    ws = reduce.reduce_block_amax(w, {-1: bs}).float() / 7.0
    ws[ws == 0] = 1.0
    assert_bits_equal(_hip.int4_pack_rows(w.to(DEV), ws.to(DEV)).cpu(), export.pack_int4_in_uint8(w, ws),
                      f"fp32 scales, seed {seed}")
    if dtype != torch.float32:
        narrow = ws.to(dtype)
        narrow[narrow == 0] = 1.0
        assert_bits_equal(_hip.int4_pack_rows(w.to(DEV), narrow.float().to(DEV), dtype).cpu(),
                          export.pack_int4_in_uint8(w, narrow), f"scales in the weight's type, seed {seed}")


@pytest.mark.parametrize("seed", range(24))
def test_int4_blocks_and_storage_casts(seed):
    from oracle import export

    dtype = (torch.bfloat16, torch.float16, torch.float32)[seed % 3]
    bs = (16, 32, 64, 128)[seed % 4]
    x = _wide_case(seed + 400, dtype, bs)
    p_o, s_o = qtensor.int4_quantize(x, bs)
    packed, scales = _hip.int4_block_quantize(x.to(DEV).view(-1), bs)
    assert_bits_equal(scales.cpu(), s_o, f"int4 scales, seed {seed}")
    assert torch.equal(packed.cpu(), p_o.reshape(-1)), f"int4 codes, seed {seed}"
    y = _hip.int4_block_dequantize(packed, scales, bs)[: x.numel()].reshape(x.shape)
    assert_bits_equal(y.cpu(), qtensor.int4_dequantize(p_o, s_o, bs, x.shape, dtype), f"int4 dequantised, seed {seed}")
    rows, k = x.shape
    amax = x.abs().amax(dim=1).float()
    amax[amax == 0] = 1.0
    for scale_dtype in (torch.float32, dtype):
        s8, s_fp8 = (amax / 127.0).to(scale_dtype), (amax / 448.0).to(scale_dtype)
        via = torch.result_type(x, s8[:, None])
        got = _hip.real_quantize(x.to(DEV), s8.to(DEV), 1, rows, k, via, _hip.MO_FMT_INT8)
        assert torch.equal(got.cpu(), export.int8_export_cast(x, s8)), f"int8 cast, {scale_dtype} scales, seed {seed}"
        got = _hip.real_quantize(x.to(DEV), s_fp8.to(DEV), 1, rows, k, via, _hip.MO_FMT_E4M3)
        assert torch.equal(got.cpu().view(torch.uint8), export.fp8_export_cast(x, s_fp8[:, None]).view(torch.uint8)), (
            f"fp8 cast, {scale_dtype} scales, seed {seed}")


@pytest.mark.parametrize("seed", range(24))
def test_scaled_block_fake_quant_and_mx_formats(seed):
    from oracle import awq as oawq
    from oracle import mx

    dtype = (torch.bfloat16, torch.float16, torch.float32)[seed % 3]
    bs = (32, 64, 128)[seed % 3]
    g = torch.Generator().manual_seed(seed + 500)
    w = _wide_case(seed + 500, dtype, bs)
    s = (torch.rand(w.shape[1], generator=g) * 1.5 + 0.25).to(dtype)
    assert_bits_equal(_hip.mul_cols(w.to(DEV), s.to(DEV)).cpu(), w * s, f"column scaling, seed {seed}")
    assert_bits_equal(_hip.scale_block_int_qdq(w.to(DEV), s.to(DEV), bs).cpu(), oawq.int4_block_qdq(w * s, bs),
                      f"scale + INT4 blocks of {bs}, seed {seed}")
    fmt = ("E2M1", "E4M3", "E2M3", "E3M2", "INT8")[seed % 5]
    x = _wide_case(seed + 600, dtype, 32)
    assert_bits_equal(_hip.block_fp_qdq(x.to(DEV), 32, fmt).cpu(), mx.block_fp_fake_quant(x, 32, fmt),
                      f"MX {fmt}, seed {seed}")


@pytest.mark.parametrize("seed", range(12))
def test_search_kernel_on_random_layer_shapes(seed):
    """The one-launch AWQ-lite search against the same step from separate kernels and a library
    GEMM, to the 1e-3 the selected alpha is required to be stable at."""
    import torch.nn.functional as F

    g = torch.Generator().manual_seed(seed + 700)
    tokens = int(torch.randint(1, 513, (1,), generator=g))
    n, k = 128 * int(torch.randint(1, 13, (1,), generator=g)), 128 * int(torch.randint(1, 9, (1,), generator=g))
    n_alpha = int(torch.randint(1, 7, (1,), generator=g))
    block = (32, 64, 128)[seed % 3]
    bits, narrow = ((4, False), (4, True), (8, False))[(seed // 3) % 3]
    w = (0.02 * torch.randn(n, k, generator=g)).to(torch.bfloat16).to(DEV)
    x = (torch.randn(tokens, k, generator=g) * torch.exp(torch.randn(k, generator=g))).to(torch.bfloat16).to(DEV)
    s = torch.exp(0.5 * torch.randn(n_alpha, k, generator=g)).to(torch.bfloat16).to(DEV)
    ref = F.linear(x, w).contiguous()
    xs = _hip.awq_scaled_activations(x, (1 / s.float()).to(torch.bfloat16))
    got = torch.zeros(n_alpha, dtype=torch.float64, device=DEV)
    assert _hip.awq_search_losses_into(xs, w, s.contiguous(), ref, block, bits, False, narrow, got)
    want = torch.zeros(n_alpha, dtype=torch.float64, device=DEV)
    for i in range(n_alpha):
        xi = _hip.mul_cols(x, (1 / s[i].float()).to(torch.bfloat16))
        wq = _hip.scale_block_int_qdq(w, s[i].contiguous(), block, bits, False, narrow)
        _hip.sq_diff_sum_into(F.linear(xi, wq).contiguous(), ref, want[i:i + 1])
    assert torch.allclose(got, want, rtol=1e-3, atol=0), (tokens, n, k, block, bits, got, want)
