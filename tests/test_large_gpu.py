"""Tensors of more than 2^31 elements (4.3 GB of bf16): every element index, byte offset and tile
count past the 32-bit range.  The kernels are element- or block-wise, so the result on the whole
tensor must equal, bit for bit, the results on its two halves (each well inside the 32-bit range,
where the other tests pin the kernels against the CPU restatement); the last rows are also checked
against the restatement directly."""

import pytest
import torch

from conftest import assert_bits_equal
from modelopt_amd import _hip
from oracle import fake_quant, qtensor, reduce

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ROWS, K = (1 << 16) + 32, 1 << 15          # 2,148,532,224 elements
HALF = ROWS // 2


@pytest.fixture(scope="module")
def big():
    g = torch.Generator(device=DEV).manual_seed(3)
    x = torch.empty(ROWS, K, dtype=torch.bfloat16, device=DEV)
    for r0 in range(0, ROWS, 8192):          # filled in slabs: no fp32 temporary of the whole size
        r1 = min(ROWS, r0 + 8192)
        x[r0:r1] = (torch.randn(r1 - r0, K, generator=g, device=DEV) * 0.05).to(torch.bfloat16)
    x[ROWS - 1, K - 1] = 3.0                 # the abs-max sits in the very last element
    yield x
    del x
    torch.cuda.empty_cache()


def _halves_equal(whole, first, second, what):
    n = first.shape[0]
    assert torch.equal(whole[:n].view(torch.uint8), first.view(torch.uint8)), f"{what}: first half"
    assert torch.equal(whole[n:].view(torch.uint8), second.view(torch.uint8)), f"{what}: second half"


def test_abs_max_past_the_32_bit_range(big):
    assert big.numel() > 2**31
    acc = torch.zeros(1, dtype=torch.float32, device=DEV)
    _hip.absmax_into(big, acc, 1, 1, big.numel())
    assert float(acc) == 3.0
    rows = torch.zeros(ROWS, dtype=torch.float32, device=DEV)
    _hip.absmax_into(big, rows, 1, ROWS, K)
    tail = big[-64:].cpu()
    assert_bits_equal(rows[-64:].cpu(), reduce.reduce_amax(tail, axis=[1]).float().reshape(-1), "last rows")
    cols = torch.zeros(K, dtype=torch.float32, device=DEV)
    _hip.absmax_into(big, cols, ROWS, K, 1)
    both = torch.zeros(2, K, dtype=torch.float32, device=DEV)
    _hip.absmax_into(big[:HALF], both[0], HALF, K, 1)
    _hip.absmax_into(big[HALF:], both[1], ROWS - HALF, K, 1)
    assert torch.equal(cols, both.amax(dim=0))
    blocks = torch.zeros(big.numel() // 16, dtype=torch.float32, device=DEV)
    _hip.absmax_into(big, blocks, 1, big.numel() // 16, 16)
    assert_bits_equal(blocks[-64 * K // 16:].cpu(), reduce.reduce_block_amax(tail, {-1: 16}).float().reshape(-1),
                      "last blocks")


def test_fake_quant_past_the_32_bit_range(big):
    amax = torch.tensor(3.0, dtype=torch.bfloat16, device=DEV)
    tail = big[-8:].cpu()
    for what, run, want in (
            ("fp8", lambda t: _hip.fp8_qdq(t, amax, 1, 1, t.numel()), lambda t: fake_quant.fp8_eager(t, amax.cpu())),
            ("int8", lambda t: _hip.int_qdq(t, amax, 1, 1, t.numel(), 8, False, False),
             lambda t: fake_quant.tensor_quant(t, amax.cpu(), 8, False, False)),
            ("nvfp4", lambda t: _hip.nvfp4_qdq(t, amax.float(), 16, 0),
             lambda t: fake_quant.nvfp4_fake_quant(t, amax.cpu(), 16))):
        whole = run(big)
        _halves_equal(whole, run(big[:HALF]), run(big[HALF:]), what)
        assert_bits_equal(whole[-8:].cpu(), want(tail), f"{what}: last rows")
        del whole


def test_quantize_and_pack_past_the_32_bit_range(big):
    amax = torch.tensor(3.0, dtype=torch.float32, device=DEV)
    packed, wsf, wsf2 = _hip.nvfp4_quantize(big, amax, 16)
    pa, wa, _ = _hip.nvfp4_quantize(big[:HALF], amax, 16)
    pb, wb, _ = _hip.nvfp4_quantize(big[HALF:], amax, 16)
    _halves_equal(packed, pa, pb, "codes")
    _halves_equal(wsf, wa, wb, "block scales")
    tail = big[-8:].cpu()
    p_o, w_o, w2_o = qtensor.nvfp4_quantize(tail, 16, None, (amax.cpu() / (6.0 * 448.0)))
    assert_bits_equal(packed[-8:].cpu(), p_o, "codes of the last rows")
    back = _hip.nvfp4_dequantize(packed, wsf, wsf2, 16, torch.bfloat16)
    assert_bits_equal(back[-8:].cpu(), qtensor.nvfp4_dequantize(p_o, w_o, w2_o, 16, tail.shape, torch.bfloat16),
                      "dequantised last rows")
    del packed, wsf, back
    row_scale = torch.full((ROWS,), 3.0 / 448.0, dtype=torch.float32, device=DEV)
    q = _hip.real_quantize(big, row_scale, 1, ROWS, K, torch.float32, _hip.MO_FMT_E4M3)
    _halves_equal(q, _hip.real_quantize(big[:HALF], row_scale[:HALF], 1, HALF, K, torch.float32, _hip.MO_FMT_E4M3),
                  _hip.real_quantize(big[HALF:], row_scale[HALF:], 1, ROWS - HALF, K, torch.float32, _hip.MO_FMT_E4M3),
                  "fp8 storage cast")
    del q
    scales = (torch.rand(K, generator=torch.Generator().manual_seed(1)) + 0.5).to(torch.bfloat16).to(DEV)
    y = _hip.mul_cols(big, scales)
    _halves_equal(y, _hip.mul_cols(big[:HALF], scales), _hip.mul_cols(big[HALF:], scales), "column scaling")
    assert_bits_equal(y[-8:].cpu(), tail * scales.cpu(), "column scaling of the last rows")


def test_block_formats_and_packs_past_the_32_bit_range(big):
    from oracle import awq as oawq
    from oracle import export, mx

    tail = big[-8:].cpu()
    packed, scales = _hip.int4_block_quantize(big.view(-1), 128)
    pa, sa = _hip.int4_block_quantize(big[:HALF].reshape(-1), 128)
    pb, sb = _hip.int4_block_quantize(big[HALF:].reshape(-1), 128)
    _halves_equal(packed, pa, pb, "int4 codes")
    _halves_equal(scales, sa, sb, "int4 scales")
    back = _hip.int4_block_dequantize(packed, scales, 128)
    p_o, s_o = qtensor.int4_quantize(tail, 128)
    assert_bits_equal(back[-8 * K:].cpu().reshape(8, K), qtensor.int4_dequantize(p_o, s_o, 128, tail.shape, torch.bfloat16),
                      "int4 dequantised last rows")
    del packed, scales, back, pa, pb
    ws = torch.full((ROWS, K // 128), 3.0 / 7.0, dtype=torch.float32, device=DEV)
    rows_packed = _hip.int4_pack_rows(big, ws)
    _halves_equal(rows_packed, _hip.int4_pack_rows(big[:HALF], ws[:HALF]), _hip.int4_pack_rows(big[HALF:], ws[HALF:]),
                  "int4 row pairs")
    assert_bits_equal(rows_packed[-4:].cpu(), export.pack_int4_in_uint8(tail, ws[-8:].cpu()), "int4 row pairs, last rows")
    del rows_packed
    y = _hip.block_fp_qdq(big, 32, "E2M1")
    _halves_equal(y, _hip.block_fp_qdq(big[:HALF], 32, "E2M1"), _hip.block_fp_qdq(big[HALF:], 32, "E2M1"), "MXFP4")
    assert_bits_equal(y[-8:].cpu(), mx.block_fp_fake_quant(tail, 32, "E2M1"), "MXFP4 last rows")
    del y
    s = (torch.rand(K, generator=torch.Generator().manual_seed(2)) + 0.5).to(torch.bfloat16).to(DEV)
    y = _hip.scale_block_int_qdq(big, s, 128)
    _halves_equal(y, _hip.scale_block_int_qdq(big[:HALF], s, 128), _hip.scale_block_int_qdq(big[HALF:], s, 128),
                  "scale + INT4 blocks")
    assert_bits_equal(y[-8:].cpu(), oawq.int4_block_qdq(tail * s.cpu(), 128), "scale + INT4 blocks, last rows")
    codes = _hip.cast_fp4(big)
    assert_bits_equal(codes[-8:].cpu(), qtensor.cast_fp4(tail.float()), "E2M1 codes, last rows")
    assert int(codes[-1, -1]) == 5          # 3.0 is ordinal 5
    del codes
    # sums: both halves' sums add up to the whole's (fp64 accumulator / fixed-order fp32 partials)
    loss = torch.zeros(3, dtype=torch.float64, device=DEV)
    _hip.sq_diff_sum_into(big, y, loss[0:1])
    _hip.sq_diff_sum_into(big[:HALF], y[:HALF], loss[1:2])
    _hip.sq_diff_sum_into(big[HALF:], y[HALF:], loss[2:3])
    assert abs(float(loss[0]) - float(loss[1] + loss[2])) <= 1e-9 * float(loss[0]) and float(loss[0]) > 0
    sums = torch.zeros(3, K, dtype=torch.float32, device=DEV)
    _hip.abs_colsum_into(big, sums[0])
    _hip.abs_colsum_into(big[:HALF], sums[1])
    _hip.abs_colsum_into(big[HALF:], sums[2])
    assert torch.allclose(sums[0], sums[1] + sums[2], rtol=1e-5)
    assert torch.allclose(sums[0], big.float().abs().sum(dim=0), rtol=1e-4)


def test_two_rows_of_a_billion_elements(big):
    """The same memory seen as two rows of 2^30 + 2^19 elements: per-row reductions and per-row
    scales with row lengths past 2^30."""
    n = big.numel() // 2
    two = big.view(2, n)
    amax = torch.zeros(2, dtype=torch.float32, device=DEV)
    _hip.absmax_into(two, amax, 1, 2, n)
    want = torch.stack([big[:HALF].abs().amax(), big[HALF:].abs().amax()]).float()
    assert torch.equal(amax, want) and float(amax[1]) == 3.0
    y = _hip.fp8_qdq(two, amax.to(torch.bfloat16), 1, 2, n)
    first = _hip.fp8_qdq(big[:HALF], amax[0:1].to(torch.bfloat16), 1, 1, n)
    second = _hip.fp8_qdq(big[HALF:], amax[1:2].to(torch.bfloat16), 1, 1, n)
    assert torch.equal(y.view(ROWS, K)[:HALF], first) and torch.equal(y.view(ROWS, K)[HALF:], second)
    del y, first, second
    scale = (amax / 127.0).contiguous()
    q = _hip.real_quantize(two, scale, 1, 2, n, torch.float32, _hip.MO_FMT_INT8)
    qa = _hip.real_quantize(big[:HALF], scale[0:1], 1, 1, n, torch.float32, _hip.MO_FMT_INT8)
    qb = _hip.real_quantize(big[HALF:], scale[1:2], 1, 1, n, torch.float32, _hip.MO_FMT_INT8)
    assert torch.equal(q.view(ROWS, K)[:HALF], qa) and torch.equal(q.view(ROWS, K)[HALF:], qb)


@pytest.mark.parametrize("rows,k", [(1 << 24, 8), (8, 1 << 24), (3, (1 << 23) + 8), ((1 << 22) + 3, 24),
                                    (1, 1 << 27), (1 << 27, 1)])
def test_extreme_aspect_ratios(rows, k):
    """Very tall and very wide matrices through the per-row / per-column reductions, the column
    scaling and the per-row fake quant, against the same tensor expressions on the device (a
    maximum and a rounded product have one right answer)."""
    g = torch.Generator(device=DEV).manual_seed(rows % 1000 + k % 1000)
    x = (torch.randn(rows, k, generator=g, device=DEV) * 0.05).to(torch.bfloat16)
    acc = torch.zeros(rows, dtype=torch.float32, device=DEV)
    _hip.absmax_into(x, acc, 1, rows, k)
    assert torch.equal(acc, x.abs().amax(dim=1).float())
    cols = torch.zeros(k, dtype=torch.float32, device=DEV)
    _hip.absmax_into(x, cols, rows, k, 1)
    assert torch.equal(cols, x.abs().amax(dim=0).float())
    s = (torch.rand(k, generator=g, device=DEV) + 0.5).to(torch.bfloat16)
    assert torch.equal(_hip.mul_cols(x, s), x * s)
    row_amax = acc.to(torch.bfloat16)
    row_amax[row_amax == 0] = 1.0
    y = _hip.int_qdq(x, row_amax, 1, rows, k, 8, False, False)
    sample = slice(0, rows, max(1, rows // 64))
    assert_bits_equal(y[sample].cpu(), fake_quant.tensor_quant(x[sample].cpu(), row_amax[sample].cpu().reshape(-1, 1),
                                                              8, False, False), "per-row INT8")
    sums = torch.zeros(k, dtype=torch.float32, device=DEV)
    _hip.abs_colsum_into(x, sums)
    assert torch.allclose(sums, x.float().abs().sum(dim=0), rtol=2e-4, atol=1e-6)
