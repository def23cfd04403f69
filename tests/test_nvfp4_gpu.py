"""GPU parity of the NVFP4 kernels (through the C ABI) against the CPU oracle."""

import pytest
import torch

from conftest import assert_bits_equal
from modelopt_amd import _hip
from oracle import fake_quant, qtensor, reduce

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _rand(shape, dtype, seed, scale=0.02):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(shape, generator=g)).to(dtype)


def _gpu_amax(xd):
    acc = torch.zeros(1, dtype=torch.float32, device=xd.device)
    _hip.absmax_into(xd, acc, 1, 1, xd.numel())
    return acc


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape,bs", [((64, 256), 16), ((33, 48), 16), ((7, 40), 16),
                                      ((5, 24), 8), ((16, 96), 32), ((3, 5, 64), 16),
                                      ((1024, 4096), 16)])
def test_quantize_pack_matches_oracle(dtype, shape, bs):
    x = _rand(shape, dtype, seed=hash((shape, bs)) % 1000)
    packed_o, wsf_o, wsf2_o = qtensor.nvfp4_quantize(x, bs)
    xd = x.to(DEV)
    amax = _gpu_amax(xd)
    assert_bits_equal(amax.cpu().reshape(()).to(dtype), reduce.reduce_amax(x), "amax")
    packed, wsf, wsf2 = _hip.nvfp4_quantize(xd, amax.reshape(()), bs)
    assert_bits_equal(wsf2.cpu(), wsf2_o, "wsf2")
    assert_bits_equal(wsf.cpu(), wsf_o, "wsf")
    assert_bits_equal(packed.cpu(), packed_o, "packed")
    # dequant round trip
    y = _hip.nvfp4_dequantize(packed, wsf, wsf2, bs, dtype)
    y_o = qtensor.nvfp4_dequantize(packed_o, wsf_o, wsf2_o, bs, packed_o.shape[:-1] + (packed_o.shape[-1] * 2,), dtype)
    assert_bits_equal(y.cpu(), y_o, "dequant")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("shape", [(64, 256), (33, 40), (512, 1024)])
def test_fake_quant_matches_oracle(dtype, mode, shape):
    x = _rand(shape, dtype, seed=7, scale=1.0)
    amax = reduce.reduce_amax(x)
    xd = x.to(DEV)
    y = _hip.nvfp4_qdq(xd, amax.to(DEV), 16, mode)
    if mode == 0:
        y_o = fake_quant.nvfp4_fake_quant(x, amax, 16)
    else:
        p, wsf, wsf2 = qtensor.nvfp4_quantize(x, 16)
        kp = p.shape[-1] * 2
        y_o = qtensor.nvfp4_dequantize(p, wsf, wsf2, 16, (shape[0], kp), dtype)[:, : shape[1]]
    assert_bits_equal(y.cpu(), y_o.contiguous(), f"qdq mode {mode}")


def _edge_tensor():
    """bf16 [rows, 64] rows built to hit every E2M1 tie, zero blocks, signed zeros, tiny values."""
    rows = []
    ties = [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0]
    base = torch.tensor(ties + [-t for t in ties])
    for s in (1.0, 0.5, 0.0234375, 3.0, 448.0, 2.0 ** -20):
        rows.append(torch.cat([base * s, (base + 0.1) * s, (base - 0.1) * s, base * s * 1.5]))
    rows.append(torch.zeros(64))
    z = torch.zeros(64); z[0] = -0.0; z[5] = 1e-30; z[6] = -1e-30; z[17] = 6.0; z[18] = -2.0 ** -126
    rows.append(z)
    z2 = torch.full((64,), -0.0); rows.append(z2)
    return torch.stack(rows).to(torch.bfloat16)


def test_edge_cases_match_oracle():
    x = _edge_tensor()
    for bs in (16,):
        po, wo, w2o = qtensor.nvfp4_quantize(x, bs)
        xd = x.to(DEV)
        p, w, w2 = _hip.nvfp4_quantize(xd, _gpu_amax(xd).reshape(()), bs)
        assert_bits_equal(w.cpu(), wo, "wsf")
        assert_bits_equal(p.cpu(), po, "packed")


def test_all_zero_tensor_matches_x86_nan_sign():
    x = torch.zeros(4, 32, dtype=torch.bfloat16)
    po, wo, w2o = qtensor.nvfp4_quantize(x, 16)
    xd = x.to(DEV)
    p, w, w2 = _hip.nvfp4_quantize(xd, _gpu_amax(xd).reshape(()), 16)
    assert_bits_equal(w.cpu(), wo, "wsf")
    assert_bits_equal(p.cpu(), po, "packed")


@pytest.mark.parametrize("special", [float("nan"), float("inf"), -float("inf")])
def test_nonfinite_inputs(special):
    x = _rand((8, 64), torch.bfloat16, 3)
    x[1, 3] = special
    amax = torch.tensor(0.1, dtype=torch.bfloat16)  # a calibrated amax, as the export path passes
    wsf2 = amax.float() / (6.0 * 448.0)
    wo, _ = qtensor.nvfp4_block_scales(x, 16, wsf2)
    po, _, _ = qtensor.nvfp4_quantize(x, 16, wo, wsf2)
    xd = x.to(DEV)
    p, w, w2 = _hip.nvfp4_quantize(xd, amax.float().to(DEV), 16)
    assert_bits_equal(w.cpu(), wo, "wsf")
    assert_bits_equal(p.cpu(), po, "packed")


def test_all_bf16_patterns_against_oracle():
    """Every bf16 bit pattern as an element, in blocks whose scale is set by a pilot value."""
    allv = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    finite = allv[torch.isfinite(allv.float())]
    finite = finite[: finite.numel() // 15 * 15].reshape(-1, 15)
    for pilot in (1.0, 0.013, 300.0):
        col = torch.full((finite.shape[0], 1), pilot, dtype=torch.bfloat16)
        x = torch.cat([col, finite], dim=1).contiguous()
        # clip magnitudes so the pilot stays the block maximum for most rows; others are fine too
        amax = torch.tensor(pilot * 4, dtype=torch.bfloat16)
        wsf2 = amax.float() / (6.0 * 448.0)
        wo, _ = qtensor.nvfp4_block_scales(x, 16, wsf2)
        po, _, _ = qtensor.nvfp4_quantize(x, 16, wo, wsf2)
        xd = x.to(DEV)
        p, w, w2 = _hip.nvfp4_quantize(xd, amax.float().to(DEV), 16)
        assert_bits_equal(w.cpu(), wo, f"wsf pilot={pilot}")
        assert_bits_equal(p.cpu(), po, f"packed pilot={pilot}")


def test_fast_path_equals_exact_division_on_large_input():
    """Same GPU, same input: multiply-and-verify codes == literal per-element division codes."""
    g = torch.Generator(device=DEV).manual_seed(11)
    x = (0.02 * torch.randn(8192, 8192, generator=g, device=DEV)).to(torch.bfloat16)
    amax = _gpu_amax(x).reshape(())
    p_fast, w_fast, _ = _hip.nvfp4_quantize(x, amax, 16)
    p_exact, w_exact, _ = _hip.nvfp4_quantize(x, amax, 16, flags=_hip.MO_FLAG_FORCE_EXACT)
    assert torch.equal(w_fast.view(torch.uint8), w_exact.view(torch.uint8))
    assert torch.equal(p_fast, p_exact)
    # and against the oracle on a slice the CPU finishes quickly
    po, wo, _ = qtensor.nvfp4_quantize(x[:512].cpu(), 16, wsf2=(amax.cpu() / 2688.0))
    assert_bits_equal(p_fast[:512].cpu(), po, "packed slice")


@pytest.mark.parametrize("dtype,block", [(torch.bfloat16, 16), (torch.bfloat16, 32),
                                         (torch.float16, 16), (torch.float32, 8)])
def test_block_scale_overflow_follows_the_flag(dtype, block):
    """A per-tensor amax below the real maximum (awq_clip's doing, TQ/model_calib.py:869-876)
    pushes block scales past E4M3's range: by default the scale byte is the NaN that torch's
    cast gives (TQ/qtensor/nvfp4_tensor.py:84-91); with MO_FLAG_SATURATE_BLOCK_SCALE it is 448,
    and the codes follow from that scale.  Single-tensor (tile and generic kernels) and
    multi-tensor launches."""
    x = _rand((256, 512), dtype, 77)
    amax = reduce.reduce_amax(x).float() * 0.4
    wsf2 = amax / 2688.0
    raw, _ = qtensor.nvfp4_block_scales(x, block, wsf2, keep_high_precision=True)
    assert bool((raw > 464).any()) and bool((raw < 400).any())
    xd = x.to(DEV)
    for saturate in (0, 1):
        wo = (raw.clamp(max=448.0) if saturate else raw).to(torch.float8_e4m3fn)
        po, _, _ = qtensor.nvfp4_quantize(x, block, wo, wsf2)
        flags = _hip.MO_FLAG_SATURATE_BLOCK_SCALE if saturate else 0
        p, w, _ = _hip.nvfp4_quantize(xd, amax.to(DEV), block, flags=flags)
        if dtype == torch.bfloat16 and block == 16:
            mp, mw, _ = _hip.Nvfp4QuantizePlan([xd], amax.to(DEV).reshape(1), flags=flags).run()
        assert_bits_equal(w.cpu(), wo, f"wsf saturate={saturate}")
        assert bool(torch.isnan(w.float()).any()) == (not saturate)
        ok = ~torch.isnan(wo.float()).repeat_interleave(block // 2, dim=-1)   # NaN scale: codes of NaN
        assert torch.equal(p.cpu()[ok], po[ok])
        if dtype == torch.bfloat16 and block == 16:
            assert torch.equal(mp[0], p) and torch.equal(mw[0].view(torch.uint8), w.view(torch.uint8))


def test_multi_tensor_plan_matches_single_calls():
    shapes = [(256, 512), (64, 4096), (1000, 48), (3, 16)]
    xs = [_rand(s, torch.bfloat16, 20 + i).to(DEV) for i, s in enumerate(shapes)]
    aplan = _hip.AbsmaxPlan(xs)
    acc = aplan.run().clone()
    for i, x in enumerate(xs):
        assert_bits_equal(acc[i].cpu(), _gpu_amax(x).cpu().reshape(()), f"amax {i}")
    qplan = _hip.Nvfp4QuantizePlan(xs, acc)
    packed, wsf, wsf2 = qplan.run()
    for i, x in enumerate(xs):
        p, w, w2 = _hip.nvfp4_quantize(x, acc[i], 16)
        assert torch.equal(packed[i], p) and torch.equal(wsf[i].view(torch.uint8), w.view(torch.uint8))
        assert_bits_equal(wsf2[i].cpu(), w2.cpu(), "wsf2")
        po, wo, w2o = qtensor.nvfp4_quantize(x.cpu(), 16)
        assert_bits_equal(packed[i].cpu(), po, f"packed {i}")
        assert_bits_equal(wsf[i].cpu(), wo, f"wsf {i}")


@pytest.mark.parametrize("mode", [0, 1])
def test_fake_quant_edge_cases_and_all_patterns(mode):
    def want(x, amax):
        if mode == 0:
            return fake_quant.nvfp4_fake_quant(x, amax, 16)
        wsf2 = amax.float() / 2688.0
        wsf, _ = qtensor.nvfp4_block_scales(x, 16, wsf2)
        p, _, _ = qtensor.nvfp4_quantize(x, 16, wsf, wsf2)
        return qtensor.nvfp4_dequantize(p, wsf, wsf2, 16, x.shape, x.dtype)

    x = _edge_tensor()
    amax = reduce.reduce_amax(x)
    assert_bits_equal(_hip.nvfp4_qdq(x.to(DEV), amax.to(DEV), 16, mode).cpu(), want(x, amax), "edge tensor")
    allv = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    finite = allv[torch.isfinite(allv.float())]
    finite = finite[: finite.numel() // 15 * 15].reshape(-1, 15)
    for pilot in (1.0, 0.013):
        col = torch.full((finite.shape[0], 1), pilot, dtype=torch.bfloat16)
        x = torch.cat([col, finite], dim=1).contiguous()
        amax = torch.tensor(pilot * 4, dtype=torch.bfloat16)
        assert_bits_equal(_hip.nvfp4_qdq(x.to(DEV), amax.to(DEV), 16, mode).cpu(), want(x, amax),
                          f"all patterns pilot={pilot}")


def test_dequantize_every_code_and_scale():
    codes = torch.arange(256, dtype=torch.uint8).repeat(8).reshape(-1, 8)          # 256 blocks
    scales = torch.arange(256, dtype=torch.uint8)[: codes.shape[0]].view(torch.float8_e4m3fn).reshape(-1, 1)
    wsf2 = torch.tensor(0.37)
    for dtype in (torch.bfloat16, torch.float16, torch.float32):
        y = _hip.nvfp4_dequantize(codes.to(DEV), scales.to(DEV), wsf2.to(DEV), 16, dtype)
        y_o = qtensor.nvfp4_dequantize(codes, scales, wsf2, 16, (codes.shape[0], 16), dtype)
        assert_bits_equal(y.cpu(), y_o, str(dtype))


@pytest.mark.parametrize("shape", [(4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336)])
def test_llama3_8b_weight_shapes_against_c_restatement(shape):
    """Full-size Llama-3-8B linear weights: abs-max, global scale, block scales, packed codes and
    the dequantised tensor, bit for bit against the C restatement of the reference arithmetic."""
    from oracle import cref

    g = torch.Generator(device=DEV).manual_seed(shape[0] * 31 + shape[1])
    xd = (torch.randn(shape, generator=g, device=DEV) * 0.02).to(torch.bfloat16)
    acc = torch.zeros(1, dtype=torch.float32, device=DEV)
    _hip.absmax_into(xd, acc, 1, 1, xd.numel())
    packed, wsf, wsf2 = _hip.nvfp4_quantize(xd, acc.reshape(()), 16)
    y = _hip.nvfp4_dequantize(packed, wsf, wsf2, 16, torch.bfloat16)
    x = xd.cpu()
    assert float(acc) == cref.absmax(x)
    p_c, w_c, w2_c = cref.nvfp4_quantize(x, 16)
    assert float(wsf2) == float(w2_c)
    assert torch.equal(wsf.cpu().view(torch.uint8), w_c.view(torch.uint8))
    assert torch.equal(packed.cpu(), p_c)
    y_c = cref.nvfp4_dequantize(p_c, w_c, w2_c, 16, torch.bfloat16)
    assert torch.equal(y.cpu().view(torch.int16), y_c.view(torch.int16))


LLAMA3_8B_LAYER = [("q", 4096, 4096), ("k", 1024, 4096), ("v", 1024, 4096), ("o", 4096, 4096),
                   ("gate", 14336, 4096), ("up", 14336, 4096), ("down", 4096, 14336)]


def test_two_full_llama3_8b_layers_through_the_multi_tensor_launches():
    """Two complete Llama-3-8B decoder layers (14 weights, all seven shapes) through the
    multi-tensor abs-max and quantize+pack launches that the benchmark times: per-tensor amax,
    global scale, every block scale and every packed code bit for bit against the C restatement."""
    from oracle import cref

    g = torch.Generator(device=DEV).manual_seed(2024)
    xs = [(torch.randn((n, k), generator=g, device=DEV) * 0.02).to(torch.bfloat16)
          for _layer in range(2) for _name, n, k in LLAMA3_8B_LAYER]
    acc = _hip.AbsmaxPlan(xs).run().clone()
    packed, wsf, wsf2 = _hip.Nvfp4QuantizePlan(xs, acc).run()
    torch.cuda.synchronize()
    for i, xd in enumerate(xs):
        x = xd.cpu()
        what = f"tensor {i} {tuple(x.shape)}"
        assert float(acc[i]) == cref.absmax(x), what
        p_c, w_c, w2_c = cref.nvfp4_quantize(x, 16)
        assert float(wsf2[i]) == float(w2_c), what
        assert torch.equal(wsf[i].cpu().view(torch.uint8), w_c.view(torch.uint8)), what
        assert torch.equal(packed[i].cpu(), p_c), what


def test_elements_on_rounding_boundaries_of_e2m1():
    """Blocks whose quotients x / s sit exactly on, one bf16 step below and one step above every
    rounding boundary of E2M1 (0.25, 0.75, ..., 5): the quotient has to be the correctly rounded
    one for these, and ties go to the even code as in the oracle."""
    bounds = [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0]
    rows = []
    for scale_exp in (-6, -3, 0, 2):
        for sign in (1.0, -1.0):
            vals = []
            for b in bounds:
                t = torch.tensor(b * 2.0 ** scale_exp, dtype=torch.bfloat16)
                bits = t.view(torch.int16)
                vals += [t, (bits - 1).view(torch.bfloat16), (bits + 1).view(torch.bfloat16)]
            blk = torch.stack(vals[:15] + [torch.tensor(6.0 * 2.0 ** scale_exp, dtype=torch.bfloat16)])
            rows.append(sign * blk.float())
            blk2 = torch.stack(vals[6:21] + [torch.tensor(6.0 * 2.0 ** scale_exp, dtype=torch.bfloat16)])
            rows.append(sign * blk2.float())
    x = torch.stack(rows).to(torch.bfloat16).reshape(4, -1)          # 16 blocks of 16
    x = torch.cat([x, _rand((60, x.shape[1]), torch.bfloat16, seed=11)])   # plus ordinary rows
    # the global scale that puts the values exactly on the boundaries, and one slightly off
    for w2 in (torch.tensor(24.0 / 2688.0), torch.tensor(0.0091)):
        w2 = w2.to(torch.float32)
        po, wo, _ = qtensor.nvfp4_quantize(x, 16, wsf2=w2)
        packed, wsf, _ = _hip.nvfp4_quantize(x.to(DEV), w2.to(DEV), 16, amax_is_wsf2=True)
        p_exact, w_exact, _ = _hip.nvfp4_quantize(x.to(DEV), w2.to(DEV), 16, amax_is_wsf2=True,
                                                  flags=_hip.MO_FLAG_FORCE_EXACT)
        assert torch.equal(packed, p_exact) and torch.equal(wsf.view(torch.uint8), w_exact.view(torch.uint8))
        assert_bits_equal(packed.cpu(), po, "codes on rounding boundaries")
        assert_bits_equal(wsf.cpu(), wo, "scales on rounding boundaries")


def test_plans_refuse_inputs_that_were_reallocated():
    """The job tables hold raw addresses: a parameter that is given new memory after the plan was
    built (``param.data = ...``) makes ``run`` raise instead of reading the old memory, which the
    plan keeps alive."""
    ws = [torch.nn.Parameter(_rand((64, 256), torch.bfloat16, seed=i).to(DEV), requires_grad=False) for i in range(3)]
    aplan = _hip.AbsmaxPlan(ws)
    acc = aplan.run().clone()
    qplan = _hip.Nvfp4QuantizePlan(ws, acc)
    before = [p.clone() for p in qplan.run()[0]]
    ws[1].data = ws[1].data.clone() * 2
    with pytest.raises(RuntimeError, match="reallocated"):
        aplan.run()
    with pytest.raises(RuntimeError, match="reallocated"):
        qplan.run()
    after = qplan.run(verify=False)[0]      # still the old memory, still valid
    assert all(torch.equal(a, b) for a, b in zip(before, after))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_stacked_expert_weights_with_one_global_scale_each(dtype):
    """A 3-D (experts, output, input) weight whose global scale is given per expert, shaped
    ``[E, 1, 1]`` so that it broadcasts (qtensor/nvfp4_tensor.py:199-203 with the scales of
    export/quant_utils.py:822-829): block scales, codes, the dequantised tensor and the export
    cast against the same expressions on the CPU."""
    from modelopt_amd.torch.export.quant_utils import to_quantized_weight
    from modelopt_amd.torch.quantization.qtensor import NVFP4QTensor

    g = torch.Generator().manual_seed(31)
    w = (torch.randn((3, 32, 80), generator=g) * torch.tensor([0.02, 0.5, 3.0]).view(-1, 1, 1)).to(dtype)
    wsf2 = (w.abs().amax(dim=(1, 2)).float() / (6.0 * 448.0)).view(-1, 1, 1)
    want_packed, want_wsf, _ = qtensor.nvfp4_quantize(w, 16, None, wsf2)
    dev = w.to(DEV)
    scales, _ = NVFP4QTensor.get_weights_scaling_factor(dev, 16, wsf2.to(DEV))
    assert_bits_equal(scales.cpu().view(torch.uint8), want_wsf.view(torch.uint8), "block scales")
    q, got_wsf, got_wsf2 = NVFP4QTensor.quantize(dev, 16, None, wsf2.to(DEV))
    assert got_wsf2.shape == (3, 1, 1)
    assert_bits_equal(got_wsf.cpu().view(torch.uint8), want_wsf.view(torch.uint8), "block scales from quantize")
    assert_bits_equal(q._quantized_data.cpu(), want_packed, "codes")
    back = q.dequantize(scale=got_wsf, double_scale=got_wsf2, block_sizes={-1: 16})
    assert_bits_equal(back.cpu(), qtensor.nvfp4_dequantize(want_packed, want_wsf, wsf2, 16, w.shape, dtype), "dequantised")
    cast = to_quantized_weight(dev, scales, "nvfp4", wsf2.reshape(-1).to(DEV), block_size=16)
    assert_bits_equal(cast.cpu(), want_packed, "export cast with a 1-D global scale")


@pytest.mark.parametrize("values", [
    None,
    [[0.25, 0.75, 1.25], [1.75, 2.5, 3.5]],
    [[0.1, 2.5, 1.0, 4.8], [1.5, 1.25, 3.25, 5.0]],
    [[0, 0.75, 1.25], [1.75, 2.5, 5.5]],
    [[-0.25, -0.75, -1.25], [-1.75, -2.5, -3.5]],
    [[-0.1, -2.5, -1.0, -4.8], [-1.5, -1.25, -3.25, -5.0]],
    [[0, -0.75, -1.25], [-1.75, -2.5, -5.5]],
    [[float("nan"), float("inf"), -float("inf"), -0.0, 1e-30, -1e-30, 6.0, -7.5, 1e30]],
])
def test_cast_fp4_codes(values):
    """``NVFP4QTensor._cast_fp4`` on the inputs of the reference's equivalence test
    (tests/gpu/torch/quantization/test_qtensor_cuda.py:399-441) plus special values, a ragged
    length and the 16-bit types, against the CPU restatement of nvfp4_tensor.py:120-140."""
    from modelopt_amd.torch.quantization.qtensor import NVFP4QTensor

    if values is None:
        x = torch.randn((32, 16), generator=torch.Generator().manual_seed(0)) * 3
    else:
        x = torch.tensor(values, dtype=torch.float32)
    got = NVFP4QTensor._cast_fp4(x.to(DEV))
    assert got.dtype == torch.uint8 and got.shape == x.shape
    assert torch.equal(got.cpu(), qtensor.cast_fp4(x.clone()))
    flat = torch.randn(1027, generator=torch.Generator().manual_seed(1)) * 4
    flat[::50] = torch.tensor([0.75, 1.75, 3.5, 0.25, 1.25, 2.5, 5.0]).repeat(3)
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        v = flat.to(dtype)
        assert torch.equal(NVFP4QTensor._cast_fp4(v.to(DEV)).cpu(), qtensor.cast_fp4(v.float())), dtype
        odd = v[1:]                                      # byte stores that are not word aligned
        assert torch.equal(_hip.cast_fp4(odd.to(DEV).contiguous()).cpu(), qtensor.cast_fp4(odd.float()))
    assert NVFP4QTensor.get_e2m1_bounds(DEV).tolist() == [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5]
    assert NVFP4QTensor.get_e2m1_values(DEV)[9].item() == -0.5
