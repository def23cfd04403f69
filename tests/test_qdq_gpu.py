"""GPU parity of the FP8 / integer quantize-dequantize kernels against the CPU oracle."""

import json
import os

import pytest
import torch

from conftest import GOLDEN, assert_bits_equal
from modelopt_amd import _hip
from oracle import fake_quant, reduce

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.bfloat16, torch.float16, torch.float32]
with open(os.path.join(GOLDEN, "reference_vectors.json")) as f:
    VEC = json.load(f)


def _rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def _c1_tensor(n=1024):
    """The FP8 benchmark input in small: N(0, 0.02) with 0.1 % of entries scaled x50."""
    g = torch.Generator().manual_seed(1)
    x = 0.02 * torch.randn(n, n, generator=g)
    idx = torch.randperm(x.numel(), generator=g)[: x.numel() // 1000]
    x.view(-1)[idx] *= 50
    return x.to(torch.bfloat16)


# ----------------------------------------------------------------------------- FP8
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(64, 256), (33, 47), (5,), (4, 3, 130)])
def test_fp8_per_tensor(dtype, shape):
    x = _rand(shape, dtype, 11)
    amax = reduce.reduce_amax(x)
    y = _hip.fp8_qdq(x.to(DEV), amax.to(DEV), 1, 1, x.numel())
    assert_bits_equal(y.cpu(), fake_quant.fp8_eager(x, amax), str(shape))


def test_fp8_config1_pipeline():
    x = _c1_tensor()
    xd = x.to(DEV)
    acc = torch.zeros(1, dtype=torch.float32, device=DEV)
    _hip.absmax_into(xd, acc, 1, 1, xd.numel())
    amax = acc.reshape(()).to(torch.bfloat16)
    assert_bits_equal(amax.cpu(), reduce.reduce_amax(x), "amax")
    y = _hip.fp8_qdq(xd, amax, 1, 1, xd.numel())
    assert_bits_equal(y.cpu(), fake_quant.fp8_eager(x, reduce.reduce_amax(x)), "qdq")


def test_fp8_clipping_gives_nan_like_cpu_and_saturates_on_request():
    x = _rand((32, 64), torch.bfloat16, 12)
    amax = reduce.reduce_amax(x) * 0.25  # amax smaller than the data
    want = fake_quant.fp8_eager(x, amax)
    assert torch.isnan(want).any()
    y = _hip.fp8_qdq(x.to(DEV), amax.to(DEV), 1, 1, x.numel())
    assert_bits_equal(y.cpu(), want, "NaN on overflow")
    ys = _hip.fp8_qdq(x.to(DEV), amax.to(DEV), 1, 1, x.numel(), saturate=True).cpu()
    assert not torch.isnan(ys).any()
    keep = ~torch.isnan(want)
    assert torch.equal(ys[keep], want[keep])
    assert (ys[~keep].abs().float() == ys.abs().float().max()).all()


def test_fp8_no_amax_is_plain_cast():
    x = _rand((40, 50), torch.float32, 13, scale=30)
    y = _hip.fp8_qdq(x.to(DEV), None, 1, 1, x.numel())
    assert_bits_equal(y.cpu(), fake_quant.fp8_eager(x, None), "cast")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("axis", [0, 1, 2])
def test_fp8_per_channel(dtype, axis):
    x = _rand((6, 16, 24), dtype, 14)
    dims = [d for d in range(3) if d != axis]
    amax = reduce.reduce_amax(x, axis=dims, keepdims=True)
    outer = int(torch.tensor(x.shape[:axis]).prod()) if axis else 1
    inner = int(torch.tensor(x.shape[axis + 1:]).prod()) if axis < 2 else 1
    y = _hip.fp8_qdq(x.to(DEV), amax.reshape(-1).contiguous().to(DEV), outer, x.shape[axis], inner)
    assert_bits_equal(y.cpu(), fake_quant.fp8_eager(x, amax), f"axis {axis}")


def test_fp8_all_bf16_patterns():
    allv = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    for amax in (torch.tensor(1.0), torch.tensor(0.37), torch.tensor(3.0e4)):
        amax = amax.to(torch.bfloat16)
        y = _hip.fp8_qdq(allv.to(DEV), amax.to(DEV), 1, 1, allv.numel())
        assert_bits_equal(y.cpu(), fake_quant.fp8_eager(allv, amax), f"amax {amax.item()}")


# ----------------------------------------------------------------------------- integer
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("num_bits", VEC["int_qdq_grid"]["num_bits"])
@pytest.mark.parametrize("unsigned", VEC["int_qdq_grid"]["unsigned"])
def test_int_per_tensor_and_per_channel(dtype, num_bits, unsigned):
    x = _rand((37, 48), dtype, num_bits)
    if unsigned:
        x = x.abs()
    for narrow in (True, False):
        amax = reduce.reduce_amax(x)
        y = _hip.int_qdq(x.to(DEV), amax.to(DEV), 1, 1, x.numel(), num_bits, unsigned, narrow)
        assert_bits_equal(y.cpu(), fake_quant.tensor_quant(x, amax, num_bits, unsigned, narrow),
                          f"tensor narrow={narrow}")
        a0 = reduce.reduce_amax(x, axis=[1], keepdims=True) * 0.8  # with clipping
        y = _hip.int_qdq(x.to(DEV), a0.reshape(-1).contiguous().to(DEV), 1, 37, 48, num_bits,
                         unsigned, narrow)
        assert_bits_equal(y.cpu(), fake_quant.tensor_quant(x, a0, num_bits, unsigned, narrow),
                          f"axis0 narrow={narrow}")
        a1 = reduce.reduce_amax(x, axis=[0], keepdims=True)
        y = _hip.int_qdq(x.to(DEV), a1.reshape(-1).contiguous().to(DEV), 37, 48, 1, num_bits,
                         unsigned, narrow)
        assert_bits_equal(y.cpu(), fake_quant.tensor_quant(x, a1, num_bits, unsigned, narrow),
                          f"axis1 narrow={narrow}")


def test_int_tiny_amax_channel_is_zero():
    c = VEC["int_tiny_amax"]
    g = torch.Generator().manual_seed(0)
    x = torch.rand(*c["shape"], generator=g)
    amax = torch.tensor(c["amax"])
    y = _hip.int_qdq(x.to(DEV), amax.to(DEV), 2, 3, 4, 8, False, True).cpu()
    assert y[:, 1, :].abs().sum() == 0
    assert_bits_equal(y, fake_quant.tensor_quant(x, amax.reshape(1, 3, 1), 8, False, True), "tiny")


def test_int_dead_channel_follows_the_cpu_path():
    """amax exactly 2^-24 counts as dead (``<=``), a dead channel gives ``rint(x * 0) / 1``: -0.0
    for negative inputs and NaN for infinite ones, as the reference's CPU path does."""
    x = torch.tensor([[0.5, -0.5, float("inf"), -0.0, 1e-9, -1e-9, float("-inf"), 3.0]] * 3).reshape(1, 3, 8)
    amax = torch.tensor([2.0 ** -24, 2.0 ** -23, 1.0])
    want = fake_quant.tensor_quant(x, amax.reshape(1, 3, 1), 8, False, True)
    got = _hip.int_qdq(x.to(DEV), amax.to(DEV), 1, 3, 8, 8, False, True).cpu()
    assert_bits_equal(got, want, "dead channel")
    assert torch.signbit(got[0, 0, 1]) and got[0, 0, 1] == 0      # -0.5 -> -0.0
    assert torch.isnan(got[0, 0, 2]) and torch.isnan(got[0, 0, 6])   # inf * 0
    assert got[0, 1, 0] != 0                                       # 2^-23 is alive


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("k", [256, 200])
def test_int4_static_block128_like_awq_weight(dtype, k):
    x = _rand((24, k), dtype, 21, scale=0.02)
    want = fake_quant.static_block_fake_quant(
        x, 128, lambda x2, amax: fake_quant.tensor_quant(x2, amax, 4, False, False))
    pad = (-k) % 128
    xp = torch.nn.functional.pad(x, (0, pad)).to(DEV).contiguous()
    rows = xp.numel() // 128
    acc = torch.zeros(rows, dtype=torch.float32, device=DEV)
    _hip.absmax_into(xp, acc, 1, rows, 128)
    y = _hip.int_qdq(xp, acc.to(dtype), 1, rows, 128, 4, False, False).reshape(24, k + pad)[:, :k]
    assert_bits_equal(y.cpu().contiguous(), want.contiguous(), "int4 block 128")


def test_inplace_alias():
    x = _rand((128, 64), torch.bfloat16, 30)
    amax = reduce.reduce_amax(x)
    xd = x.to(DEV)
    _hip.int_qdq(xd, amax.to(DEV), 1, 1, xd.numel(), 8, False, True, out=xd)
    assert_bits_equal(xd.cpu(), fake_quant.tensor_quant(x, amax, 8, False, True), "in place")


@pytest.mark.parametrize("num_bits", [(4, 3), 8])
@pytest.mark.parametrize("shape,blocks", [((256, 384), {-1: 128, -2: 128}), ((8, 64), {-1: 32, -2: 4}),
                                           ((100, 72), {-1: 16, -2: 8})])
def test_two_axis_block_fake_quant_through_the_quantizer(num_bits, shape, blocks):
    """2-D tiles (the FP8 128 x 128 weight-only config and smaller ones, with padding): the
    quantizer reshapes to [N/b0, b0, K/b1, b1] and its amax keeps dims 0 and 2 -- two runs of
    dims, which the kernels see through a transposing copy.  Against the same reshape on the CPU
    (reference nn/modules/tensor_quantizer.py:755-800)."""
    import torch.nn.functional as F

    from modelopt_amd.torch.quantization.config import QuantizerAttributeConfig
    from modelopt_amd.torch.quantization.nn import TensorQuantizer

    x = _rand(shape, torch.bfloat16, 31)
    q = TensorQuantizer(QuantizerAttributeConfig(num_bits=num_bits, block_sizes=blocks)).to(DEV)
    q.enable_calib(); q.disable_quant()
    q(x.to(DEV))
    q.load_calib_amax()
    q.enable_quant(); q.disable_calib()
    got = q(x.to(DEV)).cpu()

    b0, b1 = blocks[-2], blocks[-1]
    pad = F.pad(x, (0, -shape[1] % b1, 0, -shape[0] % b0))
    tiles = pad.reshape(pad.shape[0] // b0, b0, pad.shape[1] // b1, b1)
    amax = reduce.reduce_amax(tiles, axis=[1, 3], keepdims=True, squeeze_scalar=False)
    assert_bits_equal(q.amax.cpu(), amax, "tile amax")
    if num_bits == 8:
        want = fake_quant.tensor_quant(tiles, amax, 8, False, False)
    else:
        want = fake_quant.fp8_eager(tiles, amax)
    want = want.reshape(pad.shape)[: shape[0], : shape[1]]
    assert_bits_equal(got, want, "2-D block fake quant")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("lead,rows,cols,br,bc", [((), 256, 384, 128, 128), ((), 192, 320, 64, 32),
                                                   ((), 48, 64, 16, 8), ((3,), 128, 256, 64, 128),
                                                   ((), 1024, 4096, 128, 128)])
def test_two_dimensional_blocks(dtype, lead, rows, cols, br, bc, monkeypatch):
    """An amax per (br x bc) block of a matrix -- the reshape ``[R, br, C, bc]`` with the amax on
    dims 0 and 2 that block sizes on the last two dims set up (reference: tensor_quantizer.py
    :755-782) -- through the block abs-max and the FP8 / INT fake quant without a transposed copy:
    against the CPU restatement on the same 4-D view, and the binding's refusals."""
    from modelopt_amd.torch.quantization import kernels

    g = torch.Generator().manual_seed(rows + cols + br)
    x = (torch.randn(*lead, rows, cols, generator=g) * 0.05).to(dtype)
    x.view(-1)[::97] *= 8
    x[..., :br, :bc] = 0.0                                     # an all-zero block
    x4 = x.reshape(*lead, rows // br, br, cols // bc, bc)
    dims = (x4.dim() - 3, x4.dim() - 1)
    taken = []
    for name in ("absmax_blocks2d_into", "fp8_qdq_blocks2d", "int_qdq_blocks2d"):
        real = getattr(_hip, name)
        monkeypatch.setattr(_hip, name, lambda *a, _real=real, _name=name: taken.append(_name) or _real(*a))
    want_amax = reduce.reduce_amax(x4, axis=list(dims))
    got_amax = kernels.reduce_amax_gpu(x4.to(DEV), dims)
    assert got_amax.shape == want_amax.shape
    assert_bits_equal(got_amax.cpu(), want_amax, "block abs-max")
    amax = want_amax.clone()
    amax[amax == 0] = 1.0
    clipped = amax * 0.5                                       # half of the blocks' range clips
    for a, what in ((amax, "amax"), (clipped, "half the amax")):
        got = kernels.fake_quant_fp8(x4.to(DEV), a.to(DEV), saturate=True)
        want = fake_quant.fp8_eager(x4.clamp(-a, a) if a is clipped else x4, a)
        assert_bits_equal(got.cpu(), want, f"fp8, {what}")
        for bits, narrow in ((8, False), (4, True)):
            got = kernels.fake_quant_int(x4.to(DEV), a.to(DEV), bits, False, narrow)
            assert_bits_equal(got.cpu(), fake_quant.tensor_quant(x4, a, bits, False, narrow), f"int{bits}, {what}")
    assert taken == ["absmax_blocks2d_into"] + ["fp8_qdq_blocks2d", "int_qdq_blocks2d", "int_qdq_blocks2d"] * 2
    # what the kernels do not take goes the long way round and gives the same
    odd = x4[..., 1:].contiguous() if bc > 8 else None
    if odd is not None:
        a_odd = reduce.reduce_amax(odd, axis=list(dims))
        a_odd[a_odd == 0] = 1.0
        assert_bits_equal(kernels.fake_quant_int(odd.to(DEV), a_odd.to(DEV), 8, False, False).cpu(),
                          fake_quant.tensor_quant(odd, a_odd, 8, False, False), "block width not a multiple of 8")
