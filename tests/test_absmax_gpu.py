"""GPU parity of the abs-max kernels (through the C ABI) against the CPU oracle."""

import pytest
import torch

from conftest import assert_bits_equal
from modelopt_amd import _hip
from oracle import reduce

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.bfloat16, torch.float16, torch.float32]


def _rand(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * 3).to(dtype)


def _gpu_reduce(x, outer, axis, inner):
    acc = torch.zeros(axis, dtype=torch.float32, device=DEV)
    _hip.absmax_into(x.to(DEV).contiguous(), acc, outer, axis, inner)
    return acc.cpu()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [1, 7, 8, 1000, 4096 * 33 + 5, 1 << 22])
def test_per_tensor(dtype, n):
    x = _rand((n,), dtype, n % 97)
    got = _gpu_reduce(x, 1, 1, n).reshape(()).to(dtype)
    assert_bits_equal(got, reduce.reduce_amax(x), f"n={n}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(5, 16), (300, 128), (64, 4096), (3, 100000), (1000, 7), (2, 9)])
def test_per_row_keep_axis0(dtype, shape):
    x = _rand(shape, dtype, 1)
    got = _gpu_reduce(x, 1, shape[0], shape[1]).to(dtype)
    assert_bits_equal(got, reduce.reduce_amax(x, axis=[1], keepdims=False), str(shape))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(5, 16), (300, 128), (4096, 512), (77, 13), (8192, 8)])
def test_per_column_keep_last_axis(dtype, shape):
    x = _rand(shape, dtype, 2)
    got = _gpu_reduce(x, shape[0], shape[1], 1).to(dtype)
    assert_bits_equal(got, reduce.reduce_amax(x, axis=[0], keepdims=False), str(shape))


@pytest.mark.parametrize("dtype", DTYPES)
def test_middle_axis(dtype):
    x = _rand((6, 8, 33, 16), dtype, 3)  # e.g. [B, H, S, D] keeping H
    got = _gpu_reduce(x, 6, 8, 33 * 16).to(dtype)
    assert_bits_equal(got, reduce.reduce_amax(x, axis=[0, 2, 3], keepdims=False), "axis 1")


def test_block_amax_equals_reduce_block_amax():
    x = _rand((48, 256), torch.bfloat16, 4)
    got = _gpu_reduce(x, 1, 48 * 16, 16).to(torch.bfloat16).reshape(48, 16)
    assert_bits_equal(got, reduce.reduce_block_amax(x, {-1: 16}), "block 16")
    got = _gpu_reduce(x, 1, 48 * 2, 128).to(torch.bfloat16).reshape(48, 2)
    assert_bits_equal(got, reduce.reduce_block_amax(x, {-1: 128}), "block 128")


def test_running_max_semantics_and_nan():
    a, b = _rand((1000,), torch.bfloat16, 5), _rand((1000,), torch.bfloat16, 6) * 2
    acc = torch.zeros(1, dtype=torch.float32, device=DEV)
    _hip.absmax_into(a.to(DEV), acc, 1, 1, 1000)
    _hip.absmax_into(b.to(DEV), acc, 1, 1, 1000)
    want = torch.max(reduce.reduce_amax(a), reduce.reduce_amax(b))
    assert_bits_equal(acc.cpu().reshape(()).to(torch.bfloat16), want, "running max")
    c = a.clone(); c[17] = float("nan")
    assert torch.isnan(_gpu_reduce(c, 1, 1, 1000)).all()
    assert torch.isnan(reduce.reduce_amax(c))
    d = a.clone(); d[3] = -float("inf")
    assert torch.isinf(_gpu_reduce(d, 1, 1, 1000)).all()


def test_unaligned_view():
    x = _rand((4099,), torch.bfloat16, 7).to(DEV)
    v = x[1:]  # 2-byte offset: not 16-byte aligned
    acc = torch.zeros(1, dtype=torch.float32, device=DEV)
    _hip.absmax_into(v, acc, 1, 1, v.numel())
    assert_bits_equal(acc.cpu().reshape(()).to(torch.bfloat16), reduce.reduce_amax(v.cpu()), "offset view")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(64, 8), (65, 2048), (1000, 4096), (333, 520), (8192, 8192), (4097, 2056)])
def test_per_column_staged_path(dtype, shape):
    """Tall matrices take the two-pass route (row slabs -> workspace -> columns); ragged row
    counts, both column widths (LDS and wide kernel), NaN / inf columns, and a warm accumulator."""
    x = _rand(shape, dtype, 11)
    x[shape[0] // 2, 3] = float("nan")
    x[shape[0] - 1, 5] = float("-inf")
    want = reduce.reduce_amax(x, axis=[0], keepdims=False)
    xd = x.to(DEV)
    acc = torch.zeros(shape[1], dtype=torch.float32, device=DEV)
    _hip.absmax_into(xd, acc, shape[0], shape[1], 1)
    assert_bits_equal(acc.cpu().to(dtype), want, f"fresh {shape}")
    # the single-pass entry point gives the same accumulator
    direct = torch.zeros(shape[1], dtype=torch.float32, device=DEV)
    _hip.call("mo_absmax", xd, xd.data_ptr(), shape[0], shape[1], 1, _hip.dtype_code(dtype),
              direct.data_ptr(), _hip._stream(xd))
    assert_bits_equal(acc.cpu(), direct.cpu(), f"staged vs direct {shape}")
    # running maximum: a second, smaller tensor leaves it alone; a larger one raises it
    _hip.absmax_into((xd * 0.5).nan_to_num(0.0, 0.0, 0.0), acc, shape[0], shape[1], 1)
    assert_bits_equal(acc.cpu().to(dtype), want, f"warm, smaller {shape}")
    big = _rand(shape, dtype, 12) * 4
    _hip.absmax_into(big.to(DEV), acc, shape[0], shape[1], 1)
    want2 = torch.maximum(want.float(), reduce.reduce_amax(big, axis=[0], keepdims=False).float())
    want2[3] = float("nan")
    assert_bits_equal(acc.cpu(), want2, f"warm, larger {shape}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n0,n1", [(1, 1), (8192 * 3 + 5, 7), (16 * 8 * 512 * 128, 16 * 8 * 512 * 128), (1000, 1 << 20)])
def test_pair_of_tensors_in_one_launch(dtype, n0, n1):
    """mo_absmax_pair: each tensor into its own running maximum, NaN propagating like torch.max."""
    x0, x1 = _rand((n0,), dtype, 5), _rand((n1,), dtype, 6)
    acc0 = torch.zeros(1, dtype=torch.float32, device=DEV)
    acc1 = torch.full((1,), 2.5, dtype=torch.float32, device=DEV)          # a running maximum
    assert _hip.absmax_pair_into(x0.to(DEV), acc0, x1.to(DEV), acc1)
    assert_bits_equal(acc0.cpu().reshape(()).to(dtype), reduce.reduce_amax(x0), "first")
    want1 = torch.maximum(reduce.reduce_amax(x1).float(), torch.tensor(2.5))
    assert float(acc1) == float(want1)
    if n1 > 3:
        x1[n1 // 2] = float("nan")
        assert _hip.absmax_pair_into(x0.to(DEV), acc0, x1.to(DEV), acc1)
        assert torch.isnan(acc1).all() and not torch.isnan(acc0).any()


def test_pair_rejects_what_it_does_not_cover():
    a = torch.ones(64, dtype=torch.bfloat16, device=DEV)
    acc = torch.zeros(1, dtype=torch.float32, device=DEV)
    acc2 = torch.zeros(1, dtype=torch.float32, device=DEV)
    assert not _hip.absmax_pair_into(a, acc, a.float(), acc2)              # two dtypes
    assert not _hip.absmax_pair_into(a[1:33], acc, a, acc2)                # misaligned
    assert float(acc) == 0 and float(acc2) == 0


def test_value_ranges_of_many_small_tensors_in_one_launch():
    """mo_value_ranges: min, max (NaN elements left out) and a NaN flag per tensor, dtypes mixed."""
    g = torch.Generator().manual_seed(9)
    tensors = [torch.randn(5000, generator=g), torch.rand(1, generator=g).reshape(()),
               torch.randn(4096, generator=g).to(torch.bfloat16), torch.randn(257, generator=g).to(torch.float16),
               torch.rand(33, 7, generator=g) + 0.5, torch.randn(1000, generator=g),
               torch.tensor([1.0, float("inf"), 3.0]), torch.tensor([-2.0, float("-inf")]).to(torch.bfloat16),
               torch.rand(300001, generator=g), torch.rand(131072, generator=g).to(torch.bfloat16),
               torch.rand(4096, generator=g), torch.rand(4097, generator=g)]
    tensors[5][123] = float("nan")
    tensors[8][200000] = -3.0          # in a chunk of its own, far from the ends
    tensors[9][131071] = float("nan")  # the last element of the last chunk
    tensors[11][4096] = 7.0            # a chunk of one element
    got = _hip.value_ranges([t.to(DEV) for t in tensors])
    assert len(got) == len(tensors)
    for t, (lo, hi, has_nan) in zip(tensors, got):
        f = t.float().reshape(-1)
        keep = f[~torch.isnan(f)]
        assert has_nan == bool(torch.isnan(f).any())
        assert lo == float(keep.min()) and hi == float(keep.max()), (t.dtype, lo, hi)


def test_value_ranges_leaves_what_it_does_not_cover():
    a = torch.ones(8, device=DEV)
    assert _hip.value_ranges([]) == []
    assert _hip.value_ranges([a] * 33) is None                                  # more than one launch holds
    assert _hip.value_ranges([a, a.to(torch.int32)]) is None                     # not a float
    assert _hip.value_ranges([a, torch.ones(8, 8, device=DEV)[:, ::2]]) is None  # not dense
    assert _hip.value_ranges([a.cpu()]) is None
    assert _hip.value_ranges([torch.ones(5 << 20, device=DEV)]) is None             # more chunks than the buffer holds
    assert _hip.value_ranges([torch.ones(0, device=DEV), a]) == [(float("inf"), float("-inf"), False), (1.0, 1.0, False)]
    assert _hip.value_ranges([a] * 32) == [(1.0, 1.0, False)] * 32


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [1, 4097, 32768 * 3 + 5, 1 << 22])
def test_reread_hint_changes_nothing_but_the_cache_policy(dtype, n):
    """mo_absmax_hinted(MO_ABSMAX_REREAD): the same maximum as mo_absmax, NaN included."""
    x = _rand((n,), dtype, 8)
    plain = torch.zeros(1, dtype=torch.float32, device=DEV)
    hinted = torch.full((1,), 0.25, dtype=torch.float32, device=DEV)      # a running maximum
    _hip.absmax_into(x.to(DEV), plain, 1, 1, n)
    _hip.absmax_into(x.to(DEV), hinted, 1, 1, n, reread=True)
    assert float(hinted) == max(float(plain), 0.25)
    assert_bits_equal(plain.cpu().reshape(()).to(dtype), reduce.reduce_amax(x), "plain")
    if n > 2:
        x[n // 2] = float("nan")
        _hip.absmax_into(x.to(DEV), hinted, 1, 1, n, reread=True)
        assert torch.isnan(hinted).all()


def test_unknown_hint_bits_are_refused():
    import ctypes

    lib = _hip.load()
    x = torch.ones(64, dtype=torch.bfloat16, device=DEV)
    acc = torch.zeros(1, dtype=torch.float32, device=DEV)
    rc = lib.mo_absmax_hinted(ctypes.c_void_p(x.data_ptr()), 1, 1, 64, _hip.dtype_code(x.dtype),
                              ctypes.c_void_p(acc.data_ptr()), 2, None)
    assert rc == _hip.MO_ERR_ARG and float(acc) == 0
