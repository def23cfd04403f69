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
