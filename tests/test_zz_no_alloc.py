"""The entry point that allocates nothing (per-column abs-max through the library's fixed device
workspace) against the workspace-argument entry point it is a variant of, through the C ABI."""

import ctypes

import pytest
import torch

from modelopt_amd import _hip

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _run(name, x, acc, *extra):
    lib = _hip.load()
    stream = ctypes.c_void_p(torch.cuda.current_stream(x.device).cuda_stream)
    with torch.cuda.device(x.device):
        return getattr(lib, name)(ctypes.c_void_p(x.data_ptr()), x.shape[0], x.shape[1],
                                  _hip.dtype_code(x.dtype), ctypes.c_void_p(acc.data_ptr()), *extra, stream)


def _both(x):
    rows, cols = x.shape
    want = torch.zeros(cols, dtype=torch.float32, device=x.device)
    partial = torch.empty((64, cols), dtype=torch.int32, device=x.device)
    assert _run("mo_absmax_cols_staged", x, want, ctypes.c_void_p(partial.data_ptr()), 64) == 0
    got = torch.zeros(cols, dtype=torch.float32, device=x.device)
    assert _run("mo_absmax_cols_noalloc", x, got) == 0
    torch.cuda.synchronize()
    return got, want


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_two_calls_in_a_row_the_second_smaller(dtype):
    g = torch.Generator(device=DEV).manual_seed(7)
    big = (torch.randn((4096, 14336), generator=g, device=DEV) * 3).to(dtype)
    small = (torch.randn((96, 512), generator=g, device=DEV) * 0.01).to(dtype)  # far smaller maxima
    for x in (big, small):
        got, want = _both(x)
        assert torch.equal(got.view(torch.int32), want.view(torch.int32))
        assert torch.equal(got, x.abs().amax(dim=0).float())


def test_running_maximum_and_limits():
    x = torch.randn((256, 1024), device=DEV, dtype=torch.bfloat16)
    acc = torch.full((1024,), 2.0, dtype=torch.float32, device=DEV)
    assert _run("mo_absmax_cols_noalloc", x, acc) == 0
    torch.cuda.synchronize()
    assert torch.equal(acc, torch.maximum(x.abs().amax(dim=0).float(), torch.tensor(2.0, device=DEV)))
    lib = _hip.load()
    null, p = ctypes.c_void_p(0), ctypes.c_void_p(acc.data_ptr())
    words = 1 << 20
    assert lib.mo_absmax_cols_noalloc(p, 4, words + 8, _hip.MO_BF16, p, null) == _hip.MO_ERR_TOO_LARGE
    assert lib.mo_absmax_cols_noalloc(p, 4, 12, _hip.MO_BF16, p, null) == _hip.MO_ERR_UNSUPPORTED
    assert lib.mo_absmax_cols_noalloc(null, 4, 16, _hip.MO_BF16, p, null) == _hip.MO_ERR_ARG
    assert lib.mo_absmax_cols_noalloc(null, 0, 16, _hip.MO_BF16, p, null) == 0
    assert b"fixed workspace" in lib.mo_error_string(_hip.MO_ERR_TOO_LARGE)


def test_no_device_allocation_happens():
    x = torch.randn((512, 2048), device=DEV, dtype=torch.bfloat16)
    acc = torch.zeros(2048, dtype=torch.float32, device=DEV)
    assert _run("mo_absmax_cols_noalloc", x, acc) == 0  # first call on the device: address lookup
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    for _ in range(3):
        assert _run("mo_absmax_cols_noalloc", x, acc) == 0
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
    assert torch.cuda.mem_get_info()[0] == free_before
