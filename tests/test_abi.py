"""The C-ABI library loads and exports every symbol include/modelopt_hip.h declares (no GPU)."""

import ctypes
import os
import re

import pytest

from conftest import ROOT
from modelopt_amd import _hip

HEADER = os.path.join(ROOT, "include", "modelopt_hip.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mo_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_functions():
    names = _declared_functions()
    assert "mo_nvfp4_quantize" in names and "mo_absmax" in names and len(names) >= 10


def test_library_exports_every_declared_symbol():
    if not os.path.exists(_hip.LIB_PATH):
        pytest.fail(f"{_hip.LIB_PATH} is missing: run `python __graft_entry__.py` (build) first")
    lib = ctypes.CDLL(_hip.LIB_PATH)
    for name in _declared_functions():
        assert hasattr(lib, name), f"{name} declared in the header but not exported"


def test_binding_covers_every_declared_symbol():
    assert sorted(_hip.SIGNATURES) == _declared_functions()


def test_version_and_error_strings_without_gpu():
    lib = _hip.load()
    assert lib.mo_version() >= 1
    assert lib.mo_error_string(0) == b"ok"
    assert b"invalid argument" in lib.mo_error_string(-1)
    assert not hasattr(lib, "mo_set_option")  # no process-wide state: flags travel with each call


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_hip, "_lib", None)
    monkeypatch.setattr(_hip, "LIB_PATH", "/nonexistent/libmodelopt_hip.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        _hip.load()


def test_cpu_tensor_is_rejected():
    import torch

    with pytest.raises(RuntimeError, match="GPU memory"):
        _hip.absmax_into(torch.zeros(8), torch.zeros(1), 1, 1, 8)


def test_argument_checks_that_need_no_gpu():
    """Entry points validate before they touch the device: empty work is MO_OK, bad enums, sizes
    and null pointers come back as the documented status codes (no launch happens here)."""
    lib = _hip.load()
    OK, ARG, DTYPE, UNSUP = 0, -1, -2, -3
    null = ctypes.c_void_p(0)
    buf = (ctypes.c_float * 64)()
    p = ctypes.cast(buf, ctypes.c_void_p)
    # abs-max / qdq: empty tensors
    assert lib.mo_nvfp4_quantize(null, 0, 0, 2, 16, null, 0, null, null, null, null, 0, null) == OK
    assert lib.mo_nvfp4_quantize(p, 4, 16, 2, 12, p, 0, null, p, p, p, 0, null) == UNSUP   # block size
    assert lib.mo_nvfp4_quantize(null, 4, 16, 2, 16, p, 0, null, p, p, p, 0, null) == ARG  # null input
    assert lib.mo_nvfp4_quantize(null, 0, 0, 2, 16, null, 0, null, null, null, null, 64, null) == ARG  # flag bit
    assert lib.mo_nvfp4_quantize_multi(null, 0, null, 0, 2, 16, 0, 0, null) == OK
    assert lib.mo_nvfp4_quantize_multi(null, 1, null, 1, 2, 16, 0, 0, null) == ARG
    assert lib.mo_nvfp4_quantize_multi(p, 1, null, 1, 0, 16, 0, 0, null) == UNSUP          # fp32 tensors
    assert lib.mo_nvfp4_quantize_multi(null, 0, null, 0, 2, 16, 0, 4, null) == ARG         # flag bit
    assert lib.mo_convert_to_format(null, null, 0, 6, null) == OK
    assert lib.mo_convert_to_format(p, p, 4, 10, null) == UNSUP
    assert lib.mo_int4_block_quantize(null, 0, 128, 2, null, 1, null, null) == OK
    # clip search
    ratios = (ctypes.c_float * 2)(0.5, 1.0)
    assert lib.mo_awq_clip_losses(null, 0, null, 0, 0, 2, 128, null, 2, ratios, 2, 4, 0, 0, null, null) == OK
    assert lib.mo_awq_clip_losses(p, 8, p, 8, 256, 7, 128, p, 2, ratios, 2, 4, 0, 0, p, null) == DTYPE
    assert lib.mo_awq_clip_losses(p, 8, p, 8, 256, 2, 48, p, 2, ratios, 2, 4, 0, 0, p, null) == UNSUP
    assert lib.mo_awq_clip_losses(p, 8, p, 8, 200, 2, 128, p, 2, ratios, 2, 4, 0, 0, p, null) == UNSUP  # ragged
    assert lib.mo_awq_clip_losses(p, 8, p, 8, 256, 2, 128, p, 2, ratios, 33, 4, 0, 0, p, null) == UNSUP
    assert lib.mo_awq_clip_losses(p, 8, p, 8, 256, 2, 128, null, 2, ratios, 2, 4, 0, 0, p, null) == ARG
    assert lib.mo_awq_clip_losses(p, 8, p, 8, 256, 2, 128, p, 2, ratios, 2, 1, 0, 0, p, null) == ARG    # 1 bit
    # storage casts
    assert lib.mo_real_quantize(null, 0, 1, 0, 2, null, 2, 2, 0, null, null) == OK
    assert lib.mo_real_quantize(p, 1, 1, 8, 2, p, 2, 2, 5, p, null) == UNSUP               # format
    assert lib.mo_real_quantize(p, 1, 1, 8, 2, p, 9, 2, 0, p, null) == DTYPE
    assert lib.mo_int4_pack_rows(p, 1, 3, 16, 16, 2, p, p, null) == ARG                    # odd row count
    assert lib.mo_int4_pack_rows_via(p, 1, 4, 16, 16, 2, p, 1, p, null) == UNSUP            # bf16 weight, fp16 quotient
    assert lib.mo_int4_pack_rows_via(p, 1, 4, 16, 16, 0, p, 2, p, null) == UNSUP            # fp32 weight, bf16 quotient
    assert lib.mo_int4_pack_rows_via(p, 1, 4, 16, 16, 2, p, 7, p, null) == DTYPE
    assert lib.mo_int4_pack_rows_via(null, 0, 4, 16, 16, 2, null, 2, null, null) == OK
    # the one-launch helpers of the calibration algorithms
    TOO_LARGE = -5
    assert lib.mo_absmax_hinted(null, 0, 4, 4, 2, null, 1, null) == OK                     # empty
    assert lib.mo_absmax_hinted(p, 1, 4, 4, 2, p, 2, null) == ARG                          # unknown hint
    assert lib.mo_absmax_hinted(p, 1, 4, 4, 9, p, 1, null) == DTYPE
    assert lib.mo_absmax_hinted(null, 1, 4, 4, 2, p, 0, null) == ARG
    ptrs = (ctypes.c_void_p * 33)(*[ctypes.addressof(buf)] * 33)
    counts = (ctypes.c_int64 * 33)(*[8] * 33)
    kinds = (ctypes.c_int * 33)(*[0] * 33)
    assert lib.mo_value_ranges(null, null, null, 0, null, 0, null) == OK
    assert lib.mo_value_ranges(ptrs, counts, kinds, 33, p, 64, null) == TOO_LARGE          # > 32 tensors
    assert lib.mo_value_ranges(ptrs, counts, kinds, 4, p, 3, null) == TOO_LARGE            # output too short
    assert lib.mo_value_ranges(ptrs, counts, kinds, 4, null, 4, null) == ARG
    kinds[1] = 7
    assert lib.mo_value_ranges(ptrs, counts, kinds, 4, p, 4, null) == DTYPE
    kinds[1] = 0
    counts[2] = -1
    assert lib.mo_value_ranges(ptrs, counts, kinds, 4, p, 4, null) == ARG
    counts[2] = 8
    ptrs[3] = ctypes.addressof(buf) + 1
    assert lib.mo_value_ranges(ptrs, counts, kinds, 4, p, 4, null) == UNSUP                # misaligned fp32
    assert lib.mo_awq_pick_scale(p, 0, p, 8, p, p, p, p, p, 2, null) == ARG                # nothing to pick
    assert lib.mo_awq_pick_scale(null, 2, p, 8, p, p, p, p, p, 2, null) == ARG
    assert lib.mo_awq_pick_scale(p, 2, p, 8, p, p, p, p, p, 5, null) == DTYPE
    assert lib.mo_awq_pick_scale(p, 70000, p, 8, p, p, p, p, p, 2, null) == UNSUP
    assert lib.mo_smooth_scales(p, p, 0, 0.5, 0, 0.5, 0, 2, p, p, p, p, p, null) == ARG    # max over nothing
    assert lib.mo_smooth_scales(p, p, 8, 0.5, 4, 0.5, 0, 2, p, p, p, p, p, null) == ARG    # power mode
    assert lib.mo_smooth_scales(p, p, 8, 0.5, 0, 0.5, 0, 3, p, p, p, p, p, null) == DTYPE
    assert lib.mo_smooth_scales(p, null, 8, 0.5, 0, 0.5, 0, 2, p, p, p, p, p, null) == ARG
    assert b"unsupported" in lib.mo_error_string(UNSUP).lower() or lib.mo_error_string(UNSUP)


def test_product_never_reaches_for_the_oracle_or_scratch_files():
    """The shipped package must not import, read or run the CPU oracle (test infrastructure) or
    anything outside itself: checked on the source text and on a fresh interpreter's modules."""
    import subprocess
    import sys

    pkg = os.path.join(ROOT, "tensorrt-model-optimizer_amd", "modelopt_amd")
    for dirpath, _, files in os.walk(pkg):
        for name in files:
            if name.endswith(".py"):
                text = open(os.path.join(dirpath, name)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M), name
                assert "_work" not in text and "oracle/" not in text, name
    code = ("import sys; sys.path.insert(0, %r); sys.path.insert(0, %r);"
            "import modelopt_amd.torch.quantization, modelopt_amd.torch.export;"
            "bad = [m for m in sys.modules if m == 'oracle' or m.startswith('oracle.')];"
            "print(bad); sys.exit(1 if bad else 0)") % (os.path.join(ROOT, "tensorrt-model-optimizer_amd"), ROOT)
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
