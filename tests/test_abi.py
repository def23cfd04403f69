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
    assert lib.mo_set_option(99, 1) == -1
    assert lib.mo_get_option(_hip.MO_OPT_FORCE_EXACT) == 0
    assert lib.mo_get_option(_hip.MO_OPT_SATURATE_BLOCK_SCALE) == 0


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_hip, "_lib", None)
    monkeypatch.setattr(_hip, "LIB_PATH", "/nonexistent/libmodelopt_hip.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        _hip.load()


def test_cpu_tensor_is_rejected():
    import torch

    with pytest.raises(RuntimeError, match="GPU memory"):
        _hip.absmax_into(torch.zeros(8), torch.zeros(1), 1, 1, 8)
