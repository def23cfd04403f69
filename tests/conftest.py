import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_PARENT = os.path.join(ROOT, "tensorrt-model-optimizer_amd")
for p in (ROOT, PKG_PARENT):
    if p not in sys.path:
        sys.path.insert(0, p)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def assert_bits_equal(actual: torch.Tensor, expected: torch.Tensor, what: str = ""):
    """Bit-exact comparison of two tensors of the same dtype; any NaN matches any NaN."""
    assert actual.shape == expected.shape, f"{what}: shape {actual.shape} vs {expected.shape}"
    assert actual.dtype == expected.dtype, f"{what}: dtype {actual.dtype} vs {expected.dtype}"
    a, e = actual.detach().cpu(), expected.detach().cpu()
    if a.dtype.is_floating_point:
        if a.dtype in (torch.float8_e4m3fn,):
            # E4M3 has two NaN encodings (0x7F, 0xFF); which one the CPU produces for a NaN
            # operand depends on whether torch's vectorised or scalar loop handled the element,
            # so NaN matches NaN and everything else is compared bit for bit.
            a, e = a.view(torch.uint8), e.view(torch.uint8)
            ok = (a == e) | (((a & 0x7F) == 0x7F) & ((e & 0x7F) == 0x7F))
        else:
            nan_both = torch.isnan(a) & torch.isnan(e)
            width = {2: torch.int16, 4: torch.int32, 8: torch.int64}[a.element_size()]
            ok = (a.view(width) == e.view(width)) | nan_both
    else:
        ok = a == e
    if not bool(ok.all()):
        bad = (~ok).nonzero()
        first = tuple(bad[0].tolist())
        raise AssertionError(
            f"{what}: {bad.shape[0]} of {ok.numel()} elements differ; first at {first}: "
            f"got {a[first].item()!r} expected {e[first].item()!r}")


def load_export_vectors():
    """tests/golden/export_vectors.json (outputs of the reference's export casts) as tensors."""
    import json

    bits = {"bfloat16": torch.int16, "float16": torch.int16, "float32": torch.int32,
            "uint8": torch.uint8, "int8": torch.uint8, "float8_e4m3fn": torch.uint8}
    with open(os.path.join(GOLDEN, "export_vectors.json")) as f:
        raw = json.load(f)["cases"]
    cases = []
    for c in raw:
        wd, od = getattr(torch, c["weight_dtype"]), getattr(torch, c["out_dtype"])
        cases.append({
            "name": c["name"], "format": c["format"],
            "weight": torch.tensor(c["weight_bits"], dtype=bits[c["weight_dtype"]]).view(wd)
            .reshape(c["weight_shape"]),
            "scale": torch.tensor(c["scale_bits"], dtype=torch.int32).view(torch.float32)
            .reshape(c["scale_shape"]),
            "out": torch.tensor(c["out_bits"], dtype=torch.uint8).view(od).reshape(c["out_shape"]),
        })
    return cases


@pytest.fixture
def cpu_fp8_overflow():
    """FP8 fake quantisation with the reference's CPU semantics for out-of-range values (NaN),
    for tests that compare against the CPU restatement with an amax below the data."""
    import modelopt_amd.torch.quantization as mtq

    previous = mtq.set_fp8_overflow_behavior("nan")
    yield
    mtq.set_fp8_overflow_behavior(previous)
