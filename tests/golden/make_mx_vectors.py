"""Writes tests/golden/mx_vectors.json.

The vectors are the inline literals (inputs and expected outputs) of the reference's own test
file tests/gpu/torch/quantization/test_quantize_mxformats_cuda.py:61-317 (test_mxfp4, test_mxfp6,
test_mxfp8, test_mxint8).  The file is read as text and its list literals are picked out of the
syntax tree; nothing of the reference is imported or executed.  Run in the container that holds
the reference checkout: ``python tests/golden/make_mx_vectors.py [reference root]``.
"""

import ast
import json
import os
import sys

ROOT = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
SRC = os.path.join(ROOT, "tests/gpu/torch/quantization/test_quantize_mxformats_cuda.py")

# per test function: block sizes it runs, the repeat unit, the element formats of its
# successive expected-output tables, tolerance of its allclose, line of the function
SPEC = {
    "test_mxfp4": {"block_sizes": [8, 16, 32], "unit": 8, "formats": ["E2M1"], "atol": 1e-8},
    "test_mxfp6": {"block_sizes": [16], "unit": 32, "formats": ["E3M2", "E2M3"], "atol": 1e-3},
    "test_mxfp8": {"block_sizes": [8], "unit": 8, "formats": ["E4M3", "E5M2"], "atol": 1e-3},
    "test_mxint8": {"block_sizes": [8], "unit": 8, "formats": ["INT8"], "atol": 1e-3},
}


def tensor_literals(func):
    """First positional argument of every ``torch.tensor(...)`` call that is a nested list."""
    found = []
    for node in ast.walk(func):
        if (isinstance(node, ast.Call) and isinstance(node.func, ast.Attribute)
                and node.func.attr == "tensor" and node.args and isinstance(node.args[0], ast.List)):
            found.append((node.lineno, ast.literal_eval(node.args[0])))
    return [v for _, v in sorted(found, key=lambda t: t[0])]


def main():
    tree = ast.parse(open(SRC).read())
    out = {"source": "tests/gpu/torch/quantization/test_quantize_mxformats_cuda.py", "cases": []}
    for func in tree.body:
        if isinstance(func, ast.FunctionDef) and func.name in SPEC:
            spec = SPEC[func.name]
            tensors = tensor_literals(func)
            test_in, tables = tensors[0], tensors[1:]
            assert len(tables) == len(spec["formats"]), (func.name, len(tables))
            for fmt, table in zip(spec["formats"], tables):
                assert len(table) == len(test_in) and all(len(r) == len(test_in[0]) for r in table)
                out["cases"].append({
                    "test": func.name, "line": func.lineno, "format": fmt, "scale_format": "E8M0",
                    "block_sizes": spec["block_sizes"], "unit": spec["unit"], "atol": spec["atol"],
                    "input": test_in, "output": table})
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "mx_vectors.json")
    with open(dst, "w") as f:
        json.dump(out, f)
    print("wrote", dst, len(out["cases"]), "cases")


if __name__ == "__main__":
    main()
