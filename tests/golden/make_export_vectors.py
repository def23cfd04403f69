"""Writes tests/golden/export_vectors.json: inputs and outputs of the reference's export casts.

No test of the reference pins ``pack_int4_in_uint8`` or the FP8 / INT8 branches of
``to_quantized_weight`` (modelopt/torch/export/quant_utils.py:697-774), so this script, in the build
container only, runs those two functions on seeded inputs and records what they return.  The
package itself cannot be imported here (its ``__init__`` asks for an installed distribution and for
solver / profiler packages that are absent), so the two function definitions are taken from the
reference file's syntax tree and executed with torch and the format-name constants of
``export/model_config.py:29-42`` in scope; nothing else of the file runs.  Only the resulting
vectors are committed; the GPU box never sees the reference.

Run from the repo root: ``python tests/golden/make_export_vectors.py [/root/reference]``.
"""

import ast
import json
import os
import sys
import warnings

import torch

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
SRC = os.path.join(REF, "modelopt/torch/export/quant_utils.py")
CFG = os.path.join(REF, "modelopt/torch/export/model_config.py")
WANTED = ("pack_int4_in_uint8", "to_quantized_weight")


def _reference_functions():
    ns = {"torch": torch, "warn": warnings.warn, "clear_cuda_cache": lambda: None,
          # only the isinstance() test at the top of to_quantized_weight touches this name
          "QTensorWrapper": type("QTensorWrapper", (), {})}
    with open(CFG) as f:
        for node in ast.parse(f.read()).body:
            if (isinstance(node, ast.Assign) and isinstance(node.targets[0], ast.Name)
                    and node.targets[0].id.startswith("QUANTIZATION_")):
                ns[node.targets[0].id] = ast.literal_eval(node.value)
    with open(SRC) as f:
        tree = ast.parse(f.read())
    defs = [n for n in tree.body if isinstance(n, ast.FunctionDef) and n.name in WANTED]
    assert sorted(d.name for d in defs) == sorted(WANTED)
    exec(compile(ast.Module(body=defs, type_ignores=[]), SRC, "exec"), ns)
    return ns


def _bits(t):
    """Tensor -> nested list of its raw bit patterns (exact for every dtype used here)."""
    view = {2: torch.int16, 4: torch.int32, 1: torch.uint8}[t.element_size()]
    return t.contiguous().view(view).tolist()


def _entry(name, fmt, w, wsf, out):
    return {"name": name, "format": fmt,
            "weight_dtype": str(w.dtype).split(".")[-1], "weight_shape": list(w.shape),
            "weight_bits": _bits(w),
            "scale_shape": list(wsf.shape), "scale_bits": _bits(wsf.float()),
            "out_dtype": str(out.dtype).split(".")[-1], "out_shape": list(out.shape),
            "out_bits": _bits(out)}


def _block_scales(w, bs):
    """f32(max|w| per block) / 7 with zeros -> 1 (export/quant_utils.py:68-91); any positive scale
    would do for pinning the byte layout."""
    s = w.reshape(*w.shape[:-1], w.shape[-1] // bs, bs).abs().amax(-1).float() / 7.0
    s[s == 0] = 1.0
    return s


def main():
    ns = _reference_functions()
    pack, to_q = ns["pack_int4_in_uint8"], ns["to_quantized_weight"]
    g = torch.Generator().manual_seed(20)
    out = []

    # INT4-AWQ, 2-D: rows 0/1 of a byte pair are made asymmetric (row 2j positive, 2j+1 negative in
    # places) so a swapped nibble order or a pairing along K instead of N changes the bytes.
    w = (0.3 * torch.randn(6, 16, generator=g)).to(torch.bfloat16)
    out.append(_entry("int4_awq_2d_block8", "int4_awq", w, _block_scales(w, 8),
                      pack(w, _block_scales(w, 8))))
    w = (0.02 * torch.randn(8, 256, generator=g)).to(torch.bfloat16)
    out.append(_entry("int4_awq_2d_block128", "int4_awq", w, _block_scales(w, 128),
                      to_q(w, _block_scales(w, 128), "int4_awq")))
    # every quantised level, exact .5 ties (round half to even) and values beyond the clamp
    levels = torch.tensor([[-9.0, -8.5, -8.0, -7.5, -2.5, -1.5, -0.5, -0.0],
                           [0.0, 0.5, 1.5, 2.5, 6.5, 7.0, 7.5, 9.0],
                           [1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 7.49],
                           [-1.0, -2.0, -3.0, -4.0, -5.0, -6.0, -7.0, -8.49]])
    s = torch.tensor([[0.25], [0.5], [1.0], [2.0]])
    w = (levels * s).to(torch.bfloat16)
    out.append(_entry("int4_awq_levels_ties_clamps", "w4a8_awq", w, s, to_q(w, s, "w4a8_awq")))
    w = (0.5 * torch.randn(4, 24, generator=g)).to(torch.float16)
    out.append(_entry("int4_awq_fp16_block8", "int4_awq", w, _block_scales(w, 8),
                      pack(w, _block_scales(w, 8))))
    w = 0.5 * torch.randn(2, 8, generator=g)
    out.append(_entry("int4_awq_fp32_block4", "int4_awq", w, _block_scales(w, 4),
                      pack(w, _block_scales(w, 4))))
    # 3-D stacked experts
    w = (0.3 * torch.randn(3, 4, 16, generator=g)).to(torch.bfloat16)
    out.append(_entry("int4_awq_3d_experts_block8", "int4_awq", w, _block_scales(w, 8),
                      pack(w, _block_scales(w, 8))))

    # FP8 per tensor: 0-dim fp32 scale (bf16 quotient, rounded twice), 1-element scale (fp32
    # quotient, rounded once), stacked experts with one scale each
    w = (0.02 * torch.randn(16, 64, generator=g)).to(torch.bfloat16)
    w[0, 0] = 0.11
    s0 = w.abs().max().float() / 448.0
    out.append(_entry("fp8_0dim_scale", "fp8", w, s0, to_q(w, s0, "fp8")))
    out.append(_entry("fp8_1elem_scale", "fp8", w, s0.reshape(1), to_q(w, s0.reshape(1), "fp8")))
    wf = (0.02 * torch.randn(8, 32, generator=g)).to(torch.float16)
    sf = wf.abs().max().float() / 448.0
    out.append(_entry("fp8_fp16_0dim_scale", "fp8", wf, sf, to_q(wf, sf, "fp8")))
    w3 = (0.02 * torch.randn(3, 4, 16, generator=g)).to(torch.bfloat16)
    s3 = w3.abs().amax((1, 2)).float() / 448.0
    out.append(_entry("fp8_3d_experts", "fp8", w3, s3.unsqueeze(-1),
                      to_q(w3, s3.unsqueeze(-1), "fp8")))
    # FP8 per channel / per token
    w = (0.02 * torch.randn(8, 32, generator=g)).to(torch.bfloat16)
    s = w.abs().amax(1).float() / 448.0
    out.append(_entry("fp8_pc_pt_rows", "fp8_pc_pt", w, s, to_q(w, s, "fp8_pc_pt")))
    # INT8 per row (SmoothQuant / weight only)
    w = (0.02 * torch.randn(8, 32, generator=g)).to(torch.bfloat16)
    s = w.abs().amax(1).float() / 127.0
    out.append(_entry("int8_sq_rows", "int8_sq", w, s, to_q(w, s, "int8_sq")))
    w = torch.tensor([[-200.0, -128.5, -127.5, -0.5, 0.5, 1.5, 126.5, 127.5, 300.0, 2.5]] * 2)
    w = (w * torch.tensor([[0.5], [2.0]])).to(torch.bfloat16)
    s = torch.tensor([0.5, 2.0])
    out.append(_entry("int8_wo_ties_clamps", "int8_wo", w, s, to_q(w, s, "int8_wo")))

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "export_vectors.json")
    with open(path, "w") as f:
        json.dump({"source": "modelopt/torch/export/quant_utils.py:697-774, executed by "
                             "tests/golden/make_export_vectors.py", "cases": out}, f)
    print(path, len(out), "cases", os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
