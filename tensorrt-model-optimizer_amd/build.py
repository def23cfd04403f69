"""Build libmodelopt_hip.so for gfx950 with hipcc (in-tree, next to this file).

Usage: ``python build.py [-j N] [--force]``.  Also importable: ``build(force=False)``.
"""

import argparse
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libmodelopt_hip.so")
HEADERS = [os.path.join(CSRC, h) for h in ("common.h", "qdq_ops.h", "awq_ops.h")] + [
    os.path.join(HERE, "..", "include", "modelopt_hip.h")]

# -ffp-contract=off: the rounding tricks rely on separately rounded fp32 multiplies and adds.
# packed-fp32-ops is switched off on purpose (v_pk_*_f32 forms are not trusted on this target).
FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-ffp-contract=off",
    "-fno-fast-math", "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith((".hip", ".cpp")))


def _stale(out, deps):
    if not os.path.exists(out):
        return True
    t = os.path.getmtime(out)
    return any(os.path.getmtime(d) > t for d in deps)


def _compile(src, force):
    out = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    path = os.path.join(CSRC, src)
    if not force and not _stale(out, [path, *HEADERS]):
        return out
    cmd = ["hipcc", *FLAGS, "-x", "hip", "-c", path, "-o", out]
    subprocess.run(cmd, check=True)
    return out


def build(force=False, jobs=4):
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), _sources()))
    if force or _stale(LIB, objs):
        subprocess.run(["hipcc", "-shared", "-fPIC", "--offload-arch=gfx950", *objs, "-o", LIB],
                       check=True)
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("-j", type=int, default=4)
    ap.add_argument("--force", action="store_true")
    a = ap.parse_args()
    print(build(a.force, a.j))
    sys.exit(0)
