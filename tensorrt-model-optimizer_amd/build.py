"""Build libmodelopt_hip.so for gfx950 with hipcc (in-tree, next to this file).

Usage: ``python build.py [-j N] [--force] [--tuning]``.  Also importable: ``build(force=False)``.

``--tuning`` builds libmodelopt_hip_tuning.so instead, compiled with -DMO_TUNING: in that build
the per-kernel occupancy caps (unused dynamic LDS) are read from the environment at every launch
(``MO_BALLAST_<kernel>`` or ``MO_BALLAST_ALL``, in KiB), which is how the caps compiled into the
product library were chosen.  ``MODELOPT_AMD_LIB=<path>`` makes the Python layer load that file.
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
PROBE_SRC = os.path.join(HERE, "probe", "l2_read_probe.hip")   # measurement aid for bench.py: its own library, outside csrc/
PROBE_LIB = os.path.join(HERE, "libmodelopt_probe.so")
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


def _compile(src, force, obj_dir, extra):
    out = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
    path = os.path.join(CSRC, src)
    if not force and not _stale(out, [path, *HEADERS]):
        return out
    cmd = ["hipcc", *FLAGS, *extra, "-x", "hip", "-c", path, "-o", out]
    subprocess.run(cmd, check=True)
    return out


def build(force=False, jobs=4, tuning=False):
    obj_dir = os.path.join(OBJ, "tuning") if tuning else OBJ
    lib = LIB.replace(".so", "_tuning.so") if tuning else LIB
    extra = ["-DMO_TUNING"] if tuning else []
    os.makedirs(obj_dir, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force, obj_dir, extra), _sources()))
    if force or _stale(lib, objs):
        subprocess.run(["hipcc", "-shared", "-fPIC", "--offload-arch=gfx950", *objs, "-o", lib],
                       check=True)
    if not tuning and (force or _stale(PROBE_LIB, [PROBE_SRC])):
        subprocess.run(["hipcc", *FLAGS, "-shared", "-x", "hip", PROBE_SRC, "-o", PROBE_LIB], check=True)
    return lib


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("-j", type=int, default=4)
    ap.add_argument("--force", action="store_true")
    ap.add_argument("--tuning", action="store_true")
    a = ap.parse_args()
    print(build(a.force, a.j, a.tuning))
    sys.exit(0)
