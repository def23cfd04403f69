"""Register budgets of the kernels whose speed depends on how many wavefronts fit a SIMD, read
from the built library (no GPU needed): the code object's metadata names every kernel with its
vector-register count.  A change that makes the compiler keep more values live can halve the
occupancy of such a kernel without failing any numerical test."""

import os
import struct

import msgpack
import pytest

from modelopt_amd import _hip

MAGIC = b"__CLANG_OFFLOAD_BUNDLE__"


def _code_objects(blob):
    """The device code objects (ELF images) inside a library built by hipcc."""
    out = []
    at = blob.find(MAGIC)
    while at >= 0:
        n = struct.unpack_from("<Q", blob, at + len(MAGIC))[0]
        pos = at + len(MAGIC) + 8
        for _ in range(n):
            offset, size, tsize = struct.unpack_from("<QQQ", blob, pos)
            triple = blob[pos + 24:pos + 24 + tsize].decode()
            pos += 24 + tsize
            if "gfx950" in triple and size:
                out.append(blob[at + offset:at + offset + size])
        at = blob.find(MAGIC, at + 1)
    return out


def _kernel_metadata(elf):
    """{kernel name: metadata map} from the NT_AMDGPU_METADATA note of a 64-bit little-endian ELF."""
    shoff, = struct.unpack_from("<Q", elf, 0x28)
    shentsize, shnum = struct.unpack_from("<HH", elf, 0x3A)
    for i in range(shnum):
        base = shoff + i * shentsize
        sh_type, = struct.unpack_from("<I", elf, base + 4)
        if sh_type != 7:    # SHT_NOTE
            continue
        off, size = struct.unpack_from("<QQ", elf, base + 0x18)
        pos, end = off, off + size
        while pos + 12 <= end:
            namesz, descsz, ntype = struct.unpack_from("<III", elf, pos)
            name = elf[pos + 12:pos + 12 + namesz].rstrip(b"\0")
            desc_at = pos + 12 + (namesz + 3) // 4 * 4
            if name == b"AMDGPU" and ntype == 32:
                meta = msgpack.unpackb(elf[desc_at:desc_at + descsz], raw=False, strict_map_key=False)
                return {k[".name"]: k for k in meta["amdhsa.kernels"]}
            pos = desc_at + (descsz + 3) // 4 * 4
    return {}


@pytest.fixture(scope="module")
def kernels():
    if not os.path.exists(_hip.LIB_PATH):
        pytest.skip("library not built")
    found = {}
    with open(_hip.LIB_PATH, "rb") as f:
        blob = f.read()
    for elf in _code_objects(blob):
        found.update(_kernel_metadata(elf))
    assert found, "no gfx950 code object with kernel metadata in the library"
    return found


def _vgprs(kernels, fragment):
    hits = {n: k[".vgpr_count"] for n, k in kernels.items() if fragment in n}
    assert hits, fragment
    return hits


@pytest.mark.parametrize("fragment,limit,why", [
    # 512 registers per SIMD lane: limit = 512 // wavefronts, rounded down to the granule of 8
    ("awq_clip_loss_kernelILi2ELi128E", 168, "three wavefronts per SIMD (one: 35 % slower)"),
    ("awq_search_kernelILi2E", 256, "two wavefronts per SIMD"),
    ("nvfp4_quantize_multi_kernel", 64, "eight wavefronts per SIMD, the occupancy cap decides"),
    ("absmax_multi_kernelILi2E", 64, "eight wavefronts per SIMD"),
    ("weight_scale_colsum8_kernelILi2E", 96, "five wavefronts per SIMD (three: 25 % slower)"),
    ("nvfp4_qdq_fast_kernelILi0ELi1E", 64, "eight wavefronts per SIMD"),
    ("qdq_kernelILi2ELi0ELb0ENS_5Fp8OpILb1E", 64, "eight wavefronts per SIMD"),
])
def test_register_budget(kernels, fragment, limit, why):
    for name, count in _vgprs(kernels, fragment).items():
        assert count <= limit, f"{name}: {count} vector registers, budget {limit} ({why})"


def test_no_kernel_spills(kernels):
    spilled = {n: k[".vgpr_spill_count"] for n, k in kernels.items() if k.get(".vgpr_spill_count", 0)}
    assert not spilled, spilled
