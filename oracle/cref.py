"""ctypes loader for the C restatement in ``oracle/c`` (test infrastructure only).

``load()`` returns the library, building it with ``make`` when the shared object is missing;
the wrappers take and return CPU torch tensors.  Used by the tests to cross-check the torch
restatement bit for bit and by ``bench.py`` as the timed CPU baseline.
"""

import ctypes
import os
import subprocess

import torch

_HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c")
_LIB = None
_DT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
_P, _I64, _I, _F = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float


def build():
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)


def load():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libquant_ref.so")
        if not os.path.exists(path):
            build()
        lib = ctypes.CDLL(path)
        lib.qr_f32_to_e4m3.argtypes, lib.qr_f32_to_e4m3.restype = [_F], ctypes.c_uint8
        lib.qr_e4m3_to_f32.argtypes, lib.qr_e4m3_to_f32.restype = [ctypes.c_uint8], _F
        lib.qr_f32_to_e2m1.argtypes, lib.qr_f32_to_e2m1.restype = [_F], ctypes.c_uint8
        lib.qr_e2m1_to_f32.argtypes, lib.qr_e2m1_to_f32.restype = [ctypes.c_uint8], _F
        lib.qr_absmax.argtypes, lib.qr_absmax.restype = [_P, _I64, _I], _F
        lib.qr_threads.argtypes, lib.qr_threads.restype = [], _I
        lib.qr_nvfp4_quantize.argtypes = [_P, _I64, _I64, _I, _I, _F, _P, _P, _P]
        lib.qr_nvfp4_dequantize.argtypes = [_P, _P, _F, _I64, _I, _P, _I]
        lib.qr_fp8_qdq.argtypes = [_P, _I64, _I, _P, _P]
        lib.qr_int_qdq.argtypes = [_P, _I64, _I, _F, _I, _I, _I, _P]
        lib.qr_int4_block_quantize.argtypes = [_P, _I64, _I, _I, _P, _P]
        lib.qr_real_quantize.argtypes = [_P, _I64, _I, _F, _I, _I, _P]
        lib.qr_convert_to_types.argtypes, lib.qr_convert_to_types.restype = [_F, _I], _F
        lib.qr_block_fp_qdq.argtypes = [_P, _I64, _I64, _I, _I, _I, _I, _P, _I64, _P]
        lib.qr_block_fp_qdq.restype = None
        for name in ("qr_nvfp4_quantize", "qr_nvfp4_dequantize", "qr_fp8_qdq", "qr_int_qdq",
                     "qr_int4_block_quantize", "qr_real_quantize"):
            getattr(lib, name).restype = None
        _LIB = lib
    return _LIB


def _cpu(t):
    assert t.device.type == "cpu"
    return t.contiguous()


def threads():
    """Threads the C library's parallel loops use (OMP_NUM_THREADS or the CPU count)."""
    return load().qr_threads()


def absmax(x):
    x = _cpu(x)
    return load().qr_absmax(x.data_ptr(), x.numel(), _DT[x.dtype])


def nvfp4_quantize(x, block_size=16, amax=None):
    """-> (packed uint8 [..., k / 2], wsf float8_e4m3fn [..., k / block], wsf2 fp32 0-dim)."""
    x = _cpu(x)
    k = x.shape[-1]
    assert k % block_size == 0
    rows = x.numel() // k
    amax = absmax(x) if amax is None else float(amax)
    packed = torch.empty(x.shape[:-1] + (k // 2,), dtype=torch.uint8)
    wsf = torch.empty(x.shape[:-1] + (k // block_size,), dtype=torch.uint8)
    wsf2 = torch.empty((), dtype=torch.float32)
    load().qr_nvfp4_quantize(x.data_ptr(), rows, k, _DT[x.dtype], block_size, amax,
                             packed.data_ptr(), wsf.data_ptr(), wsf2.data_ptr())
    return packed, wsf.view(torch.float8_e4m3fn), wsf2


def nvfp4_dequantize(packed, wsf, wsf2, block_size, dtype):
    packed, wsf = _cpu(packed), _cpu(wsf.view(torch.uint8))
    n = packed.numel() * 2
    y = torch.empty(packed.shape[:-1] + (packed.shape[-1] * 2,), dtype=dtype)
    load().qr_nvfp4_dequantize(packed.data_ptr(), wsf.data_ptr(), float(wsf2), n, block_size,
                               y.data_ptr(), _DT[dtype])
    return y


def fp8_qdq(x, amax=None):
    x = _cpu(x)
    y = torch.empty_like(x)
    a = None if amax is None else torch.tensor([float(amax)], dtype=torch.float32)
    load().qr_fp8_qdq(x.data_ptr(), x.numel(), _DT[x.dtype], None if a is None else a.data_ptr(),
                      y.data_ptr())
    return y


def int_qdq(x, amax, num_bits=8, unsigned=False, narrow_range=True):
    x = _cpu(x)
    y = torch.empty_like(x)
    load().qr_int_qdq(x.data_ptr(), x.numel(), _DT[x.dtype], float(amax), num_bits, int(unsigned),
                      int(narrow_range), y.data_ptr())
    return y


def int4_block_quantize(x, block_size):
    x = _cpu(x)
    assert x.numel() % block_size == 0
    scales = torch.empty((x.numel() // block_size, 1), dtype=x.dtype)
    packed = torch.empty(x.numel() // 2, dtype=torch.uint8)
    load().qr_int4_block_quantize(x.data_ptr(), x.numel(), _DT[x.dtype], block_size,
                                  scales.data_ptr(), packed.data_ptr())
    return packed, scales


def real_quantize(x, scale, via_dtype, fmt):
    """fmt 'e4m3' -> float8_e4m3fn tensor, 'int8' -> int8 tensor."""
    x = _cpu(x)
    out = torch.empty(x.shape, dtype=torch.uint8)
    load().qr_real_quantize(x.data_ptr(), x.numel(), _DT[x.dtype], float(scale), _DT[via_dtype],
                            0 if fmt == "e4m3" else 1, out.data_ptr())
    return out.view(torch.float8_e4m3fn if fmt == "e4m3" else torch.int8)


FORMATS = ["E4M3", "E5M2", "INT8", "E0M3", "E1M2", "E3M0", "E2M1", "E3M2", "E2M3", "E8M0"]


def block_fp_fake_quant(x, block_size, fmt, scale_fmt="E8M0", global_amax=None):
    """C twin of ``oracle.mx.block_fp_fake_quant``."""
    x = _cpu(x)
    k = x.shape[-1]
    rows = x.numel() // k
    y = torch.empty_like(x)
    g = None if global_amax is None else global_amax.to(torch.float32).reshape(-1).contiguous()
    load().qr_block_fp_qdq(x.data_ptr(), rows, k, _DT[x.dtype], block_size, FORMATS.index(fmt),
                           FORMATS.index(scale_fmt), None if g is None else g.data_ptr(),
                           0 if g is None else g.numel(), y.data_ptr())
    return y
