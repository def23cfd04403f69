"""ctypes binding of ``libmodelopt_hip.so`` (the C ABI declared in ``include/modelopt_hip.h``).

There is no CPU or eager fallback behind this module: if the library is missing or a call
fails, a ``RuntimeError`` is raised.  PyTorch is used only for device memory and streams.
"""

import ctypes
import os

import torch

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_PKG_DIR), "libmodelopt_hip.so")

MO_F32, MO_F16, MO_BF16 = 0, 1, 2
_DTYPES = {torch.float32: MO_F32, torch.float16: MO_F16, torch.bfloat16: MO_BF16}

_P, _I64, _INT = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int

# name -> argtypes; must list every function include/modelopt_hip.h declares
SIGNATURES = {
    "mo_version": [],
    "mo_error_string": [_INT],
    "mo_absmax": [_P, _I64, _I64, _I64, _INT, _P, _P],
    "mo_fp8_qdq": [_P, _P, _I64, _I64, _I64, _INT, _P, _INT, _INT, _P],
    "mo_int_qdq": [_P, _P, _I64, _I64, _I64, _INT, _P, _INT, _INT, _INT, _INT, _P],
    "mo_nvfp4_qdq": [_P, _P, _I64, _I64, _INT, _P, _INT, _INT, _INT, _P],
    "mo_nvfp4_quantize": [_P, _I64, _I64, _INT, _INT, _P, _INT, _P, _P, _P, _P, _P],
    "mo_nvfp4_dequantize": [_P, _P, _P, _I64, _I64, _INT, _P, _INT, _P],
}

_lib = None


def load():
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} not found: build it with `python tensorrt-model-optimizer_amd/build.py` "
            "(hipcc, gfx950).  There is no fallback path."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = ctypes.c_char_p if name == "mo_error_string" else _INT
    _lib = lib
    return lib


def is_available() -> bool:
    return os.path.exists(LIB_PATH)


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DTYPES[dt]
    except KeyError:
        raise TypeError(f"unsupported dtype {dt}; expected float32, float16 or bfloat16") from None


def _stream(t: torch.Tensor):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _require_device(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("modelopt_amd kernels need tensors in GPU memory (got a CPU tensor)")


def call(name: str, anchor: torch.Tensor, *args):
    """Invoke ``name`` with the device of ``anchor`` current; raise on a non-zero status."""
    lib = load()
    with torch.cuda.device(anchor.device):
        rc = getattr(lib, name)(*args)
    if rc != 0:
        msg = lib.mo_error_string(rc).decode()
        raise RuntimeError(f"{name} failed: {msg} (status {rc})")


# ----------------------------------------------------------------------------- thin wrappers


def absmax_into(x: torch.Tensor, acc: torch.Tensor, outer: int, axis: int, inner: int):
    """acc[a] = max(acc[a], max |x[o, a, i]|) for x viewed as [outer, axis, inner]."""
    _require_device(x, acc)
    assert x.is_contiguous() and acc.dtype == torch.float32 and acc.numel() == axis
    assert outer * axis * inner == x.numel()
    call("mo_absmax", x, _ptr(x), outer, axis, inner, dtype_code(x.dtype), _ptr(acc), _stream(x))
    return acc


def fp8_qdq(x, amax, outer, axis, inner, saturate=False, out=None):
    _require_device(x, amax)
    assert x.is_contiguous()
    y = torch.empty_like(x) if out is None else out
    a_dt = dtype_code(amax.dtype) if amax is not None else MO_F32
    call("mo_fp8_qdq", x, _ptr(x), _ptr(y), outer, axis, inner, dtype_code(x.dtype), _ptr(amax),
         a_dt, int(saturate), _stream(x))
    return y


def int_qdq(x, amax, outer, axis, inner, num_bits, unsigned, narrow_range, out=None):
    _require_device(x, amax)
    assert x.is_contiguous() and amax.is_contiguous()
    y = torch.empty_like(x) if out is None else out
    call("mo_int_qdq", x, _ptr(x), _ptr(y), outer, axis, inner, dtype_code(x.dtype), _ptr(amax),
         dtype_code(amax.dtype), int(num_bits), int(bool(unsigned)), int(bool(narrow_range)),
         _stream(x))
    return y


def nvfp4_qdq(x, amax, block_size=16, mode=0, out=None):
    _require_device(x, amax)
    assert x.is_contiguous()
    k = x.shape[-1]
    rows = x.numel() // k if k else 0
    y = torch.empty_like(x) if out is None else out
    call("mo_nvfp4_qdq", x, _ptr(x), _ptr(y), rows, k, dtype_code(x.dtype), _ptr(amax),
         dtype_code(amax.dtype), block_size, mode, _stream(x))
    return y


def nvfp4_quantize(x, amax_f32, block_size=16, amax_is_wsf2=False, wsf_in=None):
    """Returns (packed uint8 [..., kp/2], wsf float8_e4m3fn [..., kp/bs], wsf2 f32 scalar)."""
    _require_device(x, amax_f32, wsf_in)
    assert x.is_contiguous() and amax_f32.dtype == torch.float32
    k = x.shape[-1]
    rows = x.numel() // k if k else 0
    kp = -(-k // block_size) * block_size
    lead = tuple(x.shape[:-1])
    packed = torch.empty(lead + (kp // 2,), dtype=torch.uint8, device=x.device)
    wsf2 = torch.empty((), dtype=torch.float32, device=x.device)
    if wsf_in is None:
        wsf = torch.empty(lead + (kp // block_size,), dtype=torch.uint8, device=x.device)
        wsf_arg = None
    else:
        assert wsf_in.is_contiguous() and wsf_in.numel() == rows * (kp // block_size)
        wsf = wsf_in.view(torch.uint8)
        wsf_arg = wsf
    call("mo_nvfp4_quantize", x, _ptr(x), rows, k, dtype_code(x.dtype), block_size,
         _ptr(amax_f32), int(amax_is_wsf2), _ptr(wsf_arg), _ptr(packed),
         None if wsf_in is not None else _ptr(wsf), _ptr(wsf2), _stream(x))
    return packed, wsf.view(torch.float8_e4m3fn), wsf2


def nvfp4_dequantize(packed, wsf, wsf2, block_size, dtype):
    """packed [..., kp/2] -> [..., kp] in ``dtype``."""
    _require_device(packed, wsf, wsf2)
    assert packed.is_contiguous() and wsf.is_contiguous() and wsf2.dtype == torch.float32
    kp = packed.shape[-1] * 2
    rows = packed.numel() // packed.shape[-1] if kp else 0
    y = torch.empty(tuple(packed.shape[:-1]) + (kp,), dtype=dtype, device=packed.device)
    call("mo_nvfp4_dequantize", packed, _ptr(packed), _ptr(wsf.view(torch.uint8)), _ptr(wsf2),
         rows, kp, block_size, _ptr(y), dtype_code(dtype), _stream(packed))
    return y
