"""ctypes binding of ``libmodelopt_hip.so`` (the C ABI declared in ``include/modelopt_hip.h``).

There is no CPU or eager fallback behind this module: if the library is missing or a call
fails, a ``RuntimeError`` is raised.  PyTorch is used only for device memory and streams.
"""

import ctypes
import os

import torch

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
# MODELOPT_AMD_LIB names another build of the same library (e.g. the tuning build of build.py)
LIB_PATH = os.environ.get("MODELOPT_AMD_LIB") or os.path.join(os.path.dirname(_PKG_DIR),
                                                              "libmodelopt_hip.so")

MO_F32, MO_F16, MO_BF16 = 0, 1, 2
# per-call flags of the NVFP4 quantize entry points (enum mo_quantize_flags)
MO_FLAG_FORCE_EXACT, MO_FLAG_SATURATE_BLOCK_SCALE = 1, 2
MO_ERR_ARG, MO_ERR_DTYPE, MO_ERR_UNSUPPORTED, MO_ERR_LAUNCH, MO_ERR_TOO_LARGE = -1, -2, -3, -4, -5
_DTYPES = {torch.float32: MO_F32, torch.float16: MO_F16, torch.bfloat16: MO_BF16}

_P, _I64, _INT = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int

# name -> argtypes; must list every function include/modelopt_hip.h declares
SIGNATURES = {
    "mo_version": [],
    "mo_error_string": [_INT],
    "mo_absmax": [_P, _I64, _I64, _I64, _INT, _P, _P],
    "mo_absmax_hinted": [_P, _I64, _I64, _I64, _INT, _P, ctypes.c_uint, _P],
    "mo_absmax_pair": [_P, _I64, _P, _P, _I64, _P, _INT, _P],
    "mo_value_ranges": [_P, _P, _P, _INT, _P, _I64, _P],
    "mo_awq_pick_scale": [_P, _I64, _P, _I64, _P, _P, _P, _P, _P, _INT, _P],
    "mo_smooth_scales": [_P, _P, _I64, ctypes.c_float, _INT, ctypes.c_float, _INT, _INT, _P, _P, _P, _P, _P, _P],
    "mo_absmax_tensor_parts": [_P, _I64, _INT, _P, _P, _I64, _P, _P],
    "mo_absmax_cols_staged": [_P, _I64, _I64, _INT, _P, _P, _I64, _P],
    "mo_absmax_cols_noalloc": [_P, _I64, _I64, _INT, _P, _P],
    "mo_absmax_multi": [_P, _INT, _P, _I64, _INT, _P],
    "mo_nvfp4_quantize_multi": [_P, _INT, _P, _I64, _INT, _INT, _INT, _INT, _P],
    "mo_fp8_qdq": [_P, _P, _I64, _I64, _I64, _INT, _P, _INT, _INT, _P],
    "mo_int_qdq": [_P, _P, _I64, _I64, _I64, _INT, _P, _INT, _INT, _INT, _INT, _P],
    "mo_nvfp4_qdq": [_P, _P, _I64, _I64, _INT, _P, _INT, _INT, _INT, _P],
    "mo_qdq_sq_err": [_P, _I64, _I64, _I64, _INT, _P, _INT, _INT, _INT, _INT, _INT, _INT, _P, _P],
    "mo_mxfp4_quantize": [_P, _I64, _INT, _INT, _P, _P, _P],
    "mo_mxfp4_dequantize": [_P, _P, _I64, _INT, _P, _INT, _P],
    "mo_block_fp_qdq": [_P, _P, _I64, _I64, _INT, _INT, _INT, _INT, _P, _I64, _P],
    "mo_convert_to_format": [_P, _P, _I64, _INT, _P],
    "mo_nvfp4_quantize": [_P, _I64, _I64, _INT, _INT, _P, _INT, _P, _P, _P, _P, _INT, _P],
    "mo_nvfp4_quantize_fused": [_P, _I64, _I64, _INT, _INT, _P, _P, _P, _P, _INT, _P, _I64, _P],
    "mo_fused_amax_qdq": [_P, _P, _I64, _INT, _INT, _INT, _INT, _INT, _INT, _P, _P, _I64, _P],
    "mo_nvfp4_dequantize": [_P, _P, _P, _I64, _I64, _INT, _P, _INT, _P],
    "mo_real_quantize": [_P, _I64, _I64, _I64, _INT, _P, _INT, _INT, _INT, _P, _P],
    "mo_real_dequantize": [_P, _I64, _I64, _I64, _INT, _P, _INT, _P, _INT, _P],
    "mo_int4_block_quantize": [_P, _I64, _I64, _INT, _P, _INT, _P, _P],
    "mo_int4_block_dequantize": [_P, _I64, _I64, _P, _P, _INT, _P],
    "mo_cast_fp4": [_P, _I64, _INT, _P, _P],
    "mo_fp8_qdq_blocks2d": [_P, _P, _I64, _I64, _I64, _I64, _INT, _P, _INT, _INT, _P],
    "mo_int_qdq_blocks2d": [_P, _P, _I64, _I64, _I64, _I64, _INT, _P, _INT, _INT, _INT, _INT, _P],
    "mo_absmax_blocks2d": [_P, _I64, _I64, _I64, _I64, _INT, _P, _P],
    "mo_real_quantize_blocks2d": [_P, _I64, _I64, _I64, _I64, _INT, _P, _INT, _INT, _INT, _P, _P],
    "mo_real_dequantize_blocks2d": [_P, _I64, _I64, _I64, _I64, _INT, _P, _INT, _P, _INT, _P],
    "mo_int4_pack_rows": [_P, _I64, _I64, _I64, _I64, _INT, _P, _P, _P],
    "mo_int4_pack_rows_via": [_P, _I64, _I64, _I64, _I64, _INT, _P, _INT, _P, _P],
    "mo_nf4_quantize": [_P, _I64, _I64, _INT, _P, _P, _P],
    "mo_nf4_dequantize": [_P, _I64, _I64, _P, _P, _INT, _P],
    "mo_mul_cols": [_P, _I64, _I64, _INT, _P, _INT, _P, _P],
    "mo_scale_block_int_qdq": [_P, _I64, _I64, _INT, _P, _INT, _I64, _INT, _INT, _INT, _P, _P],
    "mo_awq_scale_grid": [_P, _P, _P, _I64, _I64, _P, _P, _P, _INT, _P],
    "mo_awq_scale_activations": [_P, _P, _I64, _I64, _I64, _INT, _P, _P],
    "mo_awq_search_losses": [_P, _P, _P, _P, _I64, _I64, _I64, _I64, _INT, _I64, _INT, _INT, _INT, _P, _P],
    "mo_awq_search_losses_biased": [_P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _INT, _I64, _INT, _INT, _INT, _P, _P],
    "mo_awq_clip_losses": [_P, _I64, _P, _I64, _I64, _INT, _I64, _P, _INT, _P, _INT, _INT, _INT, _INT, _P, _P],
    "mo_abs_colsum": [_P, _I64, _I64, _INT, _P, _I64, _P, _P],
    "mo_abs_colsum_staged": [_P, _I64, _I64, _INT, _P, _I64, _P, _P, _I64, _P],
    "mo_weight_scale_colsum": [_P, _I64, _I64, _INT, _I64, _P, _P, _I64, _P],
    "mo_sq_diff_sum": [_P, _P, _I64, _INT, _P, _P],
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
    """torch's current stream on the device of ``t`` as the C ABI takes it."""
    return ctypes.c_void_p(torch._C._cuda_getCurrentRawStream(t.device.index))


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _require_device(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("modelopt_amd kernels need tensors in GPU memory (got a CPU tensor)")


_staging = {}  # (device index, raw stream) -> int32 buffer for the two-pass reducers


def _staging_words(anchor: torch.Tensor, words: int) -> torch.Tensor:
    """``words`` 4-byte words of scratch memory on the device of ``anchor`` for a kernel pair that
    runs on torch's current stream there.  One buffer per (device, stream), grown when needed and
    reused by later calls: calls in one stream follow each other, so they can share it, and the
    calibration loop allocates nothing per call."""
    index = anchor.device.index
    if torch.cuda.is_current_stream_capturing():
        # memory from a graph's private pool belongs to that graph: a buffer made here is not kept
        # (eager calls and other graphs on this stream would share it with the replays)
        return torch.empty(words, dtype=torch.int32, device=anchor.device)
    key = (index, torch._C._cuda_getCurrentRawStream(index))
    buf = _staging.get(key)
    if buf is None or buf.numel() < words:
        buf = torch.empty(max(words, 1 << 18), dtype=torch.int32, device=anchor.device)
        _staging[key] = buf
    return buf


_timer = None  # the active KernelTimer, if any


class KernelTimer:
    """Context manager that brackets every library call made through ``call`` with a pair of
    events on the stream the kernels are launched on, and sums the elapsed device time of those
    calls per entry point when it exits (one synchronisation, at exit).  Measurement aid: a call
    costs two extra event records while it is active."""

    def __init__(self):
        self.pairs = []      # (entry point, start event, end event)
        self.seconds = {}    # entry point -> summed device seconds
        self.calls = {}

    def __enter__(self):
        global _timer
        self._previous, _timer = _timer, self
        return self

    def __exit__(self, *exc):
        global _timer
        _timer = self._previous
        torch.cuda.synchronize()
        for name, start, end in self.pairs:
            self.seconds[name] = self.seconds.get(name, 0.0) + start.elapsed_time(end) * 1e-3
            self.calls[name] = self.calls.get(name, 0) + 1
        self.pairs = []
        return False

    @property
    def total_seconds(self):
        return sum(self.seconds.values())


def call(name: str, anchor: torch.Tensor, *args):
    """Invoke ``name`` with the device of ``anchor`` current; raise on a non-zero status."""
    lib = load()
    if _timer is None and anchor.device.index == torch.cuda.current_device():
        rc = getattr(lib, name)(*args)   # the common case, without the context manager's cost
    else:
        with torch.cuda.device(anchor.device):
            if _timer is None:
                rc = getattr(lib, name)(*args)
            else:
                start = torch.cuda.Event(enable_timing=True)
                end = torch.cuda.Event(enable_timing=True)
                start.record()
                rc = getattr(lib, name)(*args)
                end.record()
                _timer.pairs.append((name, start, end))
    if rc != 0:
        msg = lib.mo_error_string(rc).decode()
        raise RuntimeError(f"{name} failed: {msg} (status {rc})")


# ----------------------------------------------------------------------------- thin wrappers


MO_ABSMAX_REREAD = 1


def absmax_into(x: torch.Tensor, acc: torch.Tensor, outer: int, axis: int, inner: int, reread: bool = False):
    """acc[a] = max(acc[a], max |x[o, a, i]|) for x viewed as [outer, axis, inner].  ``reread``:
    the caller reads ``x`` again right away (a dynamic quantizer's fake quant), so a per-tensor
    reduction leaves it in the memory-side cache instead of streaming it past."""
    _require_device(x, acc)
    assert x.is_contiguous() and acc.dtype == torch.float32 and acc.numel() == axis
    assert outer * axis * inner == x.numel()
    if inner == 1 and axis % 8 == 0 and outer >= 64 and x.data_ptr() % 16 == 0:
        # per column over many rows: row slabs go to a small workspace first, so that a fresh
        # accumulator is not hit by one atomic per column from every workgroup
        # about two workgroups per compute unit in all, 32 rows or more per slab (measured best
        # from 17 MB to 537 MB)
        across = -(-axis // 2048) if axis >= 2048 else -(-axis // 512)
        slabs = max(1, min(-(-512 // across), outer // 32))
        partial = _staging_words(x, slabs * axis)
        call("mo_absmax_cols_staged", x, _ptr(x), outer, axis, dtype_code(x.dtype), _ptr(acc),
             _ptr(partial), slabs, _stream(x))
        return acc
    if reread and axis == 1:
        call("mo_absmax_hinted", x, _ptr(x), outer, axis, inner, dtype_code(x.dtype), _ptr(acc),
             MO_ABSMAX_REREAD, _stream(x))
        return acc
    call("mo_absmax", x, _ptr(x), outer, axis, inner, dtype_code(x.dtype), _ptr(acc), _stream(x))
    return acc


def absmax_pair_into(x0: torch.Tensor, acc0: torch.Tensor, x1: torch.Tensor, acc1: torch.Tensor):
    """Per-tensor ``absmax_into`` of two dense tensors of one dtype (each into its own one-element
    accumulator) in one launch.  False, with nothing launched, when the pair is not covered."""
    _require_device(x0, acc0, x1, acc1)
    if (x0.dtype != x1.dtype or x0.dtype not in _DTYPES or x0.device != x1.device
            or x0.data_ptr() % 16 or x1.data_ptr() % 16 or acc0.numel() != 1 or acc1.numel() != 1):
        return False
    assert x0.is_contiguous() and x1.is_contiguous()
    assert acc0.dtype == torch.float32 and acc1.dtype == torch.float32
    call("mo_absmax_pair", x0, _ptr(x0), x0.numel(), _ptr(acc0), _ptr(x1), x1.numel(), _ptr(acc1),
         dtype_code(x0.dtype), _stream(x0))
    return True


VALUE_RANGES_MAX = 32          # tensors per mo_value_ranges launch
VALUE_RANGES_CHUNK = 4096      # elements per workgroup, as in the kernel
VALUE_RANGES_MAX_CHUNKS = 1024


def value_ranges(tensors):
    """``[(min, max, has_nan), ...]`` of the given tensors (floats; NaN elements are left out of
    min and max) from one launch and ONE host synchronisation; None, with nothing launched, when
    the list is not covered (more than 32 tensors or 4 M elements in all, several devices, another
    dtype, a non-contiguous tensor)."""
    n = len(tensors)
    if n == 0:
        return []
    device = tensors[0].device
    if n > VALUE_RANGES_MAX or device.type != "cuda":
        return None
    chunks = []
    for t in tensors:
        if t.device != device or t.dtype not in _DTYPES or not t.is_contiguous():
            return None
        chunks.append(max(1, -(-t.numel() // VALUE_RANGES_CHUNK)))
    total = sum(chunks)
    if total > VALUE_RANGES_MAX_CHUNKS:
        return None
    # a buffer of its own per call (the caching allocator hands it out in microseconds): calls from
    # two streams must not share one
    out = torch.empty(3 * total, dtype=torch.float32, device=device)
    ptrs = (ctypes.c_void_p * n)(*[t.data_ptr() for t in tensors])
    counts = (ctypes.c_int64 * n)(*[t.numel() for t in tensors])
    dtypes = (ctypes.c_int * n)(*[dtype_code(t.dtype) for t in tensors])
    call("mo_value_ranges", tensors[0], ptrs, counts, dtypes, n, _ptr(out), total, _stream(tensors[0]))
    flat = out.tolist()
    result, at = [], 0
    for c in chunks:
        part = flat[3 * at:3 * (at + c)]
        result.append((min(part[0::3]), max(part[1::3]), any(part[2::3])))
        at += c
    return result


_parts_ring = {}   # device index -> [int32 buffer, words handed out]
_PARTS_RING_WORDS = 1 << 20


def absmax_tensor_parts_into(x: torch.Tensor, acc: torch.Tensor):
    """Per-tensor ``absmax_into`` that also returns the abs-max of every 32768-element tile of
    ``x`` (int32 bit patterns of non-negative floats, a slice of a ring buffer that stays alive as
    long as the slice does): ``parts.max()`` is the abs-max of this tensor alone.  None when the
    tensor is not covered (the accumulator is untouched then)."""
    _require_device(x, acc)
    if not x.is_contiguous() or x.dtype not in _DTYPES or x.data_ptr() % 16 or acc.numel() != 1:
        return None
    n = x.numel()
    tiles = -(-n // 32768)
    if tiles == 0 or tiles > _PARTS_RING_WORDS:
        return None
    index = x.device.index
    ring = _parts_ring.get(index)
    if ring is None or ring[1] + tiles > _PARTS_RING_WORDS:
        # slices handed out earlier keep their buffer alive; a new one starts here
        ring = [torch.empty(_PARTS_RING_WORDS, dtype=torch.int32, device=x.device), 0]
        _parts_ring[index] = ring
    parts = ring[0][ring[1]:ring[1] + tiles]
    written = ctypes.c_int64(0)
    call("mo_absmax_tensor_parts", x, _ptr(x), n, dtype_code(x.dtype), _ptr(acc), _ptr(parts), tiles,
         ctypes.byref(written), _stream(x))
    assert written.value == tiles
    ring[1] += tiles
    return parts


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


def blocks2d_covered(x, rows, cols, block_rows, block_cols) -> bool:
    """Whether the two-dimensional block kernels take ``x`` viewed as [rows, cols]."""
    return (rows > 0 and cols > 0 and rows % block_rows == 0 and cols % block_cols == 0
            and block_cols % 8 == 0 and x.data_ptr() % 16 == 0 and x.is_contiguous())


def fp8_qdq_blocks2d(x, amax, rows, cols, block_rows, block_cols, saturate=False):
    """FP8 fake quant of contiguous ``x`` seen as [rows, cols] with one amax per block of
    ``block_rows x block_cols`` (``amax`` flat, block rows major)."""
    _require_device(x, amax)
    assert x.is_contiguous() and amax.is_contiguous() and x.numel() == rows * cols
    y = torch.empty_like(x)
    call("mo_fp8_qdq_blocks2d", x, _ptr(x), _ptr(y), rows, cols, block_rows, block_cols,
         dtype_code(x.dtype), _ptr(amax), dtype_code(amax.dtype), int(saturate), _stream(x))
    return y


def int_qdq_blocks2d(x, amax, rows, cols, block_rows, block_cols, num_bits, unsigned, narrow_range):
    _require_device(x, amax)
    assert x.is_contiguous() and amax.is_contiguous() and x.numel() == rows * cols
    y = torch.empty_like(x)
    call("mo_int_qdq_blocks2d", x, _ptr(x), _ptr(y), rows, cols, block_rows, block_cols,
         dtype_code(x.dtype), _ptr(amax), dtype_code(amax.dtype), int(num_bits), int(bool(unsigned)),
         int(bool(narrow_range)), _stream(x))
    return y


def absmax_blocks2d_into(x, acc, rows, cols, block_rows, block_cols):
    """``acc[b] = max(acc[b], abs-max of block b)``, fp32 ``acc`` with one element per block."""
    _require_device(x, acc)
    assert x.is_contiguous() and acc.dtype == torch.float32 and acc.is_contiguous()
    assert acc.numel() == (rows // block_rows) * (cols // block_cols)
    call("mo_absmax_blocks2d", x, _ptr(x), rows, cols, block_rows, block_cols, dtype_code(x.dtype),
         _ptr(acc), _stream(x))
    return acc


def nvfp4_qdq(x, amax, block_size=16, mode=0, out=None):
    _require_device(x, amax)
    assert x.is_contiguous()
    k = x.shape[-1]
    rows = x.numel() // k if k else 0
    y = torch.empty_like(x) if out is None else out
    call("mo_nvfp4_qdq", x, _ptr(x), _ptr(y), rows, k, dtype_code(x.dtype), _ptr(amax),
         dtype_code(amax.dtype), block_size, mode, _stream(x))
    return y


def qdq_sq_err_into(x, cand, loss, outer, axis, inner, kind, num_bits=8, unsigned=False,
                    narrow_range=False, saturate=False):
    """loss[k, a] += sum (x - QDQ(x; cand[k, a]))^2 for every candidate k; ``cand`` and ``loss`` are
    fp32 [n_cand, axis].  Returns False when the layout is not covered by the kernel."""
    _require_device(x, cand, loss)
    assert x.is_contiguous() and cand.is_contiguous() and loss.is_contiguous()
    assert cand.dtype == torch.float32 and loss.dtype == torch.float32
    assert cand.numel() == loss.numel() and cand.numel() % axis == 0
    rc = load().mo_qdq_sq_err(_ptr(x), outer, axis, inner, dtype_code(x.dtype), _ptr(cand),
                              cand.numel() // axis, 0 if kind == "int" else 1, int(num_bits),
                              int(bool(unsigned)), int(bool(narrow_range)), int(bool(saturate)),
                              _ptr(loss), _stream(x))
    if rc == MO_ERR_UNSUPPORTED:
        return False
    if rc != 0:
        raise RuntimeError(f"mo_qdq_sq_err failed: {load().mo_error_string(rc).decode()}")
    return True


ELEM_FORMATS = ["E4M3", "E5M2", "INT8", "E0M3", "E1M2", "E3M0", "E2M1", "E3M2", "E2M3", "E8M0"]


def block_fp_qdq(x, block_size, fmt, scale_fmt="E8M0", global_amax=None, out=None):
    """Block floating point fake quantisation along the last dim (``fused_amax_convert``).
    ``fmt`` / ``scale_fmt``: names or indices of ``ELEM_FORMATS``; ``global_amax``: None, one
    fp32 element, or one per row of a 2-D ``x``."""
    _require_device(x, global_amax)
    assert x.is_contiguous()
    fmt = ELEM_FORMATS.index(fmt) if isinstance(fmt, str) else int(fmt)
    scale_fmt = ELEM_FORMATS.index(scale_fmt) if isinstance(scale_fmt, str) else int(scale_fmt)
    k = x.shape[-1]
    rows = x.numel() // k if k else 0
    y = torch.empty_like(x) if out is None else out
    n_global = 0
    if global_amax is not None:
        assert global_amax.dtype == torch.float32 and global_amax.is_contiguous()
        n_global = global_amax.numel()
        if not (n_global == 1 or (x.dim() == 2 and n_global == x.shape[0])):
            raise ValueError("global_amax needs one element, or one per row of a 2-D input")
    call("mo_block_fp_qdq", x, _ptr(x), _ptr(y), rows, k, dtype_code(x.dtype), block_size, fmt,
         scale_fmt, _ptr(global_amax), n_global, _stream(x))
    return y


def convert_to_format(x, fmt):
    """Nearest value of element format ``fmt`` (name or index of ``ELEM_FORMATS``) for every
    element of the fp32 device tensor ``x``."""
    _require_device(x)
    assert x.dtype == torch.float32 and x.is_contiguous()
    fmt = ELEM_FORMATS.index(fmt) if isinstance(fmt, str) else int(fmt)
    y = torch.empty_like(x)
    call("mo_convert_to_format", x, _ptr(x), _ptr(y), x.numel(), fmt, _stream(x))
    return y


def mxfp4_quantize(x, block_size=32):
    """-> (packed uint8 [..., k / 2], E8M0 scale bytes uint8 [numel / block_size, 1])."""
    _require_device(x)
    assert x.is_contiguous() and x.numel() % block_size == 0 and x.shape[-1] % 2 == 0
    packed = torch.empty(x.shape[:-1] + (x.shape[-1] // 2,), dtype=torch.uint8, device=x.device)
    scales = torch.empty((x.numel() // block_size, 1), dtype=torch.uint8, device=x.device)
    call("mo_mxfp4_quantize", x, _ptr(x), x.numel(), dtype_code(x.dtype), block_size, _ptr(packed),
         _ptr(scales), _stream(x))
    return packed, scales


def mxfp4_dequantize(packed, scales, block_size, dtype):
    _require_device(packed, scales)
    assert packed.is_contiguous() and scales.is_contiguous() and scales.dtype == torch.uint8
    y = torch.empty(packed.shape[:-1] + (packed.shape[-1] * 2,), dtype=dtype, device=packed.device)
    call("mo_mxfp4_dequantize", packed, _ptr(packed), _ptr(scales), y.numel(), block_size, _ptr(y),
         dtype_code(dtype), _stream(packed))
    return y


def nvfp4_quantize(x, amax_f32, block_size=16, amax_is_wsf2=False, wsf_in=None, flags=0):
    """Returns (packed uint8 [..., kp/2], wsf float8_e4m3fn [..., kp/bs], wsf2 f32 scalar).
    ``flags``: ``MO_FLAG_*`` bits."""
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
         None if wsf_in is not None else _ptr(wsf), _ptr(wsf2), int(flags), _stream(x))
    return packed, wsf.view(torch.float8_e4m3fn), wsf2


# --------------------------------------------------------------- one-launch amax -> quantize
FUSED_WS_BYTES, FUSED_WS_FAIL_OFFSET = 512, 384   # MO_FUSED_WS_BYTES, MO_FUSED_WS_FAIL_OFFSET
# polls (about a microsecond each with the round trip of the load) a workgroup waits for the
# others before it takes the abs-max of the whole tensor by itself: some 20 ms
FUSED_SPIN_LIMIT = 1 << 14
_fused_ws_by_device = {}


def fused_scratch(device, stream=None):
    """The workspace of the fused kernels for ``device`` and ``stream`` (default: torch's current
    stream there).  Calls in one stream follow each other and can share it; calls in different
    streams may overlap and get one each (overlapping calls can keep each other's workgroups off
    the device: each then ends its wait after ``FUSED_SPIN_LIMIT`` polls and finishes on its own,
    with the same results)."""
    index = torch.device(device).index
    index = torch.cuda.current_device() if index is None else index
    if stream is None:
        if torch.cuda.is_current_stream_capturing():
            # the fill that zeroes a new workspace becomes a node of the graph and does not run
            # now, so a workspace made here would reach later eager calls unzeroed: each captured
            # call gets its own, zeroed by its own node on every replay, and none is kept
            return torch.zeros(FUSED_WS_BYTES // 4, dtype=torch.int32, device=torch.device("cuda", index))
        stream = torch._C._cuda_getCurrentRawStream(index)
    ws = _fused_ws_by_device.get((index, stream))
    if ws is None:
        ws = torch.zeros(FUSED_WS_BYTES // 4, dtype=torch.int32, device=torch.device("cuda", index))
        assert ws.data_ptr() % 128 == 0
        _fused_ws_by_device[(index, stream)] = ws
    return ws


def fused_gave_up(device=None) -> bool:
    """Whether a workgroup of a fused kernel (on ``device``; default: any device) stopped waiting
    for the others and took the abs-max of the whole tensor by itself since the last look.  The
    outputs of such a call are right, but it was slow (the wait plus a pass over the tensor per
    workgroup): a caller that sees this repeatedly should stay with the two-launch path.
    Synchronises; clears the flag.  Calls recorded into a graph use workspaces of their own that
    this check does not see."""
    index = None if device is None else torch.device(device).index
    failed = False
    for (dev, _), ws in _fused_ws_by_device.items():
        if index is not None and dev != index:
            continue
        if bool(ws[FUSED_WS_FAIL_OFFSET // 4].item()):
            ws[FUSED_WS_FAIL_OFFSET // 4] = 0
            failed = True
    return failed


def _fused_rc(name, rc):
    if rc in (MO_ERR_UNSUPPORTED, MO_ERR_TOO_LARGE):
        return False
    if rc != 0:
        raise RuntimeError(f"{name} failed: {load().mo_error_string(rc).decode()} (status {rc})")
    return True


def nvfp4_quantize_fused(x, flags=0, spin_limit=FUSED_SPIN_LIMIT):
    """Per-tensor abs-max and NVFP4 quantize + pack of a bf16 tensor in one launch that reads it
    once.  Returns (packed, wsf, wsf2, amax fp32 scalar), or None when the tensor is too large
    for the registers of the chip or the layout is not covered (use the two-launch path then)."""
    _require_device(x)
    k = x.shape[-1] if x.dim() else 0
    if x.dtype != torch.bfloat16 or not x.is_contiguous() or k == 0 or k % 16 or x.data_ptr() % 16:
        return None
    rows = x.numel() // k
    lead = tuple(x.shape[:-1])
    packed = torch.empty(lead + (k // 2,), dtype=torch.uint8, device=x.device)
    wsf = torch.empty(lead + (k // 16,), dtype=torch.uint8, device=x.device)
    wsf2 = torch.empty((), dtype=torch.float32, device=x.device)
    amax = torch.empty((), dtype=torch.float32, device=x.device)
    ws = fused_scratch(x.device)
    with torch.cuda.device(x.device):
        rc = load().mo_nvfp4_quantize_fused(_ptr(x), rows, k, MO_BF16, 16, _ptr(packed), _ptr(wsf),
                                            _ptr(wsf2), _ptr(amax), int(flags), _ptr(ws),
                                            int(spin_limit), _stream(x))
    if not _fused_rc("mo_nvfp4_quantize_fused", rc):
        return None
    return packed, wsf.view(torch.float8_e4m3fn), wsf2, amax


def fused_amax_qdq(x, kind, num_bits=8, unsigned=False, narrow_range=False, saturate=False,
                   out=None, spin_limit=FUSED_SPIN_LIMIT):
    """Dynamic per-tensor fake quantisation in one launch (``kind`` "int" or "fp8"): returns
    (y, amax fp32 scalar), or None when the tensor does not fit / the layout is not covered
    (``out`` overlapping ``x`` is not: a workgroup whose wait expired reads ``x`` again)."""
    _require_device(x)
    if not x.is_contiguous() or x.dtype not in _DTYPES or x.data_ptr() % 16 or x.numel() == 0:
        return None
    y = torch.empty_like(x) if out is None else out
    amax = torch.empty((), dtype=torch.float32, device=x.device)
    ws = fused_scratch(x.device)
    with torch.cuda.device(x.device):
        rc = load().mo_fused_amax_qdq(_ptr(x), _ptr(y), x.numel(), dtype_code(x.dtype),
                                      0 if kind == "int" else 1, int(num_bits), int(bool(unsigned)),
                                      int(bool(narrow_range)), int(bool(saturate)), _ptr(amax),
                                      _ptr(ws), int(spin_limit), _stream(x))
    if not _fused_rc("mo_fused_amax_qdq", rc):
        return None
    return y, amax


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


def cast_fp4(x):
    """E2M1 codes (sign << 3 | ordinal, ties to even), one uint8 per element of ``x``."""
    _require_device(x)
    assert x.is_contiguous()
    codes = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    call("mo_cast_fp4", x, _ptr(x), x.numel(), dtype_code(x.dtype), _ptr(codes), _stream(x))
    return codes


MO_FMT_E4M3, MO_FMT_INT8 = 0, 1


def real_quantize(x, scale, outer, axis, inner, via_dtype, fmt):
    """q = fmt(via(x / scale)); returns float8_e4m3fn or int8 tensor of x's shape."""
    _require_device(x, scale)
    assert x.is_contiguous() and scale.is_contiguous() and scale.numel() == axis
    out = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    call("mo_real_quantize", x, _ptr(x), outer, axis, inner, dtype_code(x.dtype), _ptr(scale),
         dtype_code(scale.dtype), dtype_code(via_dtype), fmt, _ptr(out), _stream(x))
    return out.view(torch.float8_e4m3fn if fmt == MO_FMT_E4M3 else torch.int8)


def real_quantize_blocks2d(x, scale, rows, cols, block_rows, block_cols, via_dtype, fmt):
    """``fmt(via(x / scale[block]))`` for contiguous ``x`` seen as [rows, cols] with one scale per
    block of ``block_rows x block_cols`` (flat, block rows major); uint8 bytes of x's shape viewed
    as float8_e4m3fn or int8."""
    _require_device(x, scale)
    assert x.is_contiguous() and scale.is_contiguous() and x.numel() == rows * cols
    assert scale.numel() == (rows // block_rows) * (cols // block_cols)
    out = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    call("mo_real_quantize_blocks2d", x, _ptr(x), rows, cols, block_rows, block_cols, dtype_code(x.dtype),
         _ptr(scale), dtype_code(scale.dtype), dtype_code(via_dtype), fmt, _ptr(out), _stream(x))
    return out.view(torch.float8_e4m3fn if fmt == MO_FMT_E4M3 else torch.int8)


def real_dequantize_blocks2d(q, scale, rows, cols, block_rows, block_cols, fmt, dtype):
    _require_device(q, scale)
    assert q.is_contiguous() and scale.is_contiguous() and q.numel() == rows * cols
    assert scale.numel() == (rows // block_rows) * (cols // block_cols)
    y = torch.empty(q.shape, dtype=dtype, device=q.device)
    call("mo_real_dequantize_blocks2d", q, _ptr(q.view(torch.uint8)), rows, cols, block_rows, block_cols,
         fmt, _ptr(scale), dtype_code(scale.dtype), _ptr(y), dtype_code(dtype), _stream(q))
    return y


def real_dequantize(q, scale, outer, axis, inner, fmt, dtype):
    _require_device(q, scale)
    assert q.is_contiguous() and scale.is_contiguous() and scale.numel() == axis
    y = torch.empty(q.shape, dtype=dtype, device=q.device)
    call("mo_real_dequantize", q, _ptr(q.view(torch.uint8)), outer, axis, inner, fmt, _ptr(scale),
         dtype_code(scale.dtype), _ptr(y), dtype_code(dtype), _stream(q))
    return y


def int4_block_quantize(x, block_size, scales=None):
    """Flat-block INT4 quantize + pack: returns (packed uint8 [padded_numel / 2], scales [nblocks, 1]).
    ``scales`` (``7 / amax`` per block, dtype of ``x``) are computed unless given."""
    _require_device(x, scales)
    assert x.is_contiguous()
    n = x.numel()
    nblocks = -(-n // block_size)
    given = scales is not None
    if given:
        assert scales.is_contiguous() and scales.dtype == x.dtype and scales.numel() == nblocks
    else:
        scales = torch.empty((nblocks, 1), dtype=x.dtype, device=x.device)
    packed = torch.empty(nblocks * block_size // 2, dtype=torch.uint8, device=x.device)
    call("mo_int4_block_quantize", x, _ptr(x), n, block_size, dtype_code(x.dtype), _ptr(scales),
         int(given), _ptr(packed), _stream(x))
    return packed, scales


def int4_block_dequantize(packed, scales, block_size):
    _require_device(packed, scales)
    assert packed.is_contiguous() and scales.is_contiguous()
    y = torch.empty(packed.numel() * 2, dtype=scales.dtype, device=packed.device)
    call("mo_int4_block_dequantize", packed, _ptr(packed), packed.numel(), block_size, _ptr(scales),
         _ptr(y), dtype_code(scales.dtype), _stream(packed))
    return y


def nf4_quantize(x, block_size):
    """Flat-block NF4 quantize + pack: returns (packed uint8 [padded_numel / 2], per-block
    abs-max [nblocks] in the dtype of x)."""
    _require_device(x)
    assert x.is_contiguous()
    n = x.numel()
    nblocks = -(-n // block_size)
    scales = torch.empty(nblocks, dtype=x.dtype, device=x.device)
    packed = torch.empty(nblocks * block_size // 2, dtype=torch.uint8, device=x.device)
    call("mo_nf4_quantize", x, _ptr(x), n, block_size, dtype_code(x.dtype), _ptr(scales),
         _ptr(packed), _stream(x))
    return packed, scales


def nf4_dequantize(packed, scales, block_size):
    """``table[code] * scale`` in the dtype of ``scales``: [2 * packed.numel()]."""
    _require_device(packed, scales)
    assert packed.is_contiguous() and scales.is_contiguous()
    assert scales.numel() * block_size >= packed.numel() * 2
    y = torch.empty(packed.numel() * 2, dtype=scales.dtype, device=packed.device)
    call("mo_nf4_dequantize", packed, _ptr(packed), packed.numel(), block_size, _ptr(scales),
         _ptr(y), dtype_code(scales.dtype), _stream(packed))
    return y


def int4_pack_rows(w, ws, via_dtype=torch.float32):
    """INT4-AWQ export pack: w [..., N, K], ws fp32 [..., N, K / bs] -> uint8 [..., N / 2, K].
    ``via_dtype``: the type the quotient is rounded to before it is rounded to an integer, fp32
    or ``w.dtype`` (scales that came in the weight's own 16-bit type)."""
    _require_device(w, ws)
    assert w.is_contiguous() and ws.is_contiguous() and ws.dtype == torch.float32
    n, k = w.shape[-2], w.shape[-1]
    batch = w.numel() // (n * k) if n * k else 0
    bs = k // ws.shape[-1]
    out = torch.empty(tuple(w.shape[:-2]) + (n // 2, k), dtype=torch.uint8, device=w.device)
    call("mo_int4_pack_rows_via", w, _ptr(w), batch, n, k, bs, dtype_code(w.dtype), _ptr(ws),
         dtype_code(via_dtype), _ptr(out), _stream(w))
    return out


def awq_pick_scale(loss: torch.Tensor, scales: torch.Tensor, dtype: torch.dtype):
    """The end of an AWQ-lite search in one launch: ``(best, best_scale, pre_quant_scale,
    pre_quant_scale_t, fold)`` for float64 ``loss`` [A] and the fp32 candidate grid ``scales``
    [A, K]: ``best`` the index of the first smallest loss (0-dim int64 on the device; a NaN is
    never smaller, a NaN in front stays), ``best_scale = scales[best]``, ``pre_quant_scale =
    1 / best_scale``, the same rounded to ``dtype``, and ``fold = 1 / pre_quant_scale``."""
    _require_device(loss, scales)
    assert loss.dtype == torch.float64 and scales.dtype == torch.float32
    assert loss.is_contiguous() and scales.is_contiguous() and scales.dim() == 2
    n_alpha, k = scales.shape
    assert loss.numel() == n_alpha and n_alpha > 0
    rows = torch.empty(3, k, dtype=torch.float32, device=scales.device)
    rounded = torch.empty(k, dtype=dtype, device=scales.device)
    best = torch.empty((), dtype=torch.int64, device=scales.device)
    call("mo_awq_pick_scale", scales, _ptr(loss), n_alpha, _ptr(scales), k, _ptr(best), _ptr(rows[0]),
         _ptr(rows[1]), _ptr(rounded), _ptr(rows[2]), dtype_code(dtype), _stream(scales))
    return best, rows[0], rows[1], rounded, rows[2]


def _power_mode(exponent: float) -> int:
    """How a scalar power is evaluated: 0 ``pow``, 1 the constant one (exponent 0), 2 the base
    (exponent 1), 3 the correctly rounded square root (exponent 0.5)."""
    return {0.0: 1, 1.0: 2, 0.5: 3}.get(float(exponent), 0)


def smooth_scales(act_amax: torch.Tensor, weight_col_amax: torch.Tensor, alpha: float, dtype: torch.dtype):
    """SmoothQuant's scale of one linear and what the smoothing makes of it, in one launch:
    ``(pre_quant_scale fp32 [K], the same in dtype, 1 / pre_quant_scale fp32, dtype(max act_amax),
    dtype(max(dtype(act_amax) * pre_quant_scale)))`` from the fp32 per-channel input amax and the
    fp32 per-column abs-max of the weight."""
    _require_device(act_amax, weight_col_amax)
    assert act_amax.dtype == torch.float32 and weight_col_amax.dtype == torch.float32
    assert act_amax.is_contiguous() and weight_col_amax.is_contiguous()
    k = act_amax.numel()
    assert weight_col_amax.numel() == k and k > 0
    rows = torch.empty(2, k, dtype=torch.float32, device=act_amax.device)
    rounded = torch.empty(k, dtype=dtype, device=act_amax.device)
    maxima = torch.empty(2, dtype=dtype, device=act_amax.device)
    exp_w, exp_a = 1 - alpha, alpha
    mode_w = _power_mode(exp_w)
    if mode_w == 0 and dtype != torch.float32:
        # a power of a 16-bit tensor is taken with the exponent rounded to that dtype
        exp_w = float(torch.tensor(exp_w, dtype=dtype))
    call("mo_smooth_scales", act_amax, _ptr(act_amax), _ptr(weight_col_amax), k, exp_w, mode_w,
         exp_a, _power_mode(exp_a), dtype_code(dtype), _ptr(rows[0]), _ptr(rounded), _ptr(rows[1]),
         _ptr(maxima[0]), _ptr(maxima[1]), _stream(act_amax))
    return rows[0], rounded, rows[1], maxima[0], maxima[1]


def awq_scale_grid(x_max, w_max, exponents, dtype):
    """AWQ-lite candidate scales for every alpha of a grid: (fp32 scales [A, K], ``dtype`` copy,
    ``dtype`` copy of the reciprocals).  ``exponents``: fp32 device tensor [4, A] (alpha,
    1 - alpha, and the evaluation mode of each power, see ``mo_awq_scale_grid``)."""
    _require_device(x_max, w_max, exponents)
    assert x_max.dtype == w_max.dtype == exponents.dtype == torch.float32
    assert x_max.is_contiguous() and w_max.is_contiguous() and exponents.is_contiguous()
    n_alpha, k = exponents.shape[1], x_max.numel()
    assert exponents.shape[0] == 4 and w_max.numel() == k
    scales = torch.empty((n_alpha, k), dtype=torch.float32, device=x_max.device)
    w_scales = torch.empty((n_alpha, k), dtype=dtype, device=x_max.device)
    x_scales = torch.empty((n_alpha, k), dtype=dtype, device=x_max.device)
    call("mo_awq_scale_grid", x_max, _ptr(x_max), _ptr(w_max), _ptr(exponents), n_alpha, k,
         _ptr(scales), _ptr(w_scales), _ptr(x_scales), dtype_code(dtype), _stream(x_max))
    return scales, w_scales, x_scales


def awq_scaled_activations(x, inv_s):
    """``T(x * inv_s[a])`` for every row a of ``inv_s`` in the layout the search kernel reads:
    [n_alpha, K / 8, tokens, 8] (the 8-element chunks of a column group are contiguous over
    tokens, so that the lanes of a matrix-core operand read adjacent memory)."""
    _require_device(x, inv_s)
    n_alpha, k = inv_s.shape
    tokens = x.shape[0]
    assert x.is_contiguous() and inv_s.is_contiguous() and x.shape == (tokens, k) and k % 8 == 0
    assert x.dtype == inv_s.dtype == torch.bfloat16, "the search kernel takes bf16 activations"
    xs = torch.empty((n_alpha, k // 8, tokens, 8), dtype=x.dtype, device=x.device)
    call("mo_awq_scale_activations", x, _ptr(x), _ptr(inv_s), n_alpha, tokens, k, MO_BF16, _ptr(xs),
         _stream(x))
    return xs


def awq_search_losses_into(xs, w, s, ref, block_size, num_bits, unsigned, narrow_range, loss, bias=None):
    """loss[a] += squared error of ``bf16(x_a @ qdq(bf16(w * s[a]))^T + bias)`` against ``ref``,
    all alphas in one launch; ``xs`` = ``awq_scaled_activations(x, 1 / s)``.  Returns False
    (nothing launched) when the shapes or dtype are outside what the kernel covers."""
    _require_device(xs, w, s, ref, loss, bias)
    n_alpha, kc, tokens, eight = xs.shape
    k = kc * 8
    n = w.shape[0]
    assert eight == 8
    assert xs.is_contiguous() and w.is_contiguous() and s.is_contiguous() and ref.is_contiguous()
    assert w.shape == (n, k) and s.shape == (n_alpha, k) and ref.shape == (tokens, n)
    assert loss.dtype == torch.float64 and loss.numel() == n_alpha and loss.is_contiguous()
    if not (xs.dtype == w.dtype == s.dtype == ref.dtype == torch.bfloat16):
        return False
    if bias is not None and (bias.dtype != torch.bfloat16 or bias.numel() != n or not bias.is_contiguous()):
        return False
    lib = load()
    with torch.cuda.device(xs.device):
        rc = lib.mo_awq_search_losses_biased(_ptr(xs), _ptr(w), _ptr(s), _ptr(ref), _ptr(bias), n_alpha,
                                             tokens, n, k, MO_BF16, block_size, int(num_bits),
                                             int(bool(unsigned)), int(bool(narrow_range)), _ptr(loss),
                                             _stream(xs))
    if rc == MO_ERR_UNSUPPORTED:
        return False
    if rc != 0:
        raise RuntimeError(f"mo_awq_search_losses failed: {lib.mo_error_string(rc).decode()} (status {rc})")
    return True


def awq_clip_losses_into(x, w, w_amax, ratios, block_size, num_bits, unsigned, narrow_range, loss):
    """``loss[r, row, b] +=`` the mean over the tokens of ``x`` of the squared error that block
    ``(row, b)`` of ``w``, fake-quantised with ``ratios[r] * w_amax[row, b]``, makes on its
    partial output -- every ratio and block in one launch.  x: [tokens, k], w: [n, k] of the same
    dtype; w_amax: n * k / block_size values; loss: fp32 [len(ratios), n, k / block_size].
    Returns False (nothing written) for shapes the kernel does not cover."""
    _require_device(x, w, w_amax, loss)
    n, k = w.shape
    tokens = x.shape[0]
    assert x.dim() == 2 and x.shape[1] == k and x.dtype == w.dtype
    assert x.is_contiguous() and w.is_contiguous() and w_amax.is_contiguous() and loss.is_contiguous()
    if k % block_size or block_size not in (16, 32, 64, 128) or len(ratios) > 32:
        return False
    assert w_amax.numel() == n * (k // block_size)
    assert loss.dtype == torch.float32 and tuple(loss.shape) == (len(ratios), n, k // block_size)
    host = (ctypes.c_float * len(ratios))(*[float(r) for r in ratios])
    lib = load()
    with torch.cuda.device(x.device):
        rc = lib.mo_awq_clip_losses(_ptr(x), tokens, _ptr(w), n, k, dtype_code(w.dtype), block_size,
                                    _ptr(w_amax), dtype_code(w_amax.dtype), host, len(ratios),
                                    int(num_bits), int(bool(unsigned)), int(bool(narrow_range)),
                                    _ptr(loss), _stream(x))
    if rc == MO_ERR_UNSUPPORTED:
        return False
    if rc != 0:
        raise RuntimeError(f"mo_awq_clip_losses failed: {lib.mo_error_string(rc).decode()} (status {rc})")
    return True


def mul_cols(x, s, out=None):
    """y[..., c] = T(x[..., c] * s[c])."""
    _require_device(x, s)
    assert x.is_contiguous() and s.is_contiguous() and s.numel() == x.shape[-1]
    k = x.shape[-1]
    y = torch.empty_like(x) if out is None else out
    call("mo_mul_cols", x, _ptr(x), x.numel() // k if k else 0, k, dtype_code(x.dtype), _ptr(s),
         dtype_code(s.dtype), _ptr(y), _stream(x))
    return y


def scale_block_int_qdq(x, s, block_size, num_bits=4, unsigned=False, narrow_range=False, out=None):
    _require_device(x, s)
    assert x.is_contiguous() and (s is None or (s.is_contiguous() and s.numel() == x.shape[-1]))
    k = x.shape[-1]
    y = torch.empty_like(x) if out is None else out
    call("mo_scale_block_int_qdq", x, _ptr(x), x.numel() // k if k else 0, k, dtype_code(x.dtype),
         _ptr(s), dtype_code(s.dtype) if s is not None else MO_F32, block_size, num_bits,
         int(bool(unsigned)), int(bool(narrow_range)), _ptr(y), _stream(x))
    return y


def abs_colsum_into(x, acc, blk_amax=None, block_size=0):
    _require_device(x, acc, blk_amax)
    k = x.shape[-1]
    assert x.is_contiguous() and acc.dtype == torch.float32 and acc.numel() == k
    rows = x.numel() // k if k else 0
    # below a few million elements the launch of the second pass costs more than it saves
    big = rows * k >= ((1 << 22) if blk_amax is not None else (1 << 23))
    if (big and k % 8 == 0 and rows >= 64 and x.data_ptr() % 16 == 0 and acc.data_ptr() % 16 == 0
            and (blk_amax is None or (block_size > 0 and block_size % 8 == 0 and k % block_size == 0))):
        # two passes, no atomics: about two workgroups per compute unit in all, at least 32 rows
        # per slab (8192 x 4096: 14.0 us against 18.1 us with twice as many slabs)
        across = -(-k // 2048)
        slabs = max(1, min(-(-512 // across), rows // 32))
        partial = _staging_words(x, slabs * k)
        call("mo_abs_colsum_staged", x, _ptr(x), rows, k, dtype_code(x.dtype), _ptr(blk_amax),
             block_size, _ptr(acc), _ptr(partial), slabs, _stream(x))
        return acc
    call("mo_abs_colsum", x, _ptr(x), rows, k, dtype_code(x.dtype),
         _ptr(blk_amax), block_size, _ptr(acc), _stream(x))
    return acc


def weight_scale_colsum_into(x, acc, block_size):
    """``acc[c] +=`` the column sums of ``T(|x| / T(block abs-max + tiny))`` with the abs-max of
    every ``block_size`` adjacent columns of a row taken in the same pass over ``x``.  Returns
    False (nothing written) for block sizes the kernel does not take: anything but 8, 16, ...
    512 dividing the row length."""
    _require_device(x, acc)
    k = x.shape[-1]
    assert x.is_contiguous() and acc.dtype == torch.float32 and acc.numel() == k
    rows = x.numel() // k if k else 0
    bs = int(block_size)
    if (bs < 8 or bs > 512 or bs & (bs - 1) or k % bs or x.data_ptr() % 16 or acc.data_ptr() % 16):
        return False
    # about four workgroups per compute unit in all (the quotients give each wavefront work to
    # overlap with the loads of the others: 14336 x 4096 takes 27 us with 1024 workgroups, 29 with
    # 512, 34 with 2048), at least 16 rows per slab
    across = -(-k // 2048)
    slabs = max(1, min(-(-1024 // across), rows // 16))
    partial = _staging_words(x, slabs * k)
    call("mo_weight_scale_colsum", x, _ptr(x), rows, k, dtype_code(x.dtype), bs, _ptr(acc),
         _ptr(partial), slabs, _stream(x))
    return True


def sq_diff_sum_into(a, b, acc):
    _require_device(a, b, acc)
    assert a.is_contiguous() and b.is_contiguous() and a.shape == b.shape and a.dtype == b.dtype
    assert acc.dtype == torch.float64
    call("mo_sq_diff_sum", a, _ptr(a), _ptr(b), a.numel(), dtype_code(a.dtype), _ptr(acc), _stream(a))
    return acc


# ----------------------------------------------------------------------------- multi-tensor plans

ABSMAX_TILE_ELEMS = 32768
NVFP4_TILE_ELEMS = 16384


def _job_table(rows, device):
    """rows: list of equal-length int tuples -> device int64 tensor [n, len] (the job structs)."""
    return torch.tensor(rows, dtype=torch.int64).to(device)


def _tile_job_map(tiles_per_job, device):
    """int32[total_tiles]: index of the job that owns each tile."""
    counts = torch.tensor(tiles_per_job, dtype=torch.int64)
    return torch.repeat_interleave(torch.arange(len(tiles_per_job), dtype=torch.int32), counts).to(device)


class _PinnedInputs:
    """The input tensors of a multi-tensor plan.  The job table holds raw addresses, so the plan
    keeps the tensors' storages alive (the addresses can never point at freed memory) and
    ``verify`` raises when a tensor has been given other memory since the plan was built
    (``param.data = ...``, ``.to()``): the plan would then read the old contents."""

    def __init__(self, tensors):
        self.tensors = list(tensors)
        self._storages = [t.untyped_storage() for t in self.tensors]
        self._addresses = [t.data_ptr() for t in self.tensors]

    def verify(self):
        for i, t in enumerate(self.tensors):
            if t.data_ptr() != self._addresses[i]:
                raise RuntimeError(f"tensor {i} of the plan was reallocated after the plan was "
                                   "built; build a new plan")


class AbsmaxPlan:
    """Per-tensor abs-max of a fixed list of tensors in one launch.

    ``acc`` is a float32 vector with one running maximum per tensor, refreshed by ``run``.
    Every tile folds into an accumulator with an atomic max, and atomics that hit one cache line
    are served one after the other; so a tensor is cut into spans of ``SPAN_TILES`` tiles, each
    span is a job with an accumulator of its own on a separate 256-byte line, and ``run`` ends
    with a small reduction over the spans of each tensor.  The plan keeps the tensors' memory
    alive; ``run`` checks that none has been reallocated (``verify=False`` skips the check of
    about 0.15 us per tensor, for a caller that has just built or verified the plan).
    """

    SPAN_TILES = 64
    LINE = 64  # floats between two accumulators

    def __init__(self, tensors):
        assert len(tensors) > 0
        dev, dt = tensors[0].device, tensors[0].dtype
        self._inputs = _PinnedInputs(tensors)
        self.tensors = self._inputs.tensors
        self.dtype = dtype_code(dt)
        esize = tensors[0].element_size()
        span_elems = self.SPAN_TILES * ABSMAX_TILE_ELEMS
        spans = [max(1, -(-t.numel() // span_elems)) for t in tensors]
        self._lines = torch.zeros((len(tensors), max(spans), self.LINE), dtype=torch.float32, device=dev)
        self.acc = torch.zeros(len(tensors), dtype=torch.float32, device=dev)
        rows, tile, per_job = [], 0, []
        for i, t in enumerate(tensors):
            _require_device(t)
            if t.device != dev or t.dtype != dt or not t.is_contiguous() or t.data_ptr() % 16:
                raise ValueError("AbsmaxPlan needs contiguous, 16-byte aligned tensors of one dtype/device")
            for j in range(spans[i]):
                n = min(span_elems, t.numel() - j * span_elems)
                rows.append((t.data_ptr() + j * span_elems * esize, self._lines[i, j].data_ptr(),
                             n, tile))
                per_job.append(-(-n // ABSMAX_TILE_ELEMS))
                tile += per_job[-1]
        self.total_tiles = tile
        self.njobs = len(rows)
        self.jobs = _job_table(rows, dev)
        self.tile_job = _tile_job_map(per_job, dev)

    def verify(self):
        self._inputs.verify()

    def run(self, zero=True, verify=True):
        if verify:
            self._inputs.verify()
        if zero:
            self._lines.zero_()
        call("mo_absmax_multi", self.acc, _ptr(self.jobs), self.njobs, _ptr(self.tile_job),
             self.total_tiles, self.dtype, _stream(self.acc))
        torch.amax(self._lines[:, :, 0], dim=1, out=self.acc)  # NaN propagates
        return self.acc


class Nvfp4QuantizePlan:
    """NVFP4 quantize + pack of a fixed list of bf16 tensors (last dim % 16 == 0) in one launch.

    ``amax`` is a float32 device vector (any stride) with one global amax (or wsf2 when
    ``amax_is_wsf2``) per tensor.  Outputs are allocated once here: ``packed[i]`` uint8 [..., K/2], ``wsf[i]``
    float8_e4m3fn [..., K/16], ``wsf2`` float32 [n].  The plan keeps the inputs' memory alive and
    ``run`` checks that no input (or the amax vector) has been reallocated (``verify=False`` skips it).
    """

    def __init__(self, tensors, amax, amax_is_wsf2=False, flags=0):
        assert len(tensors) > 0 and amax.dtype == torch.float32 and amax.numel() == len(tensors)
        dev = tensors[0].device
        self._inputs = _PinnedInputs(list(tensors) + [amax])
        self.tensors, self.amax, self.amax_is_wsf2 = list(tensors), amax, bool(amax_is_wsf2)
        self.flags = int(flags)
        self.wsf2 = torch.empty(len(tensors), dtype=torch.float32, device=dev)
        self.packed, self._wsf_u8 = [], []
        rows, tile, per_job = [], 0, []
        for t in tensors:
            _require_device(t)
            if (t.dtype != torch.bfloat16 or not t.is_contiguous() or t.shape[-1] % 16
                    or t.data_ptr() % 16 or t.device != dev):
                raise ValueError("Nvfp4QuantizePlan needs contiguous bf16 tensors with last dim % 16 == 0")
        # all outputs are carved from two slabs (codes, block scales), each view 256-byte aligned
        def _pad(nbytes):
            return (nbytes + 255) // 256 * 256
        p_off, w_off = [0], [0]
        for t in tensors:
            p_off.append(p_off[-1] + _pad(t.numel() // 2))
            w_off.append(w_off[-1] + _pad(t.numel() // 16))
        self._packed_slab = torch.empty(max(p_off[-1], 1), dtype=torch.uint8, device=dev)
        self._wsf_slab = torch.empty(max(w_off[-1], 1), dtype=torch.uint8, device=dev)
        for i, t in enumerate(tensors):
            lead = tuple(t.shape[:-1])
            p = self._packed_slab[p_off[i]:p_off[i] + t.numel() // 2].view(lead + (t.shape[-1] // 2,))
            w = self._wsf_slab[w_off[i]:w_off[i] + t.numel() // 16].view(lead + (t.shape[-1] // 16,))
            self.packed.append(p)
            self._wsf_u8.append(w)
            rows.append((t.data_ptr(), p.data_ptr(), w.data_ptr(), amax[i].data_ptr(),
                         self.wsf2.data_ptr() + 4 * i, t.numel(), tile, 0))
            per_job.append(-(-t.numel() // NVFP4_TILE_ELEMS))
            tile += per_job[-1]
        self.total_tiles = tile
        self.jobs = _job_table(rows, dev)
        self.tile_job = _tile_job_map(per_job, dev)
        self.wsf = [w.view(torch.float8_e4m3fn) for w in self._wsf_u8]

    def verify(self):
        self._inputs.verify()

    def run(self, verify=True):
        if verify:
            self._inputs.verify()
        call("mo_nvfp4_quantize_multi", self.amax, _ptr(self.jobs), len(self.tensors),
             _ptr(self.tile_job), self.total_tiles, MO_BF16, 16, int(self.amax_is_wsf2),
             self.flags, _stream(self.amax))
        return self.packed, self.wsf, self.wsf2
