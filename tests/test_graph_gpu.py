"""Library calls recorded into a HIP graph (``torch.cuda.graph``) and replayed: a serving loop
replays the quantised forward instead of launching it, so every replay must give what the eager
call gives on the same input.  The graph is replayed several times with eager library work and
synchronisations in between, on fresh input each time."""

import ctypes

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

import modelopt_amd.torch.quantization as mtq
from modelopt_amd import _hip
from modelopt_amd.torch.quantization import kernels
from modelopt_amd.torch.quantization.nn import TensorQuantizer
from modelopt_amd.torch.quantization.config import QuantizerAttributeConfig
from modelopt_amd.torch.quantization.qtensor import NVFP4QTensor

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
REPLAYS = 4


def _inputs(shape, dtype, n=REPLAYS, seed=0):
    g = torch.Generator(device=DEV).manual_seed(seed)
    # a different magnitude per replay, so that a stale scale or maximum shows
    return [(torch.randn(shape, generator=g, device=DEV) * (0.05 * 7 ** i)).to(dtype) for i in range(n)]


def _replay_against_eager(fn, shape, dtype, seed=0):
    """Record ``fn(static_input)`` once; then, per fresh input: eager result, unrelated eager
    library work, a synchronisation, a replay, and a bit-for-bit comparison."""
    xs = _inputs(shape, dtype, seed=seed)
    static = xs[0].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):   # warm up outside the capture: lazy initialisation, workspaces
        fn(static)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        recorded = fn(static)
    recorded = recorded if isinstance(recorded, (tuple, list)) else (recorded,)
    for i, x in enumerate(reversed(xs)):
        want = fn(x)
        want = want if isinstance(want, (tuple, list)) else (want,)
        want = [w.clone() for w in want]
        kernels.reduce_amax_gpu(x * 3, None)            # eager work that shares the library's scratch
        kernels.fake_quant_fp8(x, x.abs().amax().float())
        torch.cuda.synchronize()
        static.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        for got, w in zip(recorded, want):
            assert torch.equal(got.view(torch.uint8) if got.dtype.itemsize == 1 else got,
                               w.view(torch.uint8) if w.dtype.itemsize == 1 else w), f"replay {i}"


def _quantizer(**attrs):
    q = TensorQuantizer(QuantizerAttributeConfig(**attrs)).to(DEV)
    return q.eval()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_static_fp8_and_int8_fake_quant(dtype):
    fp8 = _quantizer(num_bits=(4, 3), axis=None)
    fp8.amax = torch.tensor(2.5, device=DEV)
    int8 = _quantizer(num_bits=8, axis=0)
    int8.amax = torch.linspace(0.1, 4.0, 96, device=DEV).reshape(96, 1)
    with torch.no_grad():
        _replay_against_eager(lambda x: (fp8(x), int8(x)), (96, 1024), dtype)


@pytest.mark.parametrize("num_bits", [8, (4, 3)])
def test_dynamic_per_tensor_fake_quant_in_one_launch(num_bits):
    """The one-launch abs-max + quantize path waits across workgroups on a workspace; a recorded
    call brings a workspace of its own, zeroed by a node of the graph."""
    import modelopt_amd.torch.quantization as mtq

    q = _quantizer(num_bits=num_bits, axis=None)
    previous = mtq.set_one_launch_dynamic_quant(True)
    try:
        with torch.no_grad():
            assert q._fused_dynamic_per_tensor(torch.ones(8, 64, device=DEV, dtype=torch.bfloat16)) is not None
            _replay_against_eager(q, (512, 2048), torch.bfloat16, seed=1)
    finally:
        mtq.set_one_launch_dynamic_quant(previous)
    assert not _hip.fused_gave_up(DEV)


def test_dynamic_nvfp4_fake_quant():
    q = _quantizer(num_bits=(2, 1), block_sizes={-1: 16, "type": "dynamic", "scale_bits": (4, 3)}, axis=None)
    with torch.no_grad():
        _replay_against_eager(q, (256, 4096), torch.bfloat16, seed=2)   # per-tensor maximum on the fly
        q.amax = torch.tensor(3.0, device=DEV)
        _replay_against_eager(q, (256, 4096), torch.bfloat16, seed=3)   # calibrated maximum


def test_nvfp4_quantize_pack_and_dequantize():
    def run(x):
        qt, wsf, wsf2 = NVFP4QTensor.quantize(x, 16)
        back = qt.dequantize(dtype=x.dtype, scale=wsf, double_scale=wsf2, block_sizes={-1: 16})
        return qt._quantized_data, wsf, wsf2, back
    _replay_against_eager(run, (384, 2048), torch.bfloat16, seed=4)


class _MLP(nn.Module):
    def __init__(self, d=256, h=512):
        super().__init__()
        g = torch.Generator().manual_seed(0)
        self.fc1, self.fc2 = nn.Linear(d, h), nn.Linear(h, d, bias=False)
        for p in self.parameters():
            p.data = torch.randn(p.shape, generator=g) * 0.05
        self.to(torch.bfloat16)

    def forward(self, x):
        return self.fc2(F.gelu(self.fc1(x)))


@pytest.mark.parametrize("cfg", ["FP8_DEFAULT_CFG", "NVFP4_DEFAULT_CFG", "INT8_DEFAULT_CFG"])
def test_quantised_model_forward(cfg):
    model = _MLP().to(DEV).eval()
    calib = _inputs((32, 256), torch.bfloat16, n=3, seed=5)
    mtq.quantize(model, getattr(mtq, cfg), lambda m: [m(b) for b in calib])
    with torch.no_grad():
        _replay_against_eager(model, (32, 256), torch.bfloat16, seed=6)


def test_abs_max_per_column_without_allocation():
    """The entry point that allocates nothing, with its accumulator cleared by a fill kernel."""
    lib = _hip.load()

    def run(x):
        acc = torch.empty(x.shape[1], dtype=torch.float32, device=x.device)
        acc.zero_()
        stream = ctypes.c_void_p(torch.cuda.current_stream(x.device).cuda_stream)
        rc = lib.mo_absmax_cols_noalloc(ctypes.c_void_p(x.data_ptr()), x.shape[0], x.shape[1],
                                        _hip.dtype_code(x.dtype), ctypes.c_void_p(acc.data_ptr()), stream)
        assert rc == 0
        return acc
    _replay_against_eager(run, (2048, 4096), torch.bfloat16, seed=7)
