"""The names the reference's Python calls across its native seam (extensions.py:27-70, the triton
module, the torch.library operators), bound to the HIP library, against the CPU oracle."""

import pytest
import torch

import modelopt_amd.torch.quantization as mtq
from conftest import assert_bits_equal
from modelopt_amd.torch.quantization import extensions, tensor_quant
from modelopt_amd.torch.quantization import triton as fp4_kernels
from modelopt_amd.torch.quantization.config import QuantizerAttributeConfig
from modelopt_amd.torch.quantization.nn import TensorQuantizer
from modelopt_amd.torch.quantization.qtensor import NVFP4QTensor
from oracle import fake_quant, mx, qtensor, reduce

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _rand(shape, dtype=torch.bfloat16, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def test_library_operators_run_the_kernels():
    x, amax = _rand((32, 64), seed=1), torch.tensor(2.0, dtype=torch.bfloat16)
    xd, ad = x.to(DEV), amax.to(DEV)
    y = torch.ops.tensorrt.quantize_op(xd, ad, 8, 0, False, False)
    assert_bits_equal(y.cpu(), fake_quant.tensor_quant(x, amax, 8, False, False), "int8 operator")
    y = torch.ops.tensorrt.quantize_op(xd, ad * 4, 8, 4, False, False)
    assert_bits_equal(y.cpu(), fake_quant.fp8_eager(x, amax * 4), "fp8 operator")
    gamax = reduce.reduce_amax(x)
    y = torch.ops.tensorrt.dynamic_block_quantize_op(xd, 16, gamax.to(DEV), 4, 2, 8, 4)
    assert_bits_equal(y.cpu(), fake_quant.nvfp4_fake_quant(x, gamax, 16), "nvfp4 operator")
    y = torch.ops.tensorrt.dynamic_block_quantize_op(xd, 32, None, 4, 2, 9, 8)
    assert_bits_equal(y.cpu(), mx.block_fp_fake_quant(x, 32, "E2M1", "E8M0"), "mxfp4 operator, amax None")
    assert tensor_quant.dynamic_block_quantize_op is torch.ops.tensorrt.dynamic_block_quantize_op


def test_quantizer_forward_traces_to_the_operators():
    """A quantizer forward under ``make_fx`` records the reference's operator nodes (what
    torch.export / torch.compile see); tracing with fake tensors is covered on the CPU."""
    from torch.fx.experimental.proxy_tensor import make_fx

    q8 = TensorQuantizer(QuantizerAttributeConfig(num_bits=(4, 3)), amax=3.0).to(DEV)
    q4 = TensorQuantizer(QuantizerAttributeConfig(**mtq.NVFP4_DEFAULT_CFG["quant_cfg"]["*input_quantizer"]),
                         amax=2.0).to(DEV)
    x = _rand((8, 64), seed=2).to(DEV)
    traced = make_fx(lambda t: q4(q8(t)), tracing_mode="real")(x)
    targets = [str(n.target) for n in traced.graph.nodes if n.op == "call_function"]
    assert "tensorrt.quantize_op.default" in targets
    assert "tensorrt.dynamic_block_quantize_op.default" in targets
    assert torch.equal(traced(x), q4(q8(x)))


@pytest.mark.parametrize("fmt", ["E4M3", "E5M2", "INT8", "E0M3", "E1M2", "E3M0", "E2M1", "E3M2", "E2M3"])
def test_convert_to_exmy(fmt):
    ext = extensions.get_cuda_ext_mx(raise_if_failed=True)
    values = torch.tensor(mx._TABLES[fmt] if fmt in mx._TABLES else [0.0, 1.0, 100.0, 448.0])
    mids = (values[:-1] + values[1:]) / 2 if values.numel() > 1 else values
    g = torch.Generator().manual_seed(3)
    top = float(mx.FORMAT_MAX[fmt])
    x = torch.cat([values, mids, mids * 1.0001, mids * 0.9999, -values, -mids,
                   torch.tensor([0.0, top, top * 1.5, float("inf"), -float("inf"), 1e-9]),
                   (torch.rand(4096, generator=g) * 2 - 1) * top * 1.1]).float()
    got = mtq.kernels._hip.convert_to_format(x.to(DEV), fmt).cpu()
    want = mx.convert_to_types(x, fmt)
    assert torch.equal(got, want) or torch.equal(got[got == got], want[want == want])
    for v in (0.3, -2.6, 5.0, 1000.0):
        assert ext.convert_to_exmy(v, getattr(ext.Types, fmt)) == float(mx.convert_to_types(torch.tensor([v]), fmt))
    assert ext.convert_to_exmy(3.0, ext.Types.E8M0) == 0.0


def test_triton_named_module():
    assert fp4_kernels.IS_AVAILABLE
    x = _rand((40, 96), seed=4)
    gamax = reduce.reduce_amax(x)
    y = fp4_kernels.fp4_fake_quant_block(x.to(DEV), gamax.to(DEV), 16, tile_rows=32, tile_cols=128,
                                         num_warps=4, num_stages=2)
    assert_bits_equal(y.cpu(), fake_quant.nvfp4_fake_quant(x, gamax, 16), "fp4_fake_quant_block")
    packed, wsf, wsf2 = qtensor.nvfp4_quantize(x, 16)
    y = fp4_kernels.fp4_dequantize(packed.to(DEV), wsf.to(DEV), wsf2.to(DEV), 16, dtype=torch.bfloat16)
    assert_bits_equal(y.cpu(), qtensor.nvfp4_dequantize(packed, wsf, wsf2, 16, x.shape, torch.bfloat16),
                      "fp4_dequantize")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("n,bs", [(4096, 128), (1000, 10), (64, 8)])
def test_int4_quantize_uses_the_scales_it_is_given(dtype, n, bs):
    """``INT4_quantize(input, scales, block_size)`` with scales that are not ``7 / amax``: the
    bytes follow the caller's scales (``clamp(round(x * s), -8, 7) + 8``, product in the input
    dtype, high nibble first)."""
    ext = extensions.get_cuda_ext(raise_if_failed=True)
    x = _rand((n,), dtype, seed=5)
    scales = (5.0 / reduce.reduce_amax(x.view(-1, bs), axis=-1)).view(-1, 1).to(dtype)  # not 7 / amax
    got = ext.INT4_quantize(x.to(DEV), scales.to(DEV), bs).cpu()
    q = ((x.view(-1, bs) * scales).flatten().round().clamp(-8, 7) + 8).to(torch.uint8)
    want = q[::2] << 4 | q[1::2]
    assert torch.equal(got, want)
    own, _ = qtensor.int4_quantize(x, bs)
    assert not torch.equal(got, own.flatten())
    back = ext.INT4_dequantize(got.to(DEV), scales.to(DEV), bs).cpu()
    assert back.dtype == dtype and torch.allclose(back.float(), x.float(), atol=float(x.abs().max()) / 4)


@pytest.mark.parametrize("shape", [(16, 64), (3, 5, 40)])
def test_nvfp4_keep_high_precision(shape):
    """``keep_high_precision=True``: fp32 block scales before the E4M3 cast, and ``quantize``
    returns the scaled weight before the FP4 cast (qtensor/nvfp4_tensor.py:84-92,208-222)."""
    x = _rand(shape, seed=6, scale=0.02)
    wsf2 = reduce.reduce_amax(x).float() / 2688.0
    raw, _ = qtensor.nvfp4_block_scales(x, 8, wsf2, keep_high_precision=True)
    got, got2 = NVFP4QTensor.get_weights_scaling_factor(x.to(DEV), 8, wsf2.to(DEV), keep_high_precision=True)
    assert_bits_equal(got.cpu(), raw, "fp32 block scales")
    wsf, _ = qtensor.nvfp4_block_scales(x, 8, wsf2)
    want = (x.view(*shape[:-1], -1, 8) / (wsf.float() * wsf2).unsqueeze(-1)).view(shape)
    scaled = NVFP4QTensor.quantize(x.to(DEV), 8, keep_high_precision=True)
    assert scaled.dtype == torch.float32
    assert_bits_equal(scaled.cpu(), want, "scaled weight")
