"""GPU parity of the block floating point (MX / two-level) fake quantisation kernel."""

import json
import os

import pytest
import torch

from conftest import GOLDEN, assert_bits_equal
from modelopt_amd import _hip
from oracle import cref, mx
from test_mx_oracle import FORMATS, golden_inputs, golden_params

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16, torch.float16]


@pytest.mark.parametrize("case,block_size,dtype", list(golden_params()))
def test_reference_golden_tables_on_the_gpu(case, block_size, dtype):
    x, want = golden_inputs(case, block_size, dtype)
    got = _hip.block_fp_qdq(x.to(DEV), block_size, case["format"], "E8M0").cpu()
    assert torch.allclose(want, got, atol=max(case["atol"], 1e-8))
    assert_bits_equal(got, mx.block_fp_fake_quant(x, block_size, case["format"]), "vs oracle")


def _data(dtype, shape=(96, 160), seed=41):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(shape, generator=g) * torch.exp(3 * torch.randn(shape[0], 1, generator=g))).to(dtype)
    x[0, :16] = 0
    last = shape[1] - 1
    x[1, min(3, last)] = float("inf")
    x[2, min(5, last)] = float("nan")
    x[3, min(7, last)] = -0.0
    x[4] *= 1e-30            # E8M0 exponents near the bottom of the range
    x[5] *= 1e30 if dtype != torch.float16 else 1.0
    return x


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("dtype", DTYPES)
def test_e8m0_scale_all_formats(fmt, dtype):
    x = _data(dtype)
    for bs in (8, 16, 32):
        got = _hip.block_fp_qdq(x.to(DEV), bs, fmt).cpu()
        assert_bits_equal(got, mx.block_fp_fake_quant(x, bs, fmt), f"{fmt} bs{bs}")


@pytest.mark.parametrize("fmt", ["E2M1", "E4M3", "E3M2", "INT8"])
@pytest.mark.parametrize("k", [80, 77, 8, 3])
def test_padded_last_block_and_unaligned_rows(fmt, k):
    x = _data(torch.bfloat16, (33, k))
    for bs in (16, 32):
        got = _hip.block_fp_qdq(x.to(DEV), bs, fmt).cpu()
        assert_bits_equal(got, mx.block_fp_fake_quant(x, bs, fmt), f"k{k} bs{bs}")
    # a view that starts 2 bytes off a 16-byte boundary
    flat = torch.zeros(33 * k + 1, dtype=torch.bfloat16)
    flat[1:] = x.reshape(-1)
    xd = flat.to(DEV)[1:].view(33, k)
    assert_bits_equal(_hip.block_fp_qdq(xd, 16, fmt).cpu(), mx.block_fp_fake_quant(x, 16, fmt), "offset view")


@pytest.mark.parametrize("fmt", ["E2M1", "E2M3", "E4M3"])
@pytest.mark.parametrize("dtype", DTYPES)
def test_minifloat_block_scale_alone_and_under_a_global_amax(fmt, dtype):
    x = _data(dtype)[6:]
    xd = x.to(DEV)
    got = _hip.block_fp_qdq(xd, 16, fmt, "E4M3").cpu()
    assert_bits_equal(got, mx.block_fp_fake_quant(x, 16, fmt, "E4M3"), "no global amax")
    g1 = x.float().abs().amax().reshape(1)
    got = _hip.block_fp_qdq(xd, 16, fmt, "E4M3", g1.to(DEV)).cpu()
    assert_bits_equal(got, mx.block_fp_fake_quant(x, 16, fmt, "E4M3", g1), "one global amax")
    gr = x.float().abs().amax(dim=1).contiguous()
    got = _hip.block_fp_qdq(xd, 16, fmt, "E4M3", gr.to(DEV)).cpu()
    assert_bits_equal(got, mx.block_fp_fake_quant(x, 16, fmt, "E4M3", gr), "per-row global amax")
    gz = torch.zeros(1)
    got = _hip.block_fp_qdq(xd, 16, fmt, "E4M3", gz.to(DEV)).cpu()
    assert_bits_equal(got, mx.block_fp_fake_quant(x, 16, fmt, "E4M3", gz), "zero global amax")


@pytest.mark.parametrize("fmt", ["E4M3", "E2M1", "E3M2"])
def test_large_tensor_against_c_restatement(fmt):
    g = torch.Generator(device=DEV).manual_seed(43)
    xd = (torch.randn((4096, 4096), generator=g, device=DEV) * 0.02).to(torch.bfloat16)
    got = _hip.block_fp_qdq(xd, 32, fmt).cpu()
    want = cref.block_fp_fake_quant(xd.cpu(), 32, fmt)
    assert_bits_equal(got, want, fmt)


def test_argument_checks():
    x = torch.zeros(4, 32, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError):
        _hip.block_fp_qdq(x, 64, "E2M1")
    with pytest.raises(RuntimeError):
        _hip.block_fp_qdq(x, 32, "E8M0")
    with pytest.raises(RuntimeError):            # a global amax has no meaning with E8M0 scales
        _hip.block_fp_qdq(x, 32, "E2M1", "E8M0", torch.ones(1, device=DEV))
    with pytest.raises(ValueError):
        _hip.block_fp_qdq(x, 32, "E2M1", "E4M3", torch.ones(3, device=DEV))
    assert _hip.block_fp_qdq(x[:0], 32, "E2M1").shape == (0, 32)


# ----------------------------------------------------------------------------- host layer
@pytest.mark.parametrize("cfg_name,fmt", [("MXFP8_DEFAULT_CFG", "E4M3"), ("MXFP6_DEFAULT_CFG", "E3M2"),
                                          ("MXFP4_DEFAULT_CFG", "E2M1"), ("MXINT8_DEFAULT_CFG", "INT8")])
def test_mx_configs_through_quantizer_and_quantize(cfg_name, fmt):
    import modelopt_amd.torch.quantization as mtq
    from modelopt_amd.torch.quantization.config import QuantizerAttributeConfig

    cfg = getattr(mtq, cfg_name)
    x = _data(torch.bfloat16, (96, 96))[:, :80].reshape(4, 24, 80).contiguous()   # 3-D, last block padded
    q = mtq.nn.TensorQuantizer(QuantizerAttributeConfig(**cfg["quant_cfg"]["*input_quantizer"])).to(DEV)
    assert q.is_mx_format and q.amax is None
    got = q(x.to(DEV)).cpu()
    assert_bits_equal(got, mx.block_fp_fake_quant(x, 32, fmt), "TensorQuantizer")

    lin = torch.nn.Sequential(torch.nn.Linear(80, 64, bias=False)).to(torch.bfloat16).to(DEV)
    w = lin[0].weight.data.cpu().clone()
    mtq.quantize(lin, cfg, forward_loop=None)                          # algorithm None: nothing to calibrate
    y = lin(x.to(DEV))
    want = torch.nn.functional.linear(mx.block_fp_fake_quant(x, 32, fmt).to(DEV),
                                      mx.block_fp_fake_quant(w, 32, fmt).to(DEV))
    assert_bits_equal(y.detach().cpu(), want.cpu(), "quantised linear")   # rows with inf / NaN give NaN


def test_extension_shim_matches_reference_call_shape():
    from modelopt_amd.torch.quantization.extensions import get_cuda_ext_mx
    from modelopt_amd.torch.quantization.tensor_quant import mx_format_map

    ext = get_cuda_ext_mx(raise_if_failed=True)
    x = _data(torch.float16, (16, 64))
    for num_bits in [8, (2, 1), (3, 2), (2, 3), (4, 3), (5, 2)]:
        for scale_bits in [(4, 3), (8, 0)]:
            y = ext.fused_amax_convert(x.to(DEV), 16, getattr(ext.Types, mx_format_map[num_bits]),
                                       getattr(ext.Types, mx_format_map[scale_bits]), None)
            assert y.dtype == x.dtype
            assert_bits_equal(y.cpu(), mx.block_fp_fake_quant(x, 16, mx_format_map[num_bits],
                                                              mx_format_map[scale_bits]), str(num_bits))
    with pytest.raises(ValueError):
        ext.fused_amax_convert(x.to(DEV), 64, ext.Types.E2M1, ext.Types.E8M0, None)


# ----------------------------------------------------------------------------- packed MXFP4
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("block", [32, 16])
def test_mxfp4_pack_and_unpack_match_the_reference_qtensor(dtype, block):
    g = torch.Generator().manual_seed(61)
    x = (torch.randn((64, 256), generator=g) * torch.exp(3 * torch.randn((64, 1), generator=g))).to(dtype)
    x[0, :64] = 0                                              # zero blocks: scale byte 0, code 8
    x[1, :8] = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0]).to(dtype)   # exact bounds
    x[1, 8:32] = 0.1
    x[2, :32] = x[1, :32] * -4                                 # the same, negative, another scale
    x[3, 5] = -0.0
    x[4] *= 1e-30 if dtype != torch.float16 else 1e-4
    packed, scales = _hip.mxfp4_quantize(x.to(DEV), block)
    p_o, s_o = mx.mxfp4_quantize(x, block)
    assert torch.equal(scales.cpu(), s_o)
    assert torch.equal(packed.cpu(), p_o)
    y = _hip.mxfp4_dequantize(packed, scales, block, dtype)
    assert_bits_equal(y.cpu(), mx.mxfp4_dequantize(p_o, s_o, block, x.shape, dtype), "dequantised")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_mxfp4_pack_every_16_bit_value(dtype):
    """Every finite 16-bit pattern as an element, 31 to a block behind a pilot value that sets
    the block scale (values above the pilot move it, which is fine): all ties on the E2M1
    bounds, both zeros, subnormals and the largest magnitudes, at four scales."""
    allv = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype)
    finite = allv[torch.isfinite(allv.float())]
    finite = finite[: finite.numel() // 31 * 31].reshape(-1, 31)
    for pilot in (6.0, 4.0, 0.013, 300.0):
        col = torch.full((finite.shape[0], 1), pilot, dtype=dtype)
        x = torch.cat([col, finite], dim=1).contiguous()
        packed, scales = _hip.mxfp4_quantize(x.to(DEV), 32)
        p_o, s_o = mx.mxfp4_quantize(x, 32)
        assert torch.equal(scales.cpu(), s_o), pilot
        assert torch.equal(packed.cpu(), p_o), (pilot, (packed.cpu() != p_o).nonzero()[:4].tolist())


def test_mxfp4_every_code_and_scale_byte_dequantizes_like_the_reference():
    codes = torch.arange(256, dtype=torch.uint8).repeat(16).reshape(-1, 16)      # 256 blocks of 32
    scales = torch.arange(256, dtype=torch.uint8).reshape(-1, 1)
    for dtype in DTYPES:
        y = _hip.mxfp4_dequantize(codes.to(DEV), scales.to(DEV), 32, dtype)
        assert_bits_equal(y.cpu(), mx.mxfp4_dequantize(codes, scales, 32, (256, 32), dtype), str(dtype))


def test_mxfp4_through_quantizer_and_compress():
    import modelopt_amd.torch.quantization as mtq
    from modelopt_amd.torch.quantization.qtensor import MXFP4QTensor, QTensorWrapper

    lin = torch.nn.Sequential(torch.nn.Linear(128, 64, bias=False)).to(torch.bfloat16).to(DEV)
    w = lin[0].weight.data.cpu().clone()
    mtq.quantize(lin, mtq.MXFP4_DEFAULT_CFG, forward_loop=None)
    with pytest.warns(UserWarning):
        mtq.compress(lin)
    assert isinstance(lin[0].weight, QTensorWrapper) and lin[0].weight.metadata["qtensor_class"] is MXFP4QTensor
    p_o, s_o = mx.mxfp4_quantize(w, 32)
    assert torch.equal(lin[0].weight.data.cpu(), p_o)
    assert torch.equal(lin[0].weight_quantizer._scale.cpu(), s_o)
    got = lin[0].weight_quantizer(lin[0].weight)
    assert_bits_equal(got.cpu(), mx.mxfp4_dequantize(p_o, s_o, 32, w.shape, torch.bfloat16), "dequantised weight")
    x = torch.randn(4, 128, dtype=torch.bfloat16, device=DEV)
    assert torch.isfinite(lin(x).float()).all()
