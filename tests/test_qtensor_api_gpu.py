"""Real-quantization round trips through ``TensorQuantizer(fake_quant=False)`` with the shapes and
expectations of the reference's QTensor tests (tests/gpu/torch/quantization/test_qtensor_cuda.py)."""

import pytest
import torch

from modelopt_amd.torch.quantization.config import QuantizerAttributeConfig
from modelopt_amd.torch.quantization.nn import TensorQuantizer

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.float16, torch.bfloat16]


@pytest.mark.parametrize("block_sizes", [{-1: 64, "scale_bits": 8, "scale_block_sizes": {-1: 256}}, {-1: 64}])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape,check_memory", [((256, 64), True), ((256, 32), False)])
def test_four_bit_round_trip_and_footprint(block_sizes, dtype, shape, check_memory):
    """:29-68: NF4 with double-quantised scales and INT4 blocks; the packed tensor takes under
    30 % of the input's bytes and dequantises back within 0.1."""
    quantizer = TensorQuantizer(QuantizerAttributeConfig(num_bits=4, block_sizes=block_sizes, fake_quant=False)).to(DEV)
    x = torch.rand(shape, generator=torch.Generator().manual_seed(0)).to(DEV).to(dtype)
    before = torch.cuda.memory_allocated(DEV)
    packed = quantizer(x)
    grown = torch.cuda.memory_allocated(DEV) - before
    if check_memory:
        assert grown / (x.numel() * x.element_size()) < 0.3
    back = quantizer(packed)
    assert back.dtype == dtype and back.shape == x.shape
    assert torch.allclose(back, x, rtol=1e-1, atol=1e-1)


@pytest.mark.parametrize("shape", [(128, 576), (576, 128)])
def test_fp8_2d_blocks_keep_the_data_shape(shape):
    """:469-503"""
    cfg = QuantizerAttributeConfig(num_bits=(4, 3), block_sizes={-1: 128, -2: 128}, fake_quant=False)
    packed = TensorQuantizer(cfg).to(DEV)(torch.rand(shape, device=DEV))
    assert packed._quantized_data.shape == shape


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape,block_sizes", [((128, 1152), {-1: 128}), ((256, 256), {-1: 64, -2: 64})])
def test_fp8_blocks_ignore_a_scalar_amax(dtype, shape, block_sizes):
    """:573-601: a per-tensor amax left on the quantizer does not replace the per-block scales"""
    quantizer = TensorQuantizer(QuantizerAttributeConfig(num_bits=(4, 3), block_sizes=block_sizes,
                                                         fake_quant=False)).to(DEV)
    quantizer.amax = torch.tensor(1.5, device=DEV)
    x = torch.randn(shape, generator=torch.Generator().manual_seed(1)).to(DEV).to(dtype)
    back = quantizer(quantizer(x))
    assert torch.allclose(back, x, rtol=1e-1, atol=1e-1)
    assert hasattr(quantizer, "_scale") and quantizer._scale.numel() > 1
