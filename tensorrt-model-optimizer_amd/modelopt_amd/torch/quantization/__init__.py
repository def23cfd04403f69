"""``modelopt_amd.torch.quantization`` -- import as ``mtq``.

Same entry points as ``modelopt.torch.quantization``: ``quantize``, ``calibrate``, the named
configs (``NVFP4_DEFAULT_CFG`` ...), ``TensorQuantizer`` under ``nn``.
"""

from . import calib, config, conversion, kernels, model_calib, modes, nn, qtensor, tensor_quant, utils
from .compress import compress, is_real_quantized
from .config import *  # noqa: F401,F403
from .conversion import (register, replace_quant_module, set_quantizer_attribute,
                         set_quantizer_by_cfg, set_quantizer_by_cfg_context, unregister)
from .model_quant import (auto_quantize, calibrate, disable_quantizer, enable_quantizer, fold_weight,
                          postprocess_amax, print_quant_summary, quantize)
from .nn.modules.quant_module import QuantModuleRegistry
from . import plugins
from .plugins import attention as _attention_plugin  # noqa: F401  (registers KV quantizers)
from .utils import update_quant_cfg_with_kv_cache_quant
from .tensor_quant import get_fp8_overflow_behavior, set_fp8_overflow_behavior
from .modes import (one_launch_dynamic_quant, set_one_launch_dynamic_quant, set_strict_checks,
                    strict_checks)
