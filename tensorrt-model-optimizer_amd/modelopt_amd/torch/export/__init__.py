"""Export of quantised models to the unified (HF-layout) checkpoint."""

from .model_config import *  # noqa: F401,F403
from .quant_utils import *  # noqa: F401,F403
from .unified_export_hf import (export_hf_checkpoint,  # noqa: F401
                                requantize_resmooth_fused_llm_layers)
