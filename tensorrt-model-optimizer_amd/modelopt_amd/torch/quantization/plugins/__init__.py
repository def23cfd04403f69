"""Model-family plugins.  ``CUSTOM_MODEL_PLUGINS`` are run on a model right before its modules
are converted (reference: plugins/custom.py ``CUSTOM_MODEL_PLUGINS``, conversion.py:118-127)."""

from .attention import (QuantAttentionMixin, register_attention_class,
                        register_attention_for_kv_quant)
from .huggingface import register_hf_attentions_on_the_fly

CUSTOM_MODEL_PLUGINS = [register_hf_attentions_on_the_fly]

__all__ = ["CUSTOM_MODEL_PLUGINS", "QuantAttentionMixin", "register_attention_class",
           "register_attention_for_kv_quant", "register_hf_attentions_on_the_fly"]
