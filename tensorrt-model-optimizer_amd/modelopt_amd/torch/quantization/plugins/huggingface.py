"""KV-cache quantizers for Hugging Face ``transformers`` attention modules.

Follows the reference's plugin (plugins/huggingface.py:52-139, 176-235): attention classes of a
``transformers`` model that use the attention-interface dispatch (``ALL_ATTENTION_FUNCTIONS`` /
``eager_attention_forward``, transformers >= 4.48) are registered on the fly; the quantised
class wraps ``forward`` so that, for the duration of the call, the attention function the
module is about to dispatch to first passes query, key and value states ``[B, H, S, D]``
through ``q_bmm_quantizer``, ``k_bmm_quantizer`` and ``v_bmm_quantizer``.  ``transformers`` is
optional: without it the plugin does nothing.
"""

import inspect
import sys
from functools import partial

from torch import nn

from ..nn.modules.quant_module import QuantModuleRegistry
from .attention import QuantAttentionMixin

__all__ = ["register_hf_attentions_on_the_fly"]


class _QuantHFAttention(QuantAttentionMixin):
    """Attention module of a ``transformers`` model with BMM quantizers in front of its kernel."""

    @staticmethod
    def _quantized_attention(original, module, query_states, key_states, value_states, *args, **kwargs):
        query_states, key_states, value_states = module._quantize_qkv(query_states, key_states,
                                                                      value_states)
        return original(module, query_states, key_states, value_states, *args, **kwargs)

    def forward(self, *args, **kwargs):
        modeling = inspect.getmodule(self._original_cls)
        implementation = self.config._attn_implementation
        eager = implementation == "eager" or (implementation == "sdpa"
                                              and kwargs.get("output_attentions", False))
        if eager:
            if not hasattr(modeling, "eager_attention_forward"):
                raise AssertionError(
                    f"Module {modeling} does not have `eager_attention_forward` to enable KV Cache "
                    "quantization. Please use a different attention implementation such as `sdpa`.")
            original = modeling.eager_attention_forward
            modeling.eager_attention_forward = partial(self._quantized_attention, original)
        else:
            original = modeling.ALL_ATTENTION_FUNCTIONS[implementation]
            modeling.ALL_ATTENTION_FUNCTIONS[implementation] = partial(self._quantized_attention,
                                                                       original)
        try:
            return super().forward(*args, **kwargs)
        finally:
            if eager:
                modeling.eager_attention_forward = original
            else:
                modeling.ALL_ATTENTION_FUNCTIONS[implementation] = original

    @staticmethod
    def is_compatible_attention(attn_cls) -> bool:
        return getattr(inspect.getmodule(attn_cls), "ALL_ATTENTION_FUNCTIONS", None) is not None


def _is_hf_model(model: nn.Module) -> bool:
    # an instance of a transformers class can only exist if transformers is imported already;
    # importing it here would put its start-up time into the first mtq.quantize of any model
    transformers = sys.modules.get("transformers")
    if transformers is None:
        return False
    return isinstance(model, transformers.PreTrainedModel)


def register_hf_attentions_on_the_fly(model: nn.Module):
    """Register the ``*Attention`` classes found in a ``transformers`` model so that conversion
    gives their instances ``q/k/v_bmm_quantizer`` (disabled until a config enables them)."""
    if not _is_hf_model(model):
        return
    for module in model.modules():
        cls = type(module)
        if not cls.__name__.endswith("Attention") or cls in QuantModuleRegistry:
            continue
        if _QuantHFAttention.is_compatible_attention(cls):
            QuantModuleRegistry.register({cls: cls.__name__})(_QuantHFAttention)
