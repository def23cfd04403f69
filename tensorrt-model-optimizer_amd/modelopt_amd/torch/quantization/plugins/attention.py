"""KV-cache / attention-operand quantizers.

Follows the call site of the reference's HF plugin (plugins/huggingface.py:52-139): an attention
module gains ``q_bmm_quantizer``, ``k_bmm_quantizer`` and ``v_bmm_quantizer`` (disabled until a
config such as ``FP8_KV_CFG`` enables ``*[kv]_bmm_quantizer``) that are applied to the query, key
and value states ``[B, H, S, D]`` right before the attention product.  Any module class that
calls ``self._quantize_qkv(q, k, v)`` can be registered with :func:`register_attention_class`.
"""

from torch import nn

from ..nn.modules.quant_module import QuantModule, QuantModuleRegistry
from ..nn.modules.tensor_quantizer import TensorQuantizer

__all__ = ["QuantAttentionMixin", "register_attention_class"]


class QuantAttentionMixin(QuantModule):
    """Adds the three BMM quantizers; the host attention calls ``_quantize_qkv``."""

    def _setup(self):
        for name in ("q_bmm_quantizer", "k_bmm_quantizer", "v_bmm_quantizer"):
            q = TensorQuantizer()
            q.disable()
            self.add_module(name, q)

    def _quantize_qkv(self, query, key, value):
        return self.q_bmm_quantizer(query), self.k_bmm_quantizer(key), self.v_bmm_quantizer(value)


def register_attention_class(attn_cls: type):
    """Make ``mtq.quantize`` attach BMM quantizers to instances of ``attn_cls``.  Until then the
    class-level ``_quantize_qkv`` of the attention implementation is expected to be an identity."""
    QuantModuleRegistry.register({attn_cls: attn_cls.__name__})(QuantAttentionMixin)
