"""A Llama-shaped decoder in plain torch with HF module names.

Random-initialised stand-in for ``transformers``' ``LlamaForCausalLM``: the linear layers are
named ``model.layers.{i}.self_attn.{q,k,v,o}_proj``, ``model.layers.{i}.mlp.{gate,up,down}_proj``
and ``lm_head``, so the wildcards of the stock quantization configs (``*weight_quantizer``,
``*lm_head*``, ``*[kv]_bmm_quantizer``) match exactly as they do on the HF model.  The attention
module exposes ``_quantize_qkv`` (identity until converted) where the reference's HF plugin
inserts the KV-cache quantizers (plugins/huggingface.py:52-69).
"""

import math
from dataclasses import asdict, dataclass

import torch
import torch.nn.functional as F
from torch import nn

from ..torch.quantization.plugins.attention import register_attention_class

__all__ = ["LlamaConfig", "LlamaForCausalLM", "LLAMA3_8B"]


@dataclass
class LlamaConfig:
    vocab_size: int = 128256
    hidden_size: int = 4096
    intermediate_size: int = 14336
    num_hidden_layers: int = 32
    num_attention_heads: int = 32
    num_key_value_heads: int = 8
    rms_norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    torch_dtype: str = "bfloat16"
    architectures: tuple = ("LlamaForCausalLM",)
    model_type: str = "llama"

    def to_dict(self):
        d = asdict(self)
        d["architectures"] = list(self.architectures)
        return d


LLAMA3_8B = LlamaConfig()


class RMSNorm(nn.Module):
    def __init__(self, dim, eps):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim))
        self.eps = eps

    def forward(self, x):
        v = x.float()
        v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + self.eps)
        return self.weight * v.to(x.dtype)


def _rope(x, theta):
    # x: [B, H, S, D]
    b, h, s, d = x.shape
    inv = 1.0 / (theta ** (torch.arange(0, d, 2, device=x.device, dtype=torch.float32) / d))
    ang = torch.arange(s, device=x.device, dtype=torch.float32)[:, None] * inv[None, :]
    cos, sin = ang.cos().to(x.dtype), ang.sin().to(x.dtype)
    x1, x2 = x[..., : d // 2], x[..., d // 2:]
    return torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1)


class LlamaAttention(nn.Module):
    def __init__(self, cfg: LlamaConfig):
        super().__init__()
        self.config = cfg
        self.h, self.hkv = cfg.num_attention_heads, cfg.num_key_value_heads
        self.d = cfg.hidden_size // cfg.num_attention_heads
        self.theta = cfg.rope_theta
        self.q_proj = nn.Linear(cfg.hidden_size, self.h * self.d, bias=False)
        self.k_proj = nn.Linear(cfg.hidden_size, self.hkv * self.d, bias=False)
        self.v_proj = nn.Linear(cfg.hidden_size, self.hkv * self.d, bias=False)
        self.o_proj = nn.Linear(self.h * self.d, cfg.hidden_size, bias=False)

    def _quantize_qkv(self, query, key, value):
        return query, key, value

    def forward(self, x):
        b, s, _ = x.shape
        q = self.q_proj(x).view(b, s, self.h, self.d).transpose(1, 2)
        k = self.k_proj(x).view(b, s, self.hkv, self.d).transpose(1, 2)
        v = self.v_proj(x).view(b, s, self.hkv, self.d).transpose(1, 2)
        q, k = _rope(q, self.theta), _rope(k, self.theta)
        q, k, v = self._quantize_qkv(q, k, v)
        out = F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=self.h != self.hkv)
        return self.o_proj(out.transpose(1, 2).reshape(b, s, self.h * self.d))


class LlamaMLP(nn.Module):
    def __init__(self, cfg: LlamaConfig):
        super().__init__()
        self.gate_proj = nn.Linear(cfg.hidden_size, cfg.intermediate_size, bias=False)
        self.up_proj = nn.Linear(cfg.hidden_size, cfg.intermediate_size, bias=False)
        self.down_proj = nn.Linear(cfg.intermediate_size, cfg.hidden_size, bias=False)

    def forward(self, x):
        return self.down_proj(F.silu(self.gate_proj(x)) * self.up_proj(x))


class LlamaDecoderLayer(nn.Module):
    def __init__(self, cfg: LlamaConfig):
        super().__init__()
        self.self_attn = LlamaAttention(cfg)
        self.mlp = LlamaMLP(cfg)
        self.input_layernorm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps)
        self.post_attention_layernorm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps)

    def forward(self, x):
        x = x + self.self_attn(self.input_layernorm(x))
        return x + self.mlp(self.post_attention_layernorm(x))


class LlamaModel(nn.Module):
    def __init__(self, cfg: LlamaConfig):
        super().__init__()
        self.embed_tokens = nn.Embedding(cfg.vocab_size, cfg.hidden_size)
        self.layers = nn.ModuleList(LlamaDecoderLayer(cfg) for _ in range(cfg.num_hidden_layers))
        self.norm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps)

    def forward(self, input_ids):
        x = self.embed_tokens(input_ids)
        for layer in self.layers:
            x = layer(x)
        return self.norm(x)


class LlamaForCausalLM(nn.Module):
    """``logits = lm_head(model(input_ids))``; weights ~ N(0, 0.02) in ``dtype`` on ``device``."""

    def __init__(self, cfg: LlamaConfig = LLAMA3_8B, device="cpu", dtype=torch.bfloat16, seed=0):
        super().__init__()
        self.config = cfg
        with torch.device("meta"):
            self.model = LlamaModel(cfg)
            self.lm_head = nn.Linear(cfg.hidden_size, cfg.vocab_size, bias=False)
        self.to_empty(device=device)
        g = torch.Generator(device=device).manual_seed(seed)
        with torch.no_grad():
            for name, p in self.named_parameters():
                p.data = torch.empty(p.shape, device=device, dtype=dtype)
                if name.endswith("norm.weight") or "layernorm" in name:
                    p.data.fill_(1.0)
                else:
                    p.data.normal_(0.0, 0.02, generator=g)

    def forward(self, input_ids):
        return self.lm_head(self.model(input_ids))


register_attention_class(LlamaAttention)
