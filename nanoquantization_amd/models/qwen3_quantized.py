"""Qwen3 with AWQ linears: the callers of the hot path, same modules, constructor arguments and
parameter/buffer names as nanoquantization/models/qwen3_quantized.py (so its checkpoints load
unchanged), on this package's WQLinear_GEMM.

`forward(x, position_ids)` is the reference's full-sequence causal forward (no cache,
models/qwen3_quantized.py:65-102, 139-153, 194-215, 259-273).  The engine
(nanoquantization_amd/engine) drives the same weights through a paged KV cache; the reference has
no counterpart for that.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..layers.gemm import WQLinear_GEMM
from ..layers.norm import RMSNorm
from ..layers.rope import RoPE


class Qwen3QuantizedAttention(nn.Module):
    def __init__(self, hidden_size: int, total_num_heads: int, total_num_kv_heads: int,
                 max_position_embeddings: int, w_bits: int = 4, group_size: int = 128,
                 head_dim: Optional[int] = None, rope_theta: float = 10000, rms_norm_eps: float = 1e-6):
        super().__init__()
        self.head_dim = head_dim or hidden_size // total_num_heads
        self.hidden_size = hidden_size
        self.num_heads = total_num_heads
        self.num_kv_heads = total_num_kv_heads
        self.max_position_embeddings = max_position_embeddings
        self.rope = RoPE(self.head_dim, max_position_embeddings, rope_theta)
        mk = lambda i, o: WQLinear_GEMM(w_bits=w_bits, group_size=group_size, in_features=i, out_features=o)
        self.q_proj = mk(hidden_size, total_num_heads * self.head_dim)
        self.k_proj = mk(hidden_size, total_num_kv_heads * self.head_dim)
        self.v_proj = mk(hidden_size, total_num_kv_heads * self.head_dim)
        self.o_proj = mk(total_num_heads * self.head_dim, hidden_size)
        self.q_norm = RMSNorm(self.head_dim, rms_norm_eps)
        self.k_norm = RMSNorm(self.head_dim, rms_norm_eps)

    def qkv(self, x: torch.Tensor, position_ids: torch.Tensor):
        """Projections, per-head q/k RMSNorm, rotary: [b, s, heads, d], [b, s, kv, d], [b, s, kv, d]."""
        bs = x.shape[0]
        if position_ids.dim() == 1:
            position_ids = position_ids.unsqueeze(0)
        q = self.q_proj(x).view(bs, -1, self.num_heads, self.head_dim)
        k = self.k_proj(x).view(bs, -1, self.num_kv_heads, self.head_dim)
        v = self.v_proj(x).view(bs, -1, self.num_kv_heads, self.head_dim)
        q, k = self.rope(self.q_norm(q), self.k_norm(k), position_ids)
        return q, k, v

    def forward(self, x: torch.Tensor, position_ids: torch.Tensor) -> torch.Tensor:
        bs = x.shape[0]
        q, k, v = self.qkv(x, position_ids)
        o = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2),
                                           is_causal=True, enable_gqa=self.num_heads != self.num_kv_heads)
        o = o.transpose(1, 2).reshape(bs, -1, self.num_heads * self.head_dim)
        return self.o_proj(o)


class Qwen3QuantizedMLP(nn.Module):
    def __init__(self, hidden_size: int, intermediate_size: int, w_bits: int = 4, group_size: int = 128):
        super().__init__()
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        mk = lambda i, o: WQLinear_GEMM(w_bits=w_bits, group_size=group_size, in_features=i, out_features=o)
        self.up_proj = mk(hidden_size, intermediate_size)
        self.gate_proj = mk(hidden_size, intermediate_size)
        self.down_proj = mk(intermediate_size, hidden_size)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.down_proj(F.silu(self.gate_proj(x)) * self.up_proj(x))


class Qwen3QuantizedBlock(nn.Module):
    def __init__(self, hidden_size: int, total_num_heads: int, total_num_kv_heads: int,
                 max_position_embeddings: int, intermediate_size: int, w_bits: int = 4, group_size: int = 128,
                 head_dim: Optional[int] = None, rope_theta: float = 10000, rms_norm_eps: float = 1e-6):
        super().__init__()
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.self_attn = Qwen3QuantizedAttention(hidden_size, total_num_heads, total_num_kv_heads,
                                                 max_position_embeddings, w_bits, group_size, head_dim,
                                                 rope_theta, rms_norm_eps)
        self.mlp = Qwen3QuantizedMLP(hidden_size, intermediate_size, w_bits, group_size)
        self.input_layernorm = RMSNorm(hidden_size, rms_norm_eps)
        self.post_attention_layernorm = RMSNorm(hidden_size, rms_norm_eps)

    def forward(self, x: torch.Tensor, position_ids: torch.Tensor) -> torch.Tensor:
        x = x + self.self_attn(self.input_layernorm(x), position_ids)
        return x + self.mlp(self.post_attention_layernorm(x))


class Qwen3QuantizedModel(nn.Module):
    def __init__(self, num_hidden_layers: int, vocab_size: int, hidden_size: int, total_num_heads: int,
                 total_num_kv_heads: int, max_position_embeddings: int, intermediate_size: int,
                 w_bits: int = 4, group_size: int = 128, head_dim: Optional[int] = None,
                 rope_theta: float = 10000, rms_norm_eps: float = 1e-6):
        super().__init__()
        self.layers = nn.ModuleList([
            Qwen3QuantizedBlock(hidden_size, total_num_heads, total_num_kv_heads, max_position_embeddings,
                                intermediate_size, w_bits, group_size, head_dim, rope_theta, rms_norm_eps)
            for _ in range(num_hidden_layers)])
        self.norm = RMSNorm(hidden_size, rms_norm_eps)
        self.embed_tokens = nn.Embedding(vocab_size, hidden_size)

    def forward(self, x: torch.Tensor, position_ids: torch.Tensor) -> torch.Tensor:
        x = self.embed_tokens(x)
        for layer in self.layers:
            x = layer(x, position_ids)
        return self.norm(x)


class Qwen3QuantizedForCausalLM(nn.Module):
    def __init__(self, num_hidden_layers: int, vocab_size: int, hidden_size: int, total_num_heads: int,
                 total_num_kv_heads: int, max_position_embeddings: int, intermediate_size: int,
                 w_bits: int = 4, group_size: int = 128, head_dim: Optional[int] = None,
                 tie_word_embeddings: bool = False, rope_theta: float = 10000, rms_norm_eps: float = 1e-6):
        super().__init__()
        self.model = Qwen3QuantizedModel(num_hidden_layers, vocab_size, hidden_size, total_num_heads,
                                         total_num_kv_heads, max_position_embeddings, intermediate_size,
                                         w_bits, group_size, head_dim, rope_theta, rms_norm_eps)
        self.lm_head = nn.Linear(hidden_size, vocab_size)   # un-quantised, with a bias, as in the reference
        if tie_word_embeddings:
            self.lm_head.weight.data = self.model.embed_tokens.weight.data

    def forward(self, x: torch.Tensor, position_ids: torch.Tensor) -> torch.Tensor:
        return self.model(x, position_ids)

    def logits(self, hidden_states: torch.Tensor) -> torch.Tensor:
        return self.lm_head(hidden_states)

    def compute_loss(self, x: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
        position_ids = torch.arange(x.shape[1], dtype=torch.int32, device=x.device).unsqueeze(0)
        logits = self.lm_head(self.model(x, position_ids))
        return F.cross_entropy(logits.view(-1, logits.shape[-1]).float(), labels.view(-1))
