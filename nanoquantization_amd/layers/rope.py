"""NeoX (half-split) rotary embedding with the arithmetic of nanoquantization/layers/rope.py:5-45:
a non-persistent cos|sin table [max_pos, 1, head_dim], rotation in fp32, result cast back."""
from __future__ import annotations

import torch
from torch import nn


class RoPE(nn.Module):
    def __init__(self, head_dim: int, max_position_embeddings: int, base: float = 10000):
        super().__init__()
        self.head_dim = head_dim
        self.max_position_embeddings = max_position_embeddings
        self.base = base
        self.register_buffer("cos_sin_cache", self._table("cpu"), persistent=False)

    def _table(self, device) -> torch.Tensor:
        inv_freq = 1.0 / (self.base ** (torch.arange(0, self.head_dim, 2, dtype=torch.float32, device=device)
                                        / self.head_dim))
        freqs = torch.outer(torch.arange(self.max_position_embeddings, dtype=torch.float32, device=device), inv_freq)
        return torch.cat([freqs.cos(), freqs.sin()], dim=-1).unsqueeze(1)

    def _apply(self, fn, *args, **kwargs):
        # model.to(bfloat16) must not round the angle table: keep it in fp32 wherever it lives
        super()._apply(fn, *args, **kwargs)
        if self.cos_sin_cache.dtype != torch.float32:
            self.cos_sin_cache = self._table(self.cos_sin_cache.device)
        return self

    @staticmethod
    def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
        x1, x2 = torch.chunk(x.float(), 2, dim=-1)
        return torch.cat([x1 * cos - x2 * sin, x1 * sin + x2 * cos], dim=-1).to(x.dtype)

    def forward(self, query: torch.Tensor, key: torch.Tensor, position_ids: torch.Tensor):
        """query/key: [batch, seq, heads, head_dim]; position_ids: [batch, seq] (or broadcastable)."""
        cos, sin = torch.chunk(self.cos_sin_cache[position_ids], 2, dim=-1)
        return self.apply_rope(query, cos, sin), self.apply_rope(key, cos, sin)
