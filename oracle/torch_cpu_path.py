"""The reference's linear path restated on CPU torch tensors -- the timed CPU baseline.

TEST / MEASUREMENT INFRASTRUCTURE, NOT PRODUCT.  The reference's only
dequant-from-packed code is a Triton kernel (nanoquantization/layers/gemm.py:10-123),
so "the reference's CPU path" is this restatement of the same three steps:

  1. unpack int32 -> 4-bit with shifts [0,16,4,20,8,24,12,28]   (layers/gemm.py:52-69)
  2. W = (q - z) * s in the scale dtype, [K, N]                  (layers/gemm.py:112)
  3. y = torch.matmul(x, W)                                      (layers/gemm.py:560-561)
"""
from __future__ import annotations

import torch

_SHIFTS = (0, 16, 4, 20, 8, 24, 12, 28)


def unpack(packed: torch.Tensor) -> torch.Tensor:
    sh = torch.tensor(_SHIFTS, dtype=torch.int32, device=packed.device)
    return ((packed.unsqueeze(-1) >> sh) & 0xF).reshape(packed.shape[0], -1)


def dequant(qweight: torch.Tensor, qscales: torch.Tensor, qzeros: torch.Tensor) -> torch.Tensor:
    g = qweight.shape[0] // qscales.shape[0]
    q = unpack(qweight)
    z = unpack(qzeros).repeat_interleave(g, dim=0)
    s = qscales.repeat_interleave(g, dim=0)
    return (q - z).to(qscales.dtype) * s


def linear(x: torch.Tensor, qweight, qscales, qzeros, upcast: bool = False) -> torch.Tensor:
    w = dequant(qweight, qscales, qzeros)
    if upcast:
        return torch.matmul(x.float(), w.float()).to(qscales.dtype)
    return torch.matmul(x.to(qscales.dtype), w)
