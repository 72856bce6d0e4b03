"""RMSNorm with the arithmetic of nanoquantization/layers/norm.py:10-35: normalise in fp32, cast back
to the input dtype, then multiply by the weight in that dtype.  Plain torch ops (adjacent to the AWQ
path, not a kernel of this library)."""
from __future__ import annotations

import torch
from torch import nn


class RMSNorm(nn.Module):
    def __init__(self, norm_size: int, eps: float = 1e-6) -> None:
        super().__init__()
        self.norm_size = norm_size
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(norm_size))

    def rms_norm(self, x: torch.Tensor) -> torch.Tensor:
        xf = x.float()
        xf = xf * torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + self.eps)
        return xf.to(x.dtype) * self.weight

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.rms_norm(x)
