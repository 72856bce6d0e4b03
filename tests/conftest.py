import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (MI355X); run with -m gpu")


def make_case(K, N, g, dtype, seed=0, w_std=0.02):
    """Seeded AWQ-packed linear built with the oracle: weight ~ N(0, w_std) [N, K] fp32."""
    from oracle import awq_oracle as o

    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((N, K)) * w_std).astype(np.float32)
    return o.make_packed(w, g, dtype)


def random_packed(K, N, g, dtype, seed=0, scale_lo=1e-3, scale_hi=2e-2):
    """Random nibbles / zeros / positive scales (every q, z combination shows up)."""
    from oracle import awq_oracle as o

    rng = np.random.default_rng(seed)
    iw = rng.integers(0, 16, size=(K, N), dtype=np.int32)
    z = rng.integers(0, 16, size=(K // g, N), dtype=np.int32)
    s = rng.uniform(scale_lo, scale_hi, size=(K // g, N)).astype(np.float32)
    return {"qweight": o.pack_awq(iw), "qzeros": o.pack_awq(z), "qscales": o.to_bits16(s, dtype),
            "intweight": iw}


def make_x(M, K, dtype, seed=1, std=1.0):
    from oracle import awq_oracle as o

    rng = np.random.default_rng(seed)
    return o.to_bits16((rng.standard_normal((M, K)) * std).astype(np.float32), dtype)


def torch_dtype(dtype):
    import torch

    return {"f16": torch.float16, "bf16": torch.bfloat16}[dtype]


def to_dev(bits_or_int, dtype=None, device="cuda"):
    """numpy int32 -> int32 tensor; numpy uint16 bits -> fp16/bf16 tensor."""
    import torch

    a = np.ascontiguousarray(bits_or_int)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).view(torch_dtype(dtype)).to(device)
    return torch.from_numpy(a).to(device)


def to_bits(t):
    """fp16/bf16 tensor -> numpy uint16 bit patterns."""
    import torch

    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)
