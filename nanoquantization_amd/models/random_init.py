"""Random-weight AWQ Qwen3 models for tests and benchmarks: weights ~ N(0, std) quantised with the
plain min/max routine and packed -- the recipe of nanoquantization/awq/quantizer.py:150-170 without
the calibration search.  On a HIP device the one-kernel quantise+pack does it (same words as
pseudo_quantize followed by WQLinear_GEMM.from_linear); elsewhere the torch routines do."""
from __future__ import annotations

import torch
import torch.nn as nn

from ..layers.gemm import WQLinear_GEMM
from ..utils.quantization import pseudo_quantize, quantize_pack
from .qwen3_quantized import Qwen3QuantizedForCausalLM

QWEN3_32B = dict(num_hidden_layers=64, vocab_size=151936, hidden_size=5120, total_num_heads=64,
                 total_num_kv_heads=8, max_position_embeddings=40960, intermediate_size=25600, head_dim=128,
                 tie_word_embeddings=False, rope_theta=1000000.0, rms_norm_eps=1e-6)

QWEN3_0P6B = dict(num_hidden_layers=28, vocab_size=151936, hidden_size=1024, total_num_heads=16,
                  total_num_kv_heads=8, max_position_embeddings=40960, intermediate_size=3072, head_dim=128,
                  tie_word_embeddings=True, rope_theta=1000000.0, rms_norm_eps=1e-6)


def fill_awq_linear(mod: WQLinear_GEMM, gen: torch.Generator, std: float, device, dtype) -> None:
    w = torch.randn(mod.out_features, mod.in_features, generator=gen, device=device, dtype=torch.float32) * std
    if w.device.type == "cuda" and mod.w_bits == 4:
        mod.qweight, mod.qscales, mod.qzeros = quantize_pack(w, mod.group_size, dtype)
        return
    dq, s, z = pseudo_quantize(w, mod.group_size, mod.w_bits, True)
    lin = nn.Linear(mod.in_features, mod.out_features, bias=False, device=device)
    lin.weight.data = dq
    packed = WQLinear_GEMM.from_linear(lin, mod.w_bits, mod.group_size, s.t().contiguous(), z.t().contiguous(), dtype)
    mod.qweight, mod.qzeros, mod.qscales = packed.qweight, packed.qzeros, packed.qscales


def random_awq_qwen3(config: dict, seed: int = 0, std: float = 0.02, device="cuda", dtype=torch.bfloat16,
                     w_bits: int = 4, group_size: int = 128) -> Qwen3QuantizedForCausalLM:
    model = Qwen3QuantizedForCausalLM(w_bits=w_bits, group_size=group_size, **config).to(dtype).to(device)
    gen = torch.Generator(device=device).manual_seed(seed)
    for mod in model.modules():
        if isinstance(mod, WQLinear_GEMM):
            fill_awq_linear(mod, gen, std, device, dtype)
    emb = model.model.embed_tokens.weight
    emb.data = (torch.randn(emb.shape, generator=gen, device=device, dtype=torch.float32) * std).to(dtype)
    if config.get("tie_word_embeddings", False):
        model.lm_head.weight.data = emb.data
    else:
        model.lm_head.weight.data = (torch.randn(emb.shape, generator=gen, device=device, dtype=torch.float32) * std).to(dtype)
    model.lm_head.bias.data.zero_()   # the reference leaves this bias at its random init when loading HF weights
    return model.eval()
