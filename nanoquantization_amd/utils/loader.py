"""Checkpoint I/O in the reference's on-disk format.

load_model follows nanoquantization/utils/loader.py:20-48 (every key of every *.safetensors in a
directory is copied into the parameter or buffer of that name); save_quantized_model writes what
scripts/qwen3_0pt6_billion.py:188-235 writes: model.safetensors, its index, and a config.json whose
quantization_config carries w_bits / group_size (tokenizer and hub upload are out of scope).
"""
from __future__ import annotations

import glob
import json
import os

import torch
from safetensors import safe_open
from safetensors.torch import save_file
from torch import nn


def load_model(model: nn.Module, path: str) -> None:
    for tensor_file in sorted(glob.glob(os.path.join(path, "*.safetensors"))):
        with safe_open(tensor_file, framework="pt", device="cpu") as f:
            for name in f.keys():
                try:
                    tensor = model.get_parameter(name)
                except AttributeError:
                    try:
                        tensor = model.get_buffer(name)
                    except AttributeError:
                        raise AttributeError(f"`{name}` is neither a parameter nor a buffer in the model")
                tensor.data.copy_(f.get_tensor(name))


def save_quantized_model(model: nn.Module, output_dir: str, config: dict, w_bits: int = 4, group_size: int = 128,
                         zero_point: bool = True) -> None:
    os.makedirs(output_dir, exist_ok=True)
    # tied lm_head / embedding share storage: safetensors refuses aliases, so clone every tensor
    state = {k: v.detach().cpu().contiguous().clone() for k, v in model.state_dict().items()}
    save_file(state, os.path.join(output_dir, "model.safetensors"))
    with open(os.path.join(output_dir, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {"format": "pt"}, "weight_map": {k: "model.safetensors" for k in state}}, f, indent=2)
    cfg = dict(config)
    cfg["quantization_config"] = {"quant_method": "awq", "w_bits": w_bits, "group_size": group_size,
                                  "zero_point": zero_point, "version": "gemm", "modules_to_not_convert": []}
    with open(os.path.join(output_dir, "config.json"), "w") as f:
        json.dump(cfg, f, indent=2)


def model_from_config(path: str, device="cpu", dtype=torch.bfloat16):
    """Build Qwen3QuantizedForCausalLM from a checkpoint directory's config.json and load its weights
    (scripts/load_quantized_model.py:19-36)."""
    from ..models.qwen3_quantized import Qwen3QuantizedForCausalLM
    cfg = json.load(open(os.path.join(path, "config.json")))
    q = cfg["quantization_config"]
    model = Qwen3QuantizedForCausalLM(
        num_hidden_layers=cfg["num_hidden_layers"], vocab_size=cfg["vocab_size"], hidden_size=cfg["hidden_size"],
        total_num_heads=cfg["num_attention_heads"], total_num_kv_heads=cfg["num_key_value_heads"],
        max_position_embeddings=cfg["max_position_embeddings"], intermediate_size=cfg["intermediate_size"],
        w_bits=q["w_bits"], group_size=q["group_size"], head_dim=cfg.get("head_dim"),
        tie_word_embeddings=cfg.get("tie_word_embeddings", False), rope_theta=cfg.get("rope_theta", 10000),
        rms_norm_eps=cfg.get("rms_norm_eps", 1e-6))
    model = model.to(dtype)
    load_model(model, path)
    return model.to(device)
