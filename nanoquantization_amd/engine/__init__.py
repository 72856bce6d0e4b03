"""Minimal single-GPU inference engine for the AWQ Qwen3 model: paged KV cache, greedy decoding,
decode step replayed from a HIP graph.  The reference has no engine; the model semantics it must
reproduce are those of nanoquantization/models/qwen3_quantized.py."""
from .llm_engine import LLMEngine, PagedKVCache  # noqa: F401
