"""MI355X (gfx950) native AWQ W4A16 linear path.

Host-side mirror of nanoquantization/layers/gemm.py and
nanoquantization/utils/quantization.py of liyuan24/nanoquantization, running on
hand-written HIP kernels (csrc/) behind the C ABI of include/awq_hip.h.
"""
from .layers.gemm import (WQLinear_GEMM, awq_dequantize, awq_dequantize_transposed, awq_gemm,  # noqa: F401
                          prefetch_hint)
from .utils.quantization import pseudo_quantize, quantize_pack  # noqa: F401

__all__ = ["WQLinear_GEMM", "awq_dequantize", "awq_dequantize_transposed", "awq_gemm", "pseudo_quantize", "quantize_pack",
           "prefetch_hint"]
