"""Per-group min/max fake quantiser (the input generator of every AWQ linear).

Same contract as pseudo_quantize of nanoquantization/utils/quantization.py:5-58:
asymmetric (zero_point=True) maps [min, max] of each group onto 0..2^b-1,
symmetric maps [-absmax, absmax] onto -2^(b-1)..2^(b-1)-1; returns the
dequantised tensor, the scales [rows, cols/g] and the zero points (or None).
All arithmetic stays in the dtype and on the device of `x`.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch


def pseudo_quantize(
    x: torch.Tensor, group_size: int, w_bits: int, zero_point: bool
) -> Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    shape = x.shape
    if group_size > 0:
        assert shape[-1] % group_size == 0, "x.shape[-1] must be divisible by group_size"
        groups = x.reshape(-1, group_size)
    else:
        groups = x.reshape(-1, shape[-1])
    assert not bool(torch.isnan(groups).any()), "weight should not contain nan"

    if zero_point:
        q_hi, q_lo = float(2 ** w_bits - 1), 0.0
        lo, hi = torch.aminmax(groups, dim=-1, keepdim=True)
        scales = torch.clamp(hi - lo, min=1e-5) / q_hi
        zeros = torch.clamp(-torch.round(lo / scales), q_lo, q_hi)
        q = torch.clamp(torch.round(groups / scales) + zeros, q_lo, q_hi)
        deq = (q - zeros) * scales
        zeros_out = zeros.reshape(shape[0], -1)
    else:
        q_hi, q_lo = float(2 ** (w_bits - 1) - 1), float(-(2 ** (w_bits - 1)))
        scales = groups.abs().amax(dim=-1, keepdim=True) / q_hi
        deq = torch.clamp(torch.round(groups / scales), q_lo, q_hi) * scales
        zeros_out = None
    return deq.reshape(shape), scales.reshape(shape[0], -1), zeros_out


def quantize_pack(weight: torch.Tensor, group_size: int, output_dtype: torch.dtype = torch.bfloat16):
    """weight fp32 [N, K] on a HIP device -> (qweight int32 [K, N/8], qscales [K/g, N], qzeros int32
    [K/g, N/8]) in one kernel: the words that pseudo_quantize(weight, g, 4, True) followed by
    WQLinear_GEMM.from_linear would produce (utils/quantization.py:5-58, layers/gemm.py:447-550 of the
    reference), without the [N, K] temporaries."""
    from .. import _lib
    if weight.device.type != "cuda":
        raise _lib.AwqHipError(f"quantize_pack runs on a HIP device only (tensor is on {weight.device})")
    assert weight.dim() == 2 and weight.dtype == torch.float32, "an fp32 [out_features, in_features] weight"
    assert not bool(torch.isnan(weight).any()), "weight should not contain nan"
    weight = weight.contiguous()
    N, K = weight.shape
    g = K if group_size <= 0 else group_size
    assert K % g == 0 and N % 8 == 0
    dev = weight.device
    qweight = torch.empty(K, N // 8, dtype=torch.int32, device=dev)
    qzeros = torch.empty(K // g, N // 8, dtype=torch.int32, device=dev)
    qscales = torch.empty(K // g, N, dtype=output_dtype, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().awq_quantize_pack(weight.data_ptr(), qweight.data_ptr(), qscales.data_ptr(),
                                                qzeros.data_ptr(), N, K, g, _lib.dtype_id(output_dtype),
                                                torch.cuda.current_stream().cuda_stream))
    return qweight, qscales, qzeros
