"""AWQ W4A16 linear on MI355X: the module and free functions of
nanoquantization/layers/gemm.py, on hand-written HIP kernels.

Same constructor, buffers, `from_linear` and `forward` as the reference's
WQLinear_GEMM (layers/gemm.py:382-567); `awq_dequantize` / `awq_gemm` keep the
reference's signatures (:126-132, :329-338; the Triton tile-size keywords are
accepted and ignored).  Packed layout: qweight int32 [K, N/8], qzeros int32
[K/g, N/8], qscales fp16|bf16 [K/g, N]; nibble j of a word is logical column
8i + [0,2,4,6,1,3,5,7][j].

Every tensor handed to a kernel must live on a HIP device; there is no CPU path.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from .. import _lib

AWQ_SUPPORTED_GROUP_SIZES = [-1, 32, 64, 128]
_PACK_ORDER = (0, 2, 4, 6, 1, 3, 5, 7)


def _require_device(*tensors: torch.Tensor) -> torch.device:
    dev = tensors[0].device
    if dev.type != "cuda":
        raise _lib.AwqHipError(
            "AWQ kernels run on a HIP device only (tensor is on %s); there is no CPU fallback" % dev)
    for t in tensors:
        if t.device != dev:
            raise _lib.AwqHipError(f"tensors on different devices: {t.device} vs {dev}")
    return dev


def _ptr(t):
    return None if t is None else t.data_ptr()


def _check_packed(qweight, qscales, qzeros):
    K = qweight.shape[0]
    N = qscales.shape[1]
    assert K > 0 and N > 0
    group_size = K // qscales.shape[0]
    assert qweight.dtype == torch.int32 and qzeros.dtype == torch.int32
    assert qweight.shape[1] == N // 8
    assert qscales.shape[0] == K // group_size and qscales.shape[1] == N
    assert qzeros.shape[0] == K // group_size and qzeros.shape[1] == N // 8
    assert group_size <= K
    assert group_size in AWQ_SUPPORTED_GROUP_SIZES or group_size == K
    return K, N, group_size


def awq_dequantize(
    qweight: torch.Tensor,
    qscales: torch.Tensor,
    qzeros: torch.Tensor,
    block_size_x: int = 32,
    block_size_y: int = 32,
) -> torch.Tensor:
    """Packed int4 -> [K, N] weight in qscales.dtype, bit-exact RN((q - z) * s)."""
    _check_packed(qweight, qscales, qzeros)
    _require_device(qweight, qscales, qzeros)
    _lib.dtype_id(qscales.dtype)
    return _lib.torch_ops().awq_dequantize(qweight, qscales, qzeros)


def awq_dequantize_transposed(qweight: torch.Tensor, qscales: torch.Tensor, qzeros: torch.Tensor) -> torch.Tensor:
    """Packed int4 -> [N, K] weight (k-contiguous rows) in qscales.dtype: awq_dequantize(...).t(), bit for bit.
    A free-standing utility (the layout dense GEMM libraries like best); the linear itself never materialises the
    weight: every M runs the fused dequant + MFMA kernel."""
    K, N, g = _check_packed(qweight, qscales, qzeros)
    dev = _require_device(qweight, qscales, qzeros)
    qweight, qscales, qzeros = qweight.contiguous(), qscales.contiguous(), qzeros.contiguous()
    out = torch.empty(N, K, dtype=qscales.dtype, device=dev)
    with _lib.on_device(dev):
        stream = _lib.current_stream_ptr(dev)
        _lib.check(_lib.lib().awq_dequantize_transposed(_ptr(qweight), _ptr(qscales), _ptr(qzeros), _ptr(out),
                                                        K, N, g, _lib.dtype_id(qscales.dtype), stream))
    return out


def _linear(entry: str, x, qweight, qscales, qzeros, bias, extra=()):
    K, N, g = _check_packed(qweight, qscales, qzeros)
    assert x.dim() == 2 and x.shape[1] == K
    dev = _require_device(x, qweight, qscales, qzeros)
    M = x.shape[0]
    dt = qscales.dtype
    if x.dtype != dt:  # the reference casts x to the output dtype on load (layers/gemm.py:259)
        x = x.to(dt)
    if not (x.is_contiguous() and qweight.is_contiguous() and qscales.is_contiguous() and qzeros.is_contiguous()):
        x, qweight, qscales, qzeros = x.contiguous(), qweight.contiguous(), qscales.contiguous(), qzeros.contiguous()
    if bias is not None and (bias.dtype != dt or bias.device != dev or not bias.is_contiguous()):
        bias = bias.to(device=dev, dtype=dt).contiguous()
    out = torch.empty(M, N, dtype=dt, device=dev)
    if M == 0:
        return out
    L = _lib.lib()
    with _lib.on_device(dev):
        stream = _lib.current_stream_ptr(dev)
        nbytes = _lib.workspace_bytes(entry, M, N, K, tuple(extra))
        ws = _lib.workspace(dev, stream, nbytes) if nbytes else None
        status = getattr(L, entry)(x.data_ptr(), qweight.data_ptr(), qscales.data_ptr(), qzeros.data_ptr(), _ptr(bias),
                                   out.data_ptr(), M, N, K, g, _lib.dtype_id(dt), _ptr(ws),
                                   0 if ws is None else ws.numel(), stream, *extra)
        if status:
            _lib.check(status)
    return out


def prefetch_hint(*next_buffers: torch.Tensor) -> None:
    """Tell the next decode-regime AWQ launch of this thread to also pull the given tensors (the packed qweight,
    qscales, qzeros of the launch after it; at most four) into the Infinity Cache with workgroups it would leave
    idle.  Results never change."""
    L = _lib.lib()
    for t in next_buffers:
        if t.device.type != "cuda" or t.data_ptr() % 128 != 0:
            continue
        _lib.check(L.awq_prefetch_hint(t.data_ptr(), t.numel() * t.element_size()))


def awq_gemm(
    x: torch.Tensor,
    qweight: torch.Tensor,
    qscales: torch.Tensor,
    qzeros: torch.Tensor,
    split_k_iters: int,
    block_size_m: int = 32,
    block_size_n: int = 32,
    block_size_k: int = 32,
) -> torch.Tensor:
    """y[M, N] = x[M, K] @ dequant(W), fp32 accumulation, output in qscales.dtype.

    `split_k_iters` must be a power of two as in the reference; the kernels pick
    their own K split (the reduction is in fp32 and in a fixed order).
    """
    assert split_k_iters & (split_k_iters - 1) == 0
    K, N, g = _check_packed(qweight, qscales, qzeros)
    assert x.dim() == 2 and x.shape[1] == K
    _require_device(x, qweight, qscales, qzeros)
    _lib.dtype_id(qscales.dtype)
    return _lib.torch_ops().awq_linear(x, qweight, qscales, qzeros, None)


def awq_gemv_variant(x, qweight, qscales, qzeros, variant: int, split_k: int, bias=None):
    """Decode GEMV with a forced kernel variant and K split (tuning / tests)."""
    return _linear("awq_gemv_ex", x, qweight, qscales, qzeros, bias, (variant, split_k))


def awq_gemm_variant(x, qweight, qscales, qzeros, variant: int, split_k: int, bias=None):
    """Fused dequant+MFMA GEMM with a forced tile variant and K split (tuning / tests)."""
    return _linear("awq_gemm_ex", x, qweight, qscales, qzeros, bias, (variant, split_k))


_AWQ_LINEAR_OP = None


def _linear_op():
    """torch.ops.nanoquantization_amd.awq_linear (argument checks, output allocation, workspace and the launch on
    torch's current stream all happen in the C++ binding), looked up once."""
    global _AWQ_LINEAR_OP
    if _AWQ_LINEAR_OP is None:
        _AWQ_LINEAR_OP = _lib.torch_ops().awq_linear.default
    return _AWQ_LINEAR_OP


def pack_awq(intweight: torch.Tensor) -> torch.Tensor:
    """int [R, C] -> int32 [R, C/8]: word[r, i] = OR_j intweight[r, 8i + order[j]] << 4j."""
    rows, cols = intweight.shape
    v = intweight.to(torch.int64).reshape(rows, cols // 8, 8)
    word = torch.zeros(rows, cols // 8, dtype=torch.int64, device=intweight.device)
    for j, c in enumerate(_PACK_ORDER):
        word |= v[:, :, c] << (4 * j)
    # keep the low 32 bits as a two's-complement int32, as int32 shifts/ors would
    word &= 0xFFFFFFFF
    word = torch.where(word >= 2 ** 31, word - 2 ** 32, word)
    return word.to(torch.int32)


class WQLinear_GEMM(nn.Module):
    def __init__(
        self,
        w_bits: int,
        group_size: int,
        in_features: int,
        out_features: int,
        device: "str | torch.device" = "cpu",
        bias: bool = False,
        output_dtype: torch.dtype = torch.bfloat16,
    ):
        super().__init__()
        if w_bits not in [4]:
            raise ValueError("Only 4-bit quantization is supported")
        self.w_bits = w_bits
        self.group_size = group_size
        self.in_features = in_features
        self.out_features = out_features
        self.device = device
        pack = 32 // w_bits
        assert in_features % group_size == 0, "in_features must be divisible by group_size"
        assert out_features % pack == 0, "out_features must be divisible by (32 // self.w_bits)"
        groups = in_features // group_size
        self.register_buffer(
            "qweight", torch.zeros(in_features, out_features // pack, dtype=torch.int32, device=device))
        self.register_buffer(
            "qscales", torch.zeros(groups, out_features, dtype=output_dtype, device=device))
        self.register_buffer(
            "qzeros", torch.zeros(groups, out_features // pack, dtype=torch.int32, device=device))
        if bias:
            # bf16 whatever output_dtype is, as in the reference (layers/gemm.py:435-443)
            self.register_buffer("bias", torch.zeros(out_features, dtype=torch.bfloat16, device=device))
        else:
            self.bias = None

    @classmethod
    def from_linear(
        cls,
        linear_layer: nn.Linear,
        w_bits: int,
        group_size: int,
        scales: torch.Tensor,
        zeros: torch.Tensor,
        output_dtype: torch.dtype = torch.bfloat16,
    ) -> "WQLinear_GEMM":
        """linear_layer.weight [N, K] holds already fake-quantised values; scales and
        zeros are [K/g, N].  Produces the packed buffers of layers/gemm.py:474-548,
        word for word, without the per-column Python loops."""
        awq_linear = cls(
            w_bits,
            group_size,
            linear_layer.in_features,
            linear_layer.out_features,
            linear_layer.weight.device,
            linear_layer.bias is not None,
            output_dtype,
        )
        awq_linear.qscales = scales.detach().clone().to(output_dtype)
        if linear_layer.bias is not None:
            awq_linear.bias = linear_layer.bias.detach().clone().to(output_dtype)

        w = linear_layer.weight.data
        K = awq_linear.in_features
        rows = []
        # iw[k, n] = round(w[n, k] / s[k // g, n] + z[k // g, n]); whole groups at a time,
        # in slabs that keep the temporaries small for 10^8-weight layers
        slab = max(group_size, (1 << 24) // max(1, awq_linear.out_features) // group_size * group_size)
        for k0 in range(0, K, slab):
            k1 = min(K, k0 + slab)
            s = scales[k0 // group_size:k1 // group_size].repeat_interleave(group_size, dim=0)
            z = zeros[k0 // group_size:k1 // group_size].repeat_interleave(group_size, dim=0)
            rows.append(torch.round(w[:, k0:k1].t() / s + z).to(torch.int32))
        intweight = torch.cat(rows, dim=0)
        awq_linear.qweight = pack_awq(intweight)
        awq_linear.qzeros = pack_awq(zeros.to(torch.int32))
        return awq_linear

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        # One regime switch inside the library: split-K GEMV for <= 16 tokens, fused dequant + MFMA GEMM above; the
        # bias is added in the kernel epilogue.  The output is a fresh tensor outside autograd, as under the
        # reference's @torch.no_grad (layers/gemm.py:552); buffers are fetched from the module's dictionary directly
        # (nn.Module.__getattr__ costs more than the rest of this function).
        buf = self._buffers
        bias = buf["bias"] if "bias" in buf else self.bias
        if bias is not None and bias.dtype != buf["qscales"].dtype:
            # the bias buffer is bf16 whatever the output type (layers/gemm.py:435-443): convert once, not per call
            key = (bias.data_ptr(), bias._version, buf["qscales"].dtype, bias.device)
            cached = self.__dict__.get("_bias_cast")
            if cached is None or cached[0] != key:
                cached = (key, bias.to(buf["qscales"].dtype))
                self.__dict__["_bias_cast"] = cached
            bias = cached[1]
        if x.device.type != "cuda":
            raise _lib.AwqHipError(
                "AWQ kernels run on a HIP device only (tensor is on %s); there is no CPU fallback" % x.device)
        op = _AWQ_LINEAR_OP or _linear_op()
        if x.dim() == 2:
            return op(x, buf["qweight"], buf["qscales"], buf["qzeros"], bias)
        out_shape = x.shape[:-1] + (self.out_features,)
        return op(x.reshape(-1, x.shape[-1]), buf["qweight"], buf["qscales"], buf["qzeros"], bias).reshape(out_shape)

    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, "
                f"w_bits={self.w_bits}, group_size={self.group_size}, bias={self.bias is not None}")
