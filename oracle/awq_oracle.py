"""CPU oracle for the AWQ W4A16 linear path -- TEST INFRASTRUCTURE, NOT PRODUCT.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this module.  The product (nanoquantization_amd/) never does: it runs on the
HIP kernels or fails.

A numpy restatement of the reference's arithmetic, written from its formulae
(citations are paths under the reference checkout):

  quantize_minmax      nanoquantization/utils/quantization.py:5-58
  int_quantize         nanoquantization/layers/gemm.py:479-491
  pack_awq             nanoquantization/layers/gemm.py:501-520 (weights), :522-548 (zeros)
  unpack_awq           nanoquantization/layers/gemm.py:52-69
  dequant              nanoquantization/layers/gemm.py:64-69,91,110-112 (+ :474 scale cast)
  linear_fp32          nanoquantization/layers/gemm.py:259,303-311,560-561 with the
                       accumulation done in fp32/fp64 (the tolerance oracle)
  linear_splitk_ref    nanoquantization/layers/gemm.py:217,251-253,313-326,378
                       (the reference's own rounding schedule: 8 interleaved
                       K-splits, each rounded to the output dtype, summed in it)

How each function is pinned (see tests/test_oracle.py):
  * pack/unpack: the hand-derived known-answer words 0x75316420, 0xFDB9ECA8,
    -1, 0x00010000, 0x10000000; exhaustive value x position round trip; a
    pure-Python nibble-by-nibble packer; the C restatement (oracle/awq_oracle.c).
  * quantize_minmax: closed forms (q, z in 0..15, s = max(max-min,1e-5)/15,
    half-to-even, constant groups, a hand-computed linspace group) and
    idempotence; torch arithmetic on the same formula as a library cross-check.
  * dequant: brute-force scalar loop, fp16/bf16 rounding checked against torch's
    own conversions, equality with quantize_minmax's x_dq where it must hold.
  * linear_fp32: reduces to a library matmul on the dequantised matrix.
  * linear_splitk_ref: what the schedule's arithmetic fixes -- one split of
    one block is the rounded fp32 product; a one-hot x returns one row of the
    dequantised weight for every split count (each K row owned by exactly one
    split); a scalar pure-Python walk of the kernel's own pointer arithmetic
    (pid_k * BLOCK_K start, stride BLOCK_K * SPLIT_K, per-split rounding, sum,
    final rounding) on integer-valued data where every fp32 sum is exact and
    the 16-bit roundings are active -- a contiguous (wrong) block assignment
    gives different bits on the same data.

bf16 values are carried as uint16 bit patterns (numpy has no bfloat16).
"""
from __future__ import annotations

import numpy as np

# nibble j of a packed word holds logical column AWQ_ORDER[j]  (gemm.py:504-513)
AWQ_ORDER = (0, 2, 4, 6, 1, 3, 5, 7)
# logical column c lives at bit AWQ_SHIFT[c]                   (gemm.py:52-69)
AWQ_SHIFT = (0, 16, 4, 20, 8, 24, 12, 28)


# --------------------------------------------------------------------------
# 16-bit float helpers
# --------------------------------------------------------------------------
def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> bfloat16 bit pattern (uint16), round-to-nearest-even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    lsb = (u >> 16) & 1
    r = ((u + 0x7FFF + lsb) >> 16).astype(np.uint16)
    r = np.where(nan, ((u >> 16) | 0x0040).astype(np.uint16), r)
    return r


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def to_dtype_f32(x32: np.ndarray, dtype: str) -> np.ndarray:
    """Round an fp32 array to `dtype` ('f16' | 'bf16' | 'f32') and return it as fp32."""
    if dtype == "f16":
        return x32.astype(np.float16).astype(np.float32)
    if dtype == "bf16":
        return bf16_bits_to_f32(f32_to_bf16_bits(x32))
    if dtype == "f32":
        return x32.astype(np.float32)
    raise ValueError(dtype)


def to_bits16(x32: np.ndarray, dtype: str) -> np.ndarray:
    """fp32 array -> uint16 bit patterns of its `dtype` rounding."""
    if dtype == "f16":
        return x32.astype(np.float16).view(np.uint16)
    if dtype == "bf16":
        return f32_to_bf16_bits(x32)
    raise ValueError(dtype)


def from_bits16(b: np.ndarray, dtype: str) -> np.ndarray:
    if dtype == "f16":
        return np.ascontiguousarray(b, dtype=np.uint16).view(np.float16).astype(np.float32)
    if dtype == "bf16":
        return bf16_bits_to_f32(b)
    raise ValueError(dtype)


# --------------------------------------------------------------------------
# a1: asymmetric / symmetric per-group min/max fake quantiser
# --------------------------------------------------------------------------
def quantize_minmax(w: np.ndarray, group_size: int, w_bits: int = 4, zero_point: bool = True):
    """utils/quantization.py:5-58.  w: [out, in] float32 (or float16).

    Returns (w_dq [out,in], scales [out, in/g], zeros [out, in/g] or None), all
    in w's dtype, every operation rounded in that dtype as torch does on CPU
    (true division, round half to even).
    """
    w = np.asarray(w)
    dt = w.dtype.type
    out_f, in_f = w.shape
    if group_size > 0:
        assert in_f % group_size == 0, "x.shape[-1] must be divisible by group_size"
        g = w.reshape(-1, group_size)
    else:
        g = w.reshape(out_f, in_f)
    assert not np.isnan(g).any(), "weight should not contain nan"
    if zero_point:
        qmax, qmin = dt(2 ** w_bits - 1), dt(0)
        hi = g.max(axis=1, keepdims=True)
        lo = g.min(axis=1, keepdims=True)
        s = (np.maximum((hi - lo).astype(dt), dt(1e-5)) / qmax).astype(dt)
        z = np.clip(-np.rint((lo / s).astype(dt)), qmin, qmax).astype(dt)
        q = np.clip((np.rint((g / s).astype(dt)) + z).astype(dt), qmin, qmax).astype(dt)
        dq = ((q - z).astype(dt) * s).astype(dt)
        zeros = z.reshape(out_f, -1)
    else:
        qmax, qmin = dt(2 ** (w_bits - 1) - 1), dt(-(2 ** (w_bits - 1)))
        s = (np.abs(g).max(axis=1, keepdims=True) / qmax).astype(dt)
        q = np.clip(np.rint((g / s).astype(dt)), qmin, qmax).astype(dt)
        dq = (q * s).astype(dt)
        zeros = None
    return dq.reshape(out_f, in_f), s.reshape(out_f, -1), zeros


# --------------------------------------------------------------------------
# a3: real quantise + AWQ-order pack
# --------------------------------------------------------------------------
def int_quantize(w: np.ndarray, scales_gn: np.ndarray, zeros_gn: np.ndarray, group_size: int) -> np.ndarray:
    """layers/gemm.py:479-491.  w [N,K]; scales/zeros [K/g, N] -> int32 [K, N].

    iw[k, n] = int32(round(w[n, k] / s[k//g, n] + z[k//g, n])); no clamp.
    """
    dt = w.dtype.type
    s = np.repeat(scales_gn.astype(dt), group_size, axis=0)   # [K, N]
    z = np.repeat(zeros_gn.astype(dt), group_size, axis=0)
    t = ((w.T / s).astype(dt) + z).astype(dt)
    return np.rint(t).astype(np.int32)


def pack_awq(iw: np.ndarray) -> np.ndarray:
    """layers/gemm.py:501-520.  int [R, C] with values 0..15 -> int32 [R, C/8].

    word[r, i] = OR_j iw[r, 8i + AWQ_ORDER[j]] << 4j, kept as two's-complement int32.
    """
    iw = np.asarray(iw)
    rows, cols = iw.shape
    assert cols % 8 == 0
    v = iw.astype(np.int64).astype(np.uint32).reshape(rows, cols // 8, 8)
    word = np.zeros((rows, cols // 8), dtype=np.uint32)
    for j, c in enumerate(AWQ_ORDER):
        word |= (v[:, :, c] << np.uint32(4 * j)).astype(np.uint32)
    return word.view(np.int32)


def unpack_awq(packed: np.ndarray) -> np.ndarray:
    """layers/gemm.py:52-69.  int32 [R, C/8] -> int32 [R, C] (values 0..15)."""
    p = np.ascontiguousarray(packed, dtype=np.int32).view(np.uint32)
    rows, words = p.shape
    out = np.empty((rows, words, 8), dtype=np.int32)
    for c, sh in enumerate(AWQ_SHIFT):
        out[:, :, c] = ((p >> np.uint32(sh)) & np.uint32(0xF)).astype(np.int32)
    return out.reshape(rows, words * 8)


def make_packed(w: np.ndarray, group_size: int, dtype: str):
    """a1 -> transpose -> a3, the recipe of awq/quantizer.py:156-167.

    w [N, K] float32 -> dict(qweight int32 [K,N/8], qzeros int32 [K/g,N/8],
    qscales uint16 bits [K/g,N] in `dtype`, w_dq [N,K] float32).
    """
    w_dq, s, z = quantize_minmax(w, group_size, 4, True)
    s_gn = np.ascontiguousarray(s.T)
    z_gn = np.ascontiguousarray(z.T)
    iw = int_quantize(w_dq, s_gn, z_gn, group_size)
    return {
        "qweight": pack_awq(iw),
        "qzeros": pack_awq(z_gn.astype(np.int32)),
        "qscales": to_bits16(s_gn.astype(np.float32), dtype),   # gemm.py:474
        "w_dq": w_dq,
        "scales_gn": s_gn,
        "zeros_gn": z_gn,
        "intweight": iw,
    }


# --------------------------------------------------------------------------
# a4: dequantise
# --------------------------------------------------------------------------
def dequant(qweight: np.ndarray, qzeros: np.ndarray, qscales_bits: np.ndarray, dtype: str) -> np.ndarray:
    """layers/gemm.py:64-69,91,112.  Returns W [K, N] as uint16 bits of `dtype`.

    W = RN_dtype(float(q - z) * s): q - z is an exact small integer, s is already
    in `dtype`, the product is exact in fp32 and rounded once.
    """
    K = qweight.shape[0]
    G = qscales_bits.shape[0]
    assert K % G == 0
    g = K // G
    q = unpack_awq(qweight)
    z = np.repeat(unpack_awq(qzeros), g, axis=0)
    s = np.repeat(from_bits16(qscales_bits, dtype), g, axis=0)
    prod = (q - z).astype(np.float32) * s          # exact: <=5 bits x <=11 bits
    return to_bits16(prod, dtype)


def dequant_f32(qweight, qzeros, qscales_bits, dtype) -> np.ndarray:
    return from_bits16(dequant(qweight, qzeros, qscales_bits, dtype), dtype)


# --------------------------------------------------------------------------
# a5-a7: linear
# --------------------------------------------------------------------------
def linear_fp32(x_bits: np.ndarray, qweight, qzeros, qscales_bits, dtype: str, bias_f32=None) -> np.ndarray:
    """y_ref [M, N] float32 = x.float() @ dequant(W).float() (+ bias), accumulated
    in float64 and returned as float32 -- the tolerance oracle for every GEMM regime."""
    x = from_bits16(x_bits, dtype).astype(np.float64)
    w = dequant_f32(qweight, qzeros, qscales_bits, dtype).astype(np.float64)
    y = x @ w
    if bias_f32 is not None:
        y = y + bias_f32.astype(np.float64)[None, :]
    return y.astype(np.float32)


def linear_splitk_ref(x_bits, qweight, qzeros, qscales_bits, dtype: str, split_k: int = 8, block_k: int = 32):
    """The reference kernel's rounding schedule (gemm.py:217,313-326,378): split s
    owns K-blocks s, s+S, s+2S, ... of `block_k` rows; fp32 accumulate inside a
    split; each partial rounded to `dtype`; partials summed and rounded to `dtype`.
    Returns uint16 bits [M, N]."""
    x = from_bits16(x_bits, dtype)
    w = dequant_f32(qweight, qzeros, qscales_bits, dtype)
    K = w.shape[0]
    nblk = K // block_k
    parts = []
    for s in range(split_k):
        rows = np.concatenate([np.arange(b * block_k, (b + 1) * block_k) for b in range(s, nblk, split_k)]) \
            if s < nblk else np.zeros(0, dtype=np.int64)
        p = (x[:, rows].astype(np.float32) @ w[rows, :].astype(np.float32)) if rows.size else \
            np.zeros((x.shape[0], w.shape[1]), np.float32)
        parts.append(to_dtype_f32(p.astype(np.float32), dtype))
    tot = np.sum(np.stack(parts, 0).astype(np.float32), axis=0)
    return to_bits16(tot.astype(np.float32), dtype)


def max_rel_err(y: np.ndarray, y_ref: np.ndarray) -> float:
    """max|y - y_ref| / max|y_ref| -- the normalisation the 1e-2 bound is stated on."""
    y = np.asarray(y, dtype=np.float64)
    y_ref = np.asarray(y_ref, dtype=np.float64)
    den = float(np.max(np.abs(y_ref)))
    return float(np.max(np.abs(y - y_ref))) / (den if den > 0 else 1.0)


def packed_weight_bytes(K: int, N: int, g: int = 128) -> int:
    """K*N/2 (qweight) + (K/g)*N/2 (qzeros) + 2*(K/g)*N (scales)."""
    return K * N // 2 + (K // g) * N // 2 + 2 * (K // g) * N
