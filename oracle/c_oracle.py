"""ctypes binding of oracle/libawq_oracle.so (the plain-C oracle). Test infrastructure only."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libawq_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libawq_oracle.so"])
    return _SO


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def pack(iw: np.ndarray) -> np.ndarray:
    iw = np.ascontiguousarray(iw, dtype=np.int32)
    out = np.empty((iw.shape[0], iw.shape[1] // 8), dtype=np.int32)
    lib().awq_oracle_pack(_p(iw), ctypes.c_int64(iw.shape[0]), ctypes.c_int64(iw.shape[1]), _p(out))
    return out


def unpack(packed: np.ndarray) -> np.ndarray:
    packed = np.ascontiguousarray(packed, dtype=np.int32)
    out = np.empty((packed.shape[0], packed.shape[1] * 8), dtype=np.int32)
    lib().awq_oracle_unpack(_p(packed), ctypes.c_int64(packed.shape[0]), ctypes.c_int64(packed.shape[1]), _p(out))
    return out


def quantize_f32(w: np.ndarray, g: int):
    w = np.ascontiguousarray(w, dtype=np.float32)
    o, i = w.shape
    dq = np.empty_like(w)
    s = np.empty((o, i // g), np.float32)
    z = np.empty((o, i // g), np.float32)
    lib().awq_oracle_quantize_f32(_p(w), ctypes.c_int64(o), ctypes.c_int64(i), ctypes.c_int64(g), _p(dq), _p(s), _p(z))
    return dq, s, z


def dequant(qweight, qzeros, scales_bits, dtype: str) -> np.ndarray:
    qweight = np.ascontiguousarray(qweight, dtype=np.int32)
    qzeros = np.ascontiguousarray(qzeros, dtype=np.int32)
    scales_bits = np.ascontiguousarray(scales_bits, dtype=np.uint16)
    K, N = qweight.shape[0], qweight.shape[1] * 8
    g = K // scales_bits.shape[0]
    out = np.empty((K, N), np.uint16)
    lib().awq_oracle_dequant(_p(qweight), _p(qzeros), _p(scales_bits), ctypes.c_int64(K), ctypes.c_int64(N),
                             ctypes.c_int64(g), ctypes.c_int(dtype == "bf16"), _p(out))
    return out


def linear(x_bits, qweight, qzeros, scales_bits, dtype: str, bias=None) -> np.ndarray:
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    qweight = np.ascontiguousarray(qweight, dtype=np.int32)
    qzeros = np.ascontiguousarray(qzeros, dtype=np.int32)
    scales_bits = np.ascontiguousarray(scales_bits, dtype=np.uint16)
    M, K = x_bits.shape
    N = qweight.shape[1] * 8
    g = K // scales_bits.shape[0]
    y = np.empty((M, N), np.float32)
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    lib().awq_oracle_linear(_p(x_bits), _p(qweight), _p(qzeros), _p(scales_bits),
                            _p(b) if b is not None else None, ctypes.c_int64(M), ctypes.c_int64(K),
                            ctypes.c_int64(N), ctypes.c_int64(g), ctypes.c_int(dtype == "bf16"), _p(y))
    return y


def f16_roundtrip(x: np.ndarray):
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = np.empty(x.shape, np.uint16)
    back = np.empty(x.shape, np.float32)
    lib().awq_oracle_f16_roundtrip(_p(x), ctypes.c_int64(x.size), _p(bits), _p(back))
    return bits, back
