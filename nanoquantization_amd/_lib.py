"""Loaders of the two shared libraries: libawq_hip.so (the C ABI declared in include/awq_hip.h and
include/nq_engine_ops.h, bound with ctypes) and libawq_torch.so (the PyTorch operator binding over that ABI for the
linear path: torch.ops.nanoquantization_amd.*).

There is no fallback: if the library is missing or a call fails, an exception
is raised.
"""
from __future__ import annotations

import ctypes
import os
import threading

import torch

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "libawq_hip.so")

AWQ_F16, AWQ_BF16 = 0, 1
_STATUS = {1: "invalid argument", 2: "unsupported", 3: "workspace", 4: "HIP runtime"}

_lib = None
_lock = threading.Lock()

_vp, _i64, _int, _sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t
_LINEAR_ARGS = [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp, _sz, _vp]

# symbol -> (restype, argtypes); every symbol of include/awq_hip.h and include/nq_engine_ops.h
SYMBOLS = {
    "awq_hip_version": (_int, []),
    "awq_hip_last_error": (ctypes.c_char_p, []),
    "awq_dequantize": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "awq_dequantize_transposed": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "awq_quantize_pack": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "awq_gemv_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "awq_gemm_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "awq_linear_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "awq_gemv": (_int, _LINEAR_ARGS),
    "awq_gemv_static_scratch_bytes": (_sz, []),
    "awq_gemv_static": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "awq_gemv_swiglu": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp, _sz, _vp]),
    "awq_linear_swiglu": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp, _sz, _vp]),
    "awq_linear_swiglu_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "awq_gemv_qkv_rope_store": (_int, [_vp] * 12 + [_i64] * 9 + [ctypes.c_float, _int, _vp, _sz, _vp]),
    "awq_gemv_add_residual": (_int, [_vp] * 6 + [_i64] * 4 + [_int, _vp, _sz, _vp]),
    "awq_gemv_add_rmsnorm": (_int, [_vp] * 6 + [ctypes.c_float, _vp] + [_i64] * 4 + [_int, _vp, _sz, _vp]),
    "awq_gemv_rmsnorm": (_int, [_vp, _vp, _vp, ctypes.c_float] + [_vp] * 4 + [_i64] * 4 + [_int, _int, _vp, _sz, _vp]),
    "awq_gemv_rmsnorm_qkv_rope_store": (_int, [_vp, _vp, _vp, ctypes.c_float] + [_vp] * 11 + [_i64] * 9 +
                                        [ctypes.c_float, _int, _vp, _sz, _vp]),
    "awq_prefetch_hint": (_int, [_vp, _sz]),
    "awq_prefetch_pending": (_int, []),
    "awq_gemm": (_int, _LINEAR_ARGS),
    "awq_linear": (_int, _LINEAR_ARGS),
    "awq_gemv_plan": (_int, [_i64, _i64, _i64, _i64, ctypes.POINTER(_int), ctypes.POINTER(_int)]),
    "awq_gemm_plan": (_int, [_i64, _i64, _i64, _i64, _int, ctypes.POINTER(_int), ctypes.POINTER(_int)]),
    "awq_gemv_variant_count": (_int, []),
    "awq_gemm_variant_count": (_int, []),
    "awq_gemv_variant_name": (ctypes.c_char_p, [_int]),
    "awq_gemm_variant_name": (ctypes.c_char_p, [_int]),
    "awq_gemv_ex_workspace_bytes": (_sz, [_i64, _i64, _i64, _int, _int]),
    "awq_gemm_ex_workspace_bytes": (_sz, [_i64, _i64, _i64, _int, _int]),
    "awq_gemv_ex": (_int, _LINEAR_ARGS + [_int, _int]),
    "awq_gemm_ex": (_int, _LINEAR_ARGS + [_int, _int]),
    # include/nq_engine_ops.h
    "nq_add_rmsnorm": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, ctypes.c_float, _int, _vp]),
    "nq_row_ssq": (_int, [_vp, _vp, _i64, _i64, _int, _vp]),
    "nq_embed_row_ssq": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "nq_qk_norm_rope_store": (_int, [_vp] * 10 + [_i64] * 7 + [ctypes.c_float, _int, _vp]),
    "nq_paged_attention_workspace_bytes": (_sz, [_i64] * 5),
    "nq_paged_attention_decode": (_int, [_vp] * 6 + [_i64] * 7 + [ctypes.c_float, _int, _vp, _sz, _vp]),
    "nq_silu_mul": (_int, [_vp, _vp, _i64, _i64, _int, _vp]),
    "nq_silu_mul_interleaved": (_int, [_vp, _vp, _i64, _i64, _int, _vp]),
    "nq_argmax_rows": (_int, [_vp, _vp, _i64, _i64, _int, _vp]),
    "nq_decode_prepare": (_int, [_vp] * 5 + [_i64] * 3 + [_vp]),
    "nq_decode_advance": (_int, [_vp] * 6 + [_i64] * 2 + [_vp]),
}


class AwqHipError(RuntimeError):
    pass


def lib() -> ctypes.CDLL:
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                if not os.path.exists(LIB_PATH):
                    raise AwqHipError(
                        f"{LIB_PATH} is missing: build it with `python -m nanoquantization_amd.build` "
                        "(there is no CPU or eager fallback for the AWQ kernels)")
                handle = ctypes.CDLL(LIB_PATH)
                for name, (res, args) in SYMBOLS.items():
                    fn = getattr(handle, name)
                    fn.restype, fn.argtypes = res, args
                _lib = handle
    return _lib


TORCH_LIB_PATH = os.path.join(PKG_DIR, "libawq_torch.so")
_torch_ops = None


def torch_ops():
    """torch.ops.nanoquantization_amd: the operators of csrc/torch_binding.cpp (awq_dequantize, awq_linear,
    awq_linear_swiglu), registered with the dispatcher by loading libawq_torch.so.  Raises if it has not been built."""
    global _torch_ops
    if _torch_ops is None:
        lib()                                           # libawq_hip.so first: the binding links against it
        with _lock:
            if _torch_ops is None:
                if not os.path.exists(TORCH_LIB_PATH):
                    raise AwqHipError(
                        f"{TORCH_LIB_PATH} is missing: build it with `python -m nanoquantization_amd.build` "
                        "(there is no CPU or eager fallback for the AWQ kernels)")
                torch.ops.load_library(TORCH_LIB_PATH)
                _torch_ops = torch.ops.nanoquantization_amd
    return _torch_ops


def check(status: int) -> None:
    if status != 0:
        msg = lib().awq_hip_last_error().decode("utf-8", "replace")
        raise AwqHipError(f"libawq_hip: {_STATUS.get(status, status)}: {msg}")


def dtype_id(dtype: torch.dtype) -> int:
    if dtype == torch.float16:
        return AWQ_F16
    if dtype == torch.bfloat16:
        return AWQ_BF16
    raise AwqHipError(f"qscales dtype must be float16 or bfloat16, got {dtype}")


# Host-side shortcuts for the launch path (a decode-size launch takes ~5 us on the GPU; the wrappers around it
# should not take three times that).
class _NoContext:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_CONTEXT = _NoContext()


def on_device(device: torch.device):
    """Context manager that makes `device` current; free when it already is."""
    idx = device.index
    if idx is None or idx == torch._C._cuda_getDevice():
        return _NO_CONTEXT
    return torch.cuda.device(device)


def current_stream_ptr(device: torch.device) -> int:
    """The raw hipStream_t of torch's current stream on `device`."""
    idx = device.index
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice() if idx is None else idx)


_ws_bytes_cache: dict[tuple, int] = {}


def workspace_bytes(entry: str, M: int, N: int, K: int, extra: tuple = ()) -> int:
    """`<entry>_workspace_bytes(M, N, K, *extra)` of the library, remembered per shape."""
    key = (entry, M, N, K, extra)
    n = _ws_bytes_cache.get(key)
    if n is None:
        n = getattr(lib(), entry + "_workspace_bytes")(M, N, K, *extra)
        if len(_ws_bytes_cache) < 65536:
            _ws_bytes_cache[key] = n
    return n


# One zero-initialised split-K workspace per (device, stream).  The kernels leave
# it zeroed, and calls on one stream are ordered, so it is shared by every layer.
# A workspace is never freed: a HIP graph captured while it was current keeps its
# address in its kernel arguments, so when a larger one is needed the old tensor is
# retired, not released (its memory must not be handed to anyone else, and its
# arrival counters must stay zero between replays).
_workspaces: dict[tuple[int, int], torch.Tensor] = {}
_retired_workspaces: list[torch.Tensor] = []


def workspace(device: torch.device, stream_ptr: int, nbytes: int, _alloc=None) -> torch.Tensor | None:
    if nbytes == 0:
        return None
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream_ptr)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        if ws is not None:
            _retired_workspaces.append(ws)
        size = max(nbytes, 8 << 20)
        ws = (_alloc or torch.zeros)(size, dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws
