"""awq_gemv_static: the GEMV entry point that allocates nothing (static device scratch) against awq_gemv."""
import ctypes

import pytest
import torch

from nanoquantization_amd import _lib

pytestmark = pytest.mark.gpu


def _case(M, K, N, dtype, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (K, N // 8), dtype=torch.int32, device="cuda", generator=g)
    qz = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 128, N // 8), dtype=torch.int32, device="cuda", generator=g)
    qs = (torch.rand(K // 128, N, device="cuda", generator=g) * 0.02 + 0.001).to(dtype)
    x = torch.randn(M, K, device="cuda", generator=g).to(dtype)
    bias = torch.randn(N, device="cuda", generator=g).to(dtype)
    return x, qw, qs, qz, bias


def _both(L, M, K, N, dtype, seed, with_bias):
    x, qw, qs, qz, bias = _case(M, K, N, dtype, seed)
    b = bias.data_ptr() if with_bias else None
    did = _lib.dtype_id(dtype)
    stream = _lib.current_stream_ptr(x.device)
    nbytes = L.awq_gemv_workspace_bytes(M, N, K)
    ws = torch.zeros(max(nbytes, 16), dtype=torch.uint8, device="cuda")
    want = torch.empty(M, N, dtype=dtype, device="cuda")
    _lib.check(L.awq_gemv(x.data_ptr(), qw.data_ptr(), qs.data_ptr(), qz.data_ptr(), b, want.data_ptr(), M, N, K, 128,
                          did, ws.data_ptr(), ws.numel(), stream))
    got = torch.full((M, N), float("nan"), dtype=dtype, device="cuda")
    before = torch.cuda.memory_allocated()
    _lib.check(L.awq_gemv_static(x.data_ptr(), qw.data_ptr(), qs.data_ptr(), qz.data_ptr(), b, got.data_ptr(), M, N, K,
                                 128, did, stream))
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    return got, want, nbytes


def test_gemv_static_equals_gemv_on_two_calls_in_a_row():
    L = _lib.lib()
    cap = L.awq_gemv_static_scratch_bytes()
    assert cap == (16 << 10) + (16 << 20)
    # a split-K shape that uses most of what a decode GEMV ever needs, then a smaller one on the same scratch, then
    # more rows, a shape without K split, and the first again
    for i, (M, K, N, dtype, bias) in enumerate([(16, 5120, 25600, torch.bfloat16, False),
                                                 (3, 2048, 1024, torch.float16, True),
                                                 (32, 3072, 1024, torch.bfloat16, False),
                                                 (1, 1024, 3072, torch.float16, False),
                                                 (16, 5120, 25600, torch.bfloat16, True)]):
        print(f"gemv_static M={M} K={K} N={N} {dtype} bias={bias}", flush=True)
        got, want, nbytes = _both(L, M, K, N, dtype, 100 + i, bias)
        assert nbytes <= cap
        assert torch.equal(got, want), (M, K, N)


def test_gemv_static_rejects_what_does_not_fit():
    L = _lib.lib()
    M, K, N = 64, 25600, 5120          # shared-chunk kernel, 25 K-splits of 64 x 5120 fp32 partials
    assert L.awq_gemv_workspace_bytes(M, N, K) > L.awq_gemv_static_scratch_bytes()
    x, qw, qs, qz, _ = _case(M, K, N, torch.bfloat16, 7)
    y = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
    rc = L.awq_gemv_static(x.data_ptr(), qw.data_ptr(), qs.data_ptr(), qz.data_ptr(), None, y.data_ptr(), M, N, K, 128,
                           _lib.AWQ_BF16, _lib.current_stream_ptr(x.device))
    assert rc == 2 and b"static buffer holds" in L.awq_hip_last_error()
    torch.cuda.synchronize()
    assert torch.count_nonzero(y) == 0
