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
    torch.cuda.synchronize()
    # the driver's own count of free device memory sees an allocation by anyone (torch's counter would only see
    # torch's); the first call on a device has looked up the scratch address already (_warm)
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    _lib.check(L.awq_gemv_static(x.data_ptr(), qw.data_ptr(), qs.data_ptr(), qz.data_ptr(), b, got.data_ptr(), M, N, K,
                                 128, did, stream))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before and torch.cuda.mem_get_info()[0] == free_before
    return got, want, nbytes


def _warm(L):
    """One split-K call, so that the once-per-device set-up (the address of the static array) is behind us."""
    x, qw, qs, qz, _ = _case(1, 2048, 1024, torch.float16, 1)
    y = torch.empty(1, 1024, dtype=torch.float16, device="cuda")
    _lib.check(L.awq_gemv_static(x.data_ptr(), qw.data_ptr(), qs.data_ptr(), qz.data_ptr(), None, y.data_ptr(), 1, 1024,
                                 2048, 128, _lib.AWQ_F16, _lib.current_stream_ptr(x.device)))
    torch.cuda.synchronize()


def test_gemv_static_equals_gemv_on_two_calls_in_a_row():
    L = _lib.lib()
    cap = L.awq_gemv_static_scratch_bytes()
    assert cap == (16 << 10) + (16 << 20)
    _warm(L)
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


def test_gemv_static_under_graph_capture():
    """After one warm call the entry point can be recorded into a HIP graph (nothing in it allocates or asks the
    runtime for anything a capture forbids); every replay gives awq_gemv's bits, with eager work in between."""
    L = _lib.lib()
    _warm(L)
    M, K, N, dtype = 4, 2048, 1024, torch.float16           # split over K: the static scratch is in use
    x, qw, qs, qz, _ = _case(M, K, N, dtype, 11)
    did = _lib.dtype_id(dtype)
    ws = torch.zeros(max(L.awq_gemv_workspace_bytes(M, N, K), 16), dtype=torch.uint8, device="cuda")
    want = torch.empty(M, N, dtype=dtype, device="cuda")
    _lib.check(L.awq_gemv(x.data_ptr(), qw.data_ptr(), qs.data_ptr(), qz.data_ptr(), None, want.data_ptr(), M, N, K, 128,
                          did, ws.data_ptr(), ws.numel(), _lib.current_stream_ptr(x.device)))
    got = torch.zeros(M, N, dtype=dtype, device="cuda")
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            _lib.check(L.awq_gemv_static(x.data_ptr(), qw.data_ptr(), qs.data_ptr(), qz.data_ptr(), None, got.data_ptr(),
                                         M, N, K, 128, did, _lib.current_stream_ptr(x.device)))
    torch.cuda.synchronize()
    for rep in range(4):
        got.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {rep}"
        # eager work of the same kind between the replays (shares the static scratch, in stream order)
        eager = torch.empty(M, N, dtype=dtype, device="cuda")
        _lib.check(L.awq_gemv_static(x.data_ptr(), qw.data_ptr(), qs.data_ptr(), qz.data_ptr(), None, eager.data_ptr(),
                                     M, N, K, 128, did, _lib.current_stream_ptr(x.device)))
        torch.cuda.synchronize()
        assert torch.equal(eager, want)
