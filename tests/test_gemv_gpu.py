"""Kernel (b): decode-regime split-K GEMV through the C ABI against the fp32-accumulation oracle.

Tolerance (stated by the task): max|y - y_ref| / max|y_ref| <= 1e-2; the kernels are expected to be
far inside it, so a tighter bound is asserted as well to catch indexing slips that a loose bound hides."""
import numpy as np
import pytest
import torch

import nanoquantization_amd as nq
from nanoquantization_amd import _lib
from nanoquantization_amd.layers.gemm import awq_gemv_variant
from conftest import make_case, make_x, random_packed, to_bits, to_dev
from oracle import awq_oracle as o

pytestmark = pytest.mark.gpu

TOL = 1e-2
# with a bias the reference rounds twice (the product, then out.add_(bias), layers/gemm.py:561-566): one more half ulp
BIAS_STEP = {"f16": 2.0 ** -11, "bf16": 2.0 ** -8}
TIGHT = {"f16": 1.5e-3, "bf16": 6e-3}   # output rounding alone is 2^-11 / 2^-8 of the value

QWEN3_0P6B = [(1024, 2048), (1024, 1024), (2048, 1024), (1024, 3072), (3072, 1024)]


def _check(y, xb, p, dtype, bias=None):
    ref = o.linear_fp32(xb, p["qweight"], p["qzeros"], p["qscales"], dtype, bias)
    err = o.max_rel_err(o.from_bits16(to_bits(y), dtype), ref)
    assert err <= TOL, f"max rel err {err}"
    assert err <= TIGHT[dtype] + BIAS_STEP[dtype] * (bias is not None), \
        f"max rel err {err} (inside the 1e-2 bound but worse than rounding explains)"
    return err


@pytest.mark.parametrize("K,N", QWEN3_0P6B)
@pytest.mark.parametrize("M", [1, 2, 4, 8, 16])
def test_gemv_decode_sweep_f16(K, N, M):
    print(f"gemv sweep f16 M={M} K={K} N={N}", flush=True)
    p = make_case(K, N, 128, "f16", seed=K * 7 + N)
    xb = make_x(M, K, "f16", seed=M)
    y = nq.awq_gemm(to_dev(xb, "f16"), to_dev(p["qweight"]), to_dev(p["qscales"], "f16"), to_dev(p["qzeros"]), 8)
    torch.cuda.synchronize()
    assert tuple(y.shape) == (M, N) and y.dtype == torch.float16
    _check(y, xb, p, "f16")


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("K,N", [(1024, 2048), (2048, 1024)])
def test_gemv_every_row_count_step_by_step_form(dtype, K, N):
    """1..16 rows on decode-size shapes (one chunk per wave: the step-by-step form, which waits for its loads by
    count).  Between 5 and 15 rows the activation loads run under a lane mask that cuts a wave in two."""
    p = make_case(K, N, 128, dtype, seed=K + 3 * N)
    dev = [to_dev(p["qweight"]), to_dev(p["qscales"], dtype), to_dev(p["qzeros"])]
    for M in range(1, 17):
        print(f"gemv rows {dtype} M={M} K={K} N={N}", flush=True)
        xb = make_x(M, K, dtype, seed=40 + M)
        y = nq.awq_gemm(to_dev(xb, dtype), *dev, 8)
        _check(y, xb, p, dtype)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_gemv_every_variant_and_split(dtype):
    L = _lib.lib()
    K, N = 1024, 1024
    p = random_packed(K, N, 128, dtype, seed=21)
    dev = [to_dev(p["qweight"]), to_dev(p["qscales"], dtype), to_dev(p["qzeros"])]
    for M in (1, 3, 16, 24, 40):
        xb = make_x(M, K, dtype, seed=30 + M)
        xd = to_dev(xb, dtype)
        for v in range(L.awq_gemv_variant_count()):
            for split in (1, 2, 5, 32):
                print(f"gemv variant {L.awq_gemv_variant_name(v).decode()} split={split} M={M} {dtype}", flush=True)
                try:
                    y = awq_gemv_variant(xd, *dev, v, split)
                except _lib.AwqHipError as e:
                    if "does not fit the LDS" in str(e) or "takes at most" in str(e):
                        continue    # 16-wave staging variants at large M; single-m-tile variants above 16 rows
                    raise
                torch.cuda.synchronize()
                _check(y, xb, p, dtype)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("K", [1024, 2048])
def test_gemv_staged_variants_with_one_group(dtype, K):
    # group_size == K, the one size above 128 the reference admits (layers/gemm.py:7,152): every 128-row chunk
    # shares one scale/zero row; on every staged variant, row blocks (17..64 rows on the one-m-tile kernels) and
    # the shared-chunk kernel included
    L = _lib.lib()
    names = [L.awq_gemv_variant_name(i).decode() for i in range(L.awq_gemv_variant_count())]
    N, g = 512, K
    p = random_packed(K, N, g, dtype, seed=g)
    dev = [to_dev(p["qweight"]), to_dev(p["qscales"], dtype), to_dev(p["qzeros"])]
    for M in (5, 17, 64):
        xb = make_x(M, K, dtype, seed=M + g)
        xd = to_dev(xb, dtype)
        for v, name in enumerate(names):
            if not (name.startswith("dma") or name.startswith("wide")):
                continue
            for split in (1, 3):
                print(f"gemv g={g} variant {name} split={split} M={M} {dtype}", flush=True)
                try:
                    y = awq_gemv_variant(xd, *dev, v, split)
                except _lib.AwqHipError as e:
                    if "does not fit the LDS" in str(e) or "takes at most" in str(e) or "needs N %" in str(e):
                        continue
                    raise
                torch.cuda.synchronize()
                _check(y, xb, p, dtype)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("K,N,g", [(256, 8, 128), (128, 136, 32), (512, 1000, 64), (384, 2056, 128), (512, 264, 512)])
def test_gemv_ragged_shapes_and_groups(dtype, K, N, g):
    print(f"gemv ragged {dtype} K={K} N={N} g={g}", flush=True)
    p = random_packed(K, N, g, dtype, seed=K + N + g)
    for M in (1, 7, 16):
        xb = make_x(M, K, dtype, seed=M + 3)
        y = nq.awq_gemm(to_dev(xb, dtype), to_dev(p["qweight"]), to_dev(p["qscales"], dtype), to_dev(p["qzeros"]), 8)
        torch.cuda.synchronize()
        _check(y, xb, p, dtype)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M", [17, 32, 33, 48, 64])
def test_gemv_batched_decode_rows(dtype, M):
    # decode batches of 17..64 rows (Qwen3 configs 4 and 5 decode at batch 32 / 64) run on the staged GEMV
    print(f"gemv batched decode {dtype} M={M}", flush=True)
    for (K, N) in [(1024, 3072), (3072, 1024), (2048, 1024)]:
        p = make_case(K, N, 128, dtype, seed=K + N + M)
        xb = make_x(M, K, dtype, seed=M)
        y = nq.awq_gemm(to_dev(xb, dtype), to_dev(p["qweight"]), to_dev(p["qscales"], dtype), to_dev(p["qzeros"]), 8)
        torch.cuda.synchronize()
        assert tuple(y.shape) == (M, N)
        _check(y, xb, p, dtype)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M,K,N,plan", [(64, 4096, 6144, "dma1x4"), (33, 4096, 6144, "dma1x4"), (24, 8192, 5120, "dma1x4"),
                                        (17, 8192, 5120, "dma1x4"), (24, 8192, 8192, "wide2d3m2/8"),
                                        (32, 5120, 17408, "wide2d2m2/7"), (17, 12288, 4096, "wide2d3m2/16"),
                                        (64, 5120, 17408, "wide2d2m4/7"), (32, 4096, 28672, "wided2m2/4")])
def test_gemv_batched_decode_rows_large_weights(dtype, M, K, N, plan):
    # 17..64 rows, with a bias: blocks of 16 rows on the one-tile kernel, and on larger weights the shared-chunk kernel
    # (256 columns x two m-tiles with two or three staging buffers or x four m-tiles; 512 columns x two m-tiles),
    # K split, second-pass reduction
    import ctypes
    L = _lib.lib()
    names = [L.awq_gemv_variant_name(i).decode() for i in range(L.awq_gemv_variant_count())]
    v, sp = ctypes.c_int(), ctypes.c_int()
    assert L.awq_gemv_plan(M, N, K, 128, ctypes.byref(v), ctypes.byref(sp)) == 0
    assert f"{names[v.value]}/{sp.value}".startswith(plan), (names[v.value], sp.value)
    print(f"gemv {names[v.value]} {dtype} M={M} K={K} N={N}", flush=True)
    p = random_packed(K, N, 128, dtype, seed=K + N + M)
    xb = make_x(M, K, dtype, seed=M)
    bias = np.linspace(-1, 1, N).astype(np.float32)
    dev = [to_dev(p["qweight"]), to_dev(p["qscales"], dtype), to_dev(p["qzeros"])]
    from nanoquantization_amd.layers.gemm import _linear   # awq_gemm's entry point, with the bias argument
    bd = to_dev(o.to_bits16(bias, dtype), dtype)
    y = _linear("awq_linear", to_dev(xb, dtype), *dev, bd)
    torch.cuda.synchronize()
    _check(y, xb, p, dtype, o.to_dtype_f32(bias, dtype))
    assert torch.equal(y, _linear("awq_linear", to_dev(xb, dtype), *dev, bd))


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M,K,N,plan", [(1, 4096, 24576, "wide2d2m1t/5"), (5, 4096, 24576, "wide2d2m1t/5"),
                                        (9, 4096, 24576, "wided2m1/5"), (16, 4096, 24576, "wided2m1/5"),
                                        (3, 4096, 28672, "wided3m1t/4"), (16, 4096, 28672, "wided3m1/4"),
                                        (1, 12288, 8192, "wide2d3m1t/8"), (8, 12288, 8192, "wide2d3m1t/8"),
                                        (16, 5120, 20480, "wide2d3m1/3"), (2, 5120, 17408, "wide2d2m1t/7")])
def test_gemv_shared_chunk_one_m_tile(dtype, M, K, N, plan):
    """Up to 16 rows on wide, large weights: the default dispatch takes a one-m-tile form of the shared-chunk kernel
    (512 or 256 columns per workgroup; the odd byte halves hand their fragments to their partners; two or three
    staging buffers; the K splits added by the last workgroup to arrive or by a second pass).  The planned form with
    and without a bias, and every form forced with other split counts, against the oracle; run-to-run equal bits."""
    import ctypes
    L = _lib.lib()
    names = [L.awq_gemv_variant_name(i).decode() for i in range(L.awq_gemv_variant_count())]
    v, sp = ctypes.c_int(), ctypes.c_int()
    assert L.awq_gemv_plan(M, N, K, 128, ctypes.byref(v), ctypes.byref(sp)) == 0
    assert f"{names[v.value]}/{sp.value}" == plan
    print(f"gemv shared-chunk, one m-tile {dtype} M={M} K={K} N={N}", flush=True)
    p = random_packed(K, N, 128, dtype, seed=K + N + M)
    xb = make_x(M, K, dtype, seed=M)
    bias = np.linspace(-1, 1, N).astype(np.float32)
    dev = [to_dev(p["qweight"]), to_dev(p["qscales"], dtype), to_dev(p["qzeros"])]
    from nanoquantization_amd.layers.gemm import _linear
    bd = to_dev(o.to_bits16(bias, dtype), dtype)
    xd = to_dev(xb, dtype)
    y = _linear("awq_linear", xd, *dev, bd)
    _check(y, xb, p, dtype, o.to_dtype_f32(bias, dtype))
    assert torch.equal(y, _linear("awq_linear", xd, *dev, bd))
    ref = o.linear_fp32(xb, p["qweight"], p["qzeros"], p["qscales"], dtype, None)   # once: 100 M weights on the CPU

    def check_plain(yv, what):
        err = o.max_rel_err(o.from_bits16(to_bits(yv), dtype), ref)
        assert err <= TIGHT[dtype], (what, err)

    check_plain(nq.awq_gemm(xd, *dev, 8), "default")
    forms = [n for n in names if n.startswith("wide") and n.endswith(("m1", "m1t"))]
    assert len(forms) == 8, forms
    for vn in forms:
        for split in (1, 2, 8):
            yv = awq_gemv_variant(xd, *dev, names.index(vn), split)
            check_plain(yv, (vn, split))
            assert torch.equal(yv, awq_gemv_variant(xd, *dev, names.index(vn), split)), (vn, split)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M,K,N,plan", [(64, 8192, 8192, "wide2d2m4/8"), (33, 4096, 12288, "wide2d2m4/5"),
                                        (50, 5120, 17408, "wide2d2m4/7"), (48, 12288, 4096, "wide2d2m4/16")])
def test_gemv_shared_chunk_four_m_tiles(dtype, M, K, N, plan):
    """33..64 rows on 45 M weights or more: 256 columns per workgroup, four m-tiles, a chunk taken one 32-row step at
    a time.  The planned form with a bias against the oracle; forced with other split counts it must give, bit for
    bit, what the 512-column form gives (the same MFMA chains and the same fold per column), run after run."""
    import ctypes
    L = _lib.lib()
    names = [L.awq_gemv_variant_name(i).decode() for i in range(L.awq_gemv_variant_count())]
    v, sp = ctypes.c_int(), ctypes.c_int()
    assert L.awq_gemv_plan(M, N, K, 128, ctypes.byref(v), ctypes.byref(sp)) == 0
    assert f"{names[v.value]}/{sp.value}" == plan
    print(f"gemv shared-chunk, four m-tiles {dtype} M={M} K={K} N={N}", flush=True)
    p = random_packed(K, N, 128, dtype, seed=K + N + M)
    xb = make_x(M, K, dtype, seed=M)
    bias = np.linspace(-1, 1, N).astype(np.float32)
    dev = [to_dev(p["qweight"]), to_dev(p["qscales"], dtype), to_dev(p["qzeros"])]
    from nanoquantization_amd.layers.gemm import _linear
    bd = to_dev(o.to_bits16(bias, dtype), dtype)
    xd = to_dev(xb, dtype)
    y = _linear("awq_linear", xd, *dev, bd)
    _check(y, xb, p, dtype, o.to_dtype_f32(bias, dtype))
    assert torch.equal(y, _linear("awq_linear", xd, *dev, bd))
    new, old = names.index("wide2d2m4"), names.index("wided2m4")
    for split in (1, 3, sp.value, 25):
        yv = awq_gemv_variant(xd, *dev, new, split, bias=bd)
        assert torch.equal(yv, awq_gemv_variant(xd, *dev, old, split, bias=bd)), split
        assert torch.equal(yv, awq_gemv_variant(xd, *dev, new, split, bias=bd)), split
        if split == sp.value:
            assert torch.equal(yv, y)


def test_gemv_reference_test_shape():
    # the reference's own GEMM test: K=1024, N=2048, g=32, 8 tokens, atol=1.0 against x @ w_dq.T
    # (awq/tests/dequantization_kernel.py:108-138)
    print("gemv reference test shape", flush=True)
    p = make_case(1024, 2048, 32, "f16", seed=3, w_std=1.0)
    xb = make_x(8, 1024, "f16", seed=4)
    y = nq.awq_gemm(to_dev(xb, "f16"), to_dev(p["qweight"]), to_dev(p["qscales"], "f16"), to_dev(p["qzeros"]), 8)
    expect = o.from_bits16(xb, "f16").astype(np.float64) @ p["w_dq"].T.astype(np.float64)
    assert np.abs(y.float().cpu().numpy() - expect).max() <= 1.0
    _check(y, xb, p, "f16")


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_gemv_bias_linearity_and_determinism(dtype):
    print(f"gemv bias/linearity {dtype}", flush=True)
    K, N, M = 2048, 1024, 4
    p = make_case(K, N, 128, dtype, seed=40)
    dev = [to_dev(p["qweight"]), to_dev(p["qscales"], dtype), to_dev(p["qzeros"])]
    xb = make_x(M, K, dtype, seed=41)
    xd = to_dev(xb, dtype)
    bias = np.linspace(-2, 2, N).astype(np.float32)
    bias16 = o.to_dtype_f32(bias, dtype)
    for split in (1, 4):
        y = awq_gemv_variant(xd, *dev, 0, split, bias=to_dev(o.to_bits16(bias, dtype), dtype))
        _check(y, xb, p, dtype, bias16)
    # bit-stable run to run (fixed reduction order)
    y1 = awq_gemv_variant(xd, *dev, 0, 8)
    y2 = awq_gemv_variant(xd, *dev, 0, 8)
    assert torch.equal(y1, y2)
    # x = 0 -> exactly 0; scaling x by 2 scales y by exactly 2 (power of two commutes with every rounding)
    assert torch.count_nonzero(awq_gemv_variant(torch.zeros_like(xd), *dev, 0, 8)) == 0
    assert torch.equal(awq_gemv_variant(xd * 2, *dev, 0, 8), y1 * 2)


def test_gemv_large_streaming_shape():
    # Qwen3-32B MLP shape at its real size: property checks (too big for the scalar oracle; the numpy one is fine)
    print("gemv large 5120x25600 f16", flush=True)
    K, N = 5120, 25600
    p = random_packed(K, N, 128, "f16", seed=50)
    xb = make_x(16, K, "f16", seed=51)
    y = nq.awq_gemm(to_dev(xb, "f16"), to_dev(p["qweight"]), to_dev(p["qscales"], "f16"), to_dev(p["qzeros"]), 8)
    _check(y, xb, p, "f16")


def test_gemv_errors():
    p = random_packed(256, 64, 128, "f16")
    dev = [to_dev(p["qweight"]), to_dev(p["qscales"], "f16"), to_dev(p["qzeros"])]
    x = torch.zeros(17, 256, dtype=torch.float16, device="cuda")
    with pytest.raises(_lib.AwqHipError, match="takes at most 16 rows"):
        awq_gemv_variant(x, *dev, 0, 1)
    with pytest.raises(_lib.AwqHipError, match="decode regime"):
        awq_gemv_variant(torch.zeros(129, 256, dtype=torch.float16, device="cuda"), *dev, 0, 1)
    with pytest.raises(AssertionError):
        nq.awq_gemm(x[:, :128], *dev, 8)
    with pytest.raises(AssertionError):
        nq.awq_gemm(x, *dev, 6)       # split_k_iters must be a power of two, as in the reference


def test_prefetch_hint_never_changes_results():
    """A pending hint adds workgroups that only read the hinted region; y must stay bit-identical, with and
    without K splits, and the hint must be gone after one launch."""
    import ctypes
    L = _lib.lib()
    for (M, K, N) in ((1, 1024, 1024), (16, 1024, 3072), (4, 2048, 1024), (32, 3072, 1024), (1, 5120, 25600)):
        p = random_packed(K, N, 128, "f16", seed=K + N)
        dev = [to_dev(p["qweight"]), to_dev(p["qscales"], "f16"), to_dev(p["qzeros"])]
        xd = to_dev(make_x(M, K, "f16", seed=M), "f16")
        other = torch.randint(-2 ** 31, 2 ** 31 - 1, (2048, 384), dtype=torch.int32, device="cuda")
        print(f"prefetch hint M={M} K={K} N={N}", flush=True)
        ref = nq.awq_gemm(xd, *dev, 8)
        nq.prefetch_hint(other, dev[1], dev[2])
        got = nq.awq_gemm(xd, *dev, 8)
        assert L.awq_prefetch_pending() == 0       # the hint was consumed
        again = nq.awq_gemm(xd, *dev, 8)
        torch.cuda.synchronize()
        assert torch.equal(got, ref) and torch.equal(again, ref)
    assert L.awq_prefetch_hint(ctypes.c_void_p(64), 1024) == 1      # not 128-byte aligned
    assert L.awq_prefetch_hint(None, 0) == 0
    buf = torch.zeros(1024, dtype=torch.uint8, device="cuda")
    for _ in range(4):
        assert L.awq_prefetch_hint(buf.data_ptr(), 1024) == 0
    assert L.awq_prefetch_hint(buf.data_ptr(), 1024) == 0           # a fifth region is ignored, not an error
    assert L.awq_prefetch_pending() == 4
    assert L.awq_prefetch_hint(None, 0) == 0 and L.awq_prefetch_pending() == 0


@pytest.mark.parametrize("dt", ["f16", "bf16"])
def test_gemv_row_blocks_up_to_128_rows(dt):
    """65..128 rows as blocks of 16 rows of the one-tile staged kernels (what awq_linear runs on small weights), with
    and without a K split and a bias, against the fp32 oracle; a ragged last block included."""
    tdt = torch.float16 if dt == "f16" else torch.bfloat16
    for (M, K, N, variant, split) in [(65, 512, 384, 2, 1), (100, 1024, 1024, 3, 1), (128, 2048, 1024, 2, 2),
                                      (127, 1024, 3072, 3, 1)]:
        print(f"row blocks {dt} M={M} K={K} N={N} variant={variant} split={split}", flush=True)
        p = random_packed(K, N, 128, dt, seed=M)
        xb = make_x(M, K, dt, seed=M + 1)
        dev = [to_dev(p["qweight"]), to_dev(p["qscales"], dt), to_dev(p["qzeros"])]
        y = awq_gemv_variant(to_dev(xb, dt), *dev, variant, split)
        _check(y, xb, p, dt)
        assert torch.equal(y, awq_gemv_variant(to_dev(xb, dt), *dev, variant, split))
        yd = nq.awq_gemm(to_dev(xb, dt), *dev, 8)          # the default dispatch takes the same route
        _check(yd, xb, p, dt)


def test_gemv_splitk_exchange_endurance():
    """About 670 launches cycling four split-K problems (1, 16 and 32 rows on the one-tile kernels, 2 rows on the
    shared-chunk kernel's in-kernel tail) back to back on one stream, sharing one workspace: the cross-workgroup
    exchange of partials (write-through stores, arrival counter, last arriver adds in split order, counter left at
    zero) must give the bits of the first launch every time.  Stops at the first mismatch."""
    import ctypes
    L = _lib.lib()
    names = [L.awq_gemv_variant_name(i).decode() for i in range(L.awq_gemv_variant_count())]
    cases = []
    for (M, K, N, dtype) in ((1, 2048, 1024, "f16"), (16, 4096, 4096, "bf16"), (32, 3072, 1024, "f16"),
                             (2, 4096, 24576, "bf16")):
        v, sp = ctypes.c_int(), ctypes.c_int()
        assert L.awq_gemv_plan(M, N, K, 128, ctypes.byref(v), ctypes.byref(sp)) == 0
        assert sp.value > 1 and names[v.value].endswith("m1t") == (N == 24576), (M, K, N, names[v.value], sp.value)
        gen = torch.Generator(device="cuda").manual_seed(M + K)
        tdt = torch.float16 if dtype == "f16" else torch.bfloat16
        qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (K, N // 8), dtype=torch.int32, device="cuda", generator=gen)
        qz = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 128, N // 8), dtype=torch.int32, device="cuda", generator=gen)
        qs = (torch.rand(K // 128, N, device="cuda", generator=gen) * 0.02 + 0.001).to(tdt)
        x = torch.randn(M, K, device="cuda", generator=gen).to(tdt)
        cases.append((M, K, N, _lib.dtype_id(tdt), x, qw, qs, qz, torch.empty(M, N, dtype=tdt, device="cuda")))
    nbytes = max(L.awq_gemv_workspace_bytes(M, N, K) for (M, K, N, *_rest) in cases)
    ws = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    stream = _lib.current_stream_ptr(ws.device)

    def launch(c):
        M, K, N, did, x, qw, qs, qz, y = c
        _lib.check(L.awq_gemv(x.data_ptr(), qw.data_ptr(), qs.data_ptr(), qz.data_ptr(), None, y.data_ptr(), M, N, K, 128,
                              did, ws.data_ptr(), ws.numel(), stream))
    first = []
    for c in cases:
        launch(c)
        first.append(c[-1].clone())
    print("gemv split-K endurance: 168 rounds of 4 launches", flush=True)
    for rnd in range(168):
        for c in cases:
            c[-1].fill_(float("nan"))
        for c in cases:      # launches back to back: the second starts while the first's tail may still run
            launch(c)
        for i, c in enumerate(cases):
            assert torch.equal(c[-1], first[i]), f"round {rnd}: launch {i} (M={c[0]} K={c[1]} N={c[2]}) changed bits"
    # every arrival counter is back at zero (the first 16 KiB of the workspace)
    assert torch.count_nonzero(ws[:16384]) == 0
