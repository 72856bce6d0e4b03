"""Kernel (c): fused dequant + MFMA GEMM through the C ABI against the fp32-accumulation oracle."""
import numpy as np
import pytest
import torch

import nanoquantization_amd as nq
from nanoquantization_amd import _lib
from nanoquantization_amd.layers.gemm import awq_gemm_variant
from conftest import make_case, make_x, random_packed, to_bits, to_dev
from oracle import awq_oracle as o

pytestmark = pytest.mark.gpu

TOL = 1e-2
# with a bias the reference rounds twice (the product, then out.add_(bias), layers/gemm.py:561-566): one more half ulp
BIAS_STEP = {"f16": 2.0 ** -11, "bf16": 2.0 ** -8}
TIGHT = {"f16": 1.5e-3, "bf16": 6e-3}


def _check(y, xb, p, dtype, bias=None):
    ref = o.linear_fp32(xb, p["qweight"], p["qzeros"], p["qscales"], dtype, bias)
    err = o.max_rel_err(o.from_bits16(to_bits(y), dtype), ref)
    assert err <= TOL, f"max rel err {err}"
    assert err <= TIGHT[dtype] + BIAS_STEP[dtype] * (bias is not None), f"max rel err {err}"
    return err


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_gemm_every_variant_and_split(dtype):
    L = _lib.lib()
    K, N = 512, 520            # N not a multiple of any tile: exercises the column masks
    p = random_packed(K, N, 128, dtype, seed=60)
    dev = [to_dev(p["qweight"]), to_dev(p["qscales"], dtype), to_dev(p["qzeros"])]
    for M in (17, 128, 300):
        xb = make_x(M, K, dtype, seed=61 + M)
        xd = to_dev(xb, dtype)
        for v in range(L.awq_gemm_variant_count()):
            for split in (1, 3):
                print(f"gemm variant {L.awq_gemm_variant_name(v).decode()} split={split} M={M} {dtype}", flush=True)
                y = awq_gemm_variant(xd, *dev, v, split)
                torch.cuda.synchronize()
                _check(y, xb, p, dtype)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M,K,N,g", [(32, 1024, 3072, 128), (64, 3072, 1024, 128), (256, 1024, 2048, 32),
                                      (512, 4096, 1024, 128), (130, 256, 8, 64), (1000, 2048, 264, 128)])
def test_gemm_default_dispatch(dtype, M, K, N, g):
    print(f"gemm default {dtype} M={M} K={K} N={N} g={g}", flush=True)
    p = make_case(K, N, g, dtype, seed=M + K)
    xb = make_x(M, K, dtype, seed=M)
    y = nq.awq_gemm(to_dev(xb, dtype), to_dev(p["qweight"]), to_dev(p["qscales"], dtype), to_dev(p["qzeros"]), 8)
    torch.cuda.synchronize()
    assert tuple(y.shape) == (M, N)
    _check(y, xb, p, dtype)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_gemm_equals_dequant_then_matmul(dtype):
    # the reference's M >= 256 branch: awq_dequantize + torch.matmul (layers/gemm.py:559-561); the fused
    # kernel multiplies the very same rounded weights, so it must agree with that path to fp32-sum accuracy
    print(f"gemm vs dequant+matmul {dtype}", flush=True)
    M, K, N = 384, 1024, 1024
    p = make_case(K, N, 128, dtype, seed=70)
    xb = make_x(M, K, dtype, seed=71)
    qw, qs, qz = to_dev(p["qweight"]), to_dev(p["qscales"], dtype), to_dev(p["qzeros"])
    xd = to_dev(xb, dtype)
    w = nq.awq_dequantize(qw, qs, qz)
    y_unfused = torch.matmul(xd.float(), w.float())
    y = nq.awq_gemm(xd, qw, qs, qz, 8)
    err = (y.float() - y_unfused).abs().max().item() / y_unfused.abs().max().item()
    assert err <= (1e-3 if dtype == "f16" else 5e-3), err


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_gemm_bias_and_determinism(dtype):
    print(f"gemm bias {dtype}", flush=True)
    M, K, N = 200, 1024, 512
    p = make_case(K, N, 128, dtype, seed=80)
    dev = [to_dev(p["qweight"]), to_dev(p["qscales"], dtype), to_dev(p["qzeros"])]
    xb = make_x(M, K, dtype, seed=81)
    xd = to_dev(xb, dtype)
    bias = np.linspace(-2, 2, N).astype(np.float32)
    v = 0   # the 128 x 128 tile
    for split in (1, 4):
        y = awq_gemm_variant(xd, *dev, v, split, bias=to_dev(o.to_bits16(bias, dtype), dtype))
        _check(y, xb, p, dtype, o.to_dtype_f32(bias, dtype))
    y1 = awq_gemm_variant(xd, *dev, v, 4)
    y2 = awq_gemm_variant(xd, *dev, v, 4)
    assert torch.equal(y1, y2)
    assert torch.count_nonzero(awq_gemm_variant(torch.zeros_like(xd), *dev, v, 4)) == 0


@pytest.mark.parametrize("form", ["p", "r"])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_gemm_tail_tiles_split(dtype, form):
    # 9 x 30 = 270 tiles of 256 x 256 (ragged in M and N): 256 whole tiles and a tail of 14 whose K range is cut;
    # the mixed launch must agree with the oracle, with the uncut launch bit for bit where no cut applies,
    # and be bit-stable -- for the pipelined kernel (p) and the one that builds its B operands in registers (r)
    L = _lib.lib()
    names = [L.awq_gemm_variant_name(i).decode() for i in range(L.awq_gemm_variant_count())]
    tail, whole = names.index(f"256x256{form}t"), names.index(f"256x256{form}")
    # (the register-operand kernel takes widths that are multiples of 128; other widths run the pipelined one under
    # its name: its case has the last tile half empty instead of ragged)
    M, K, N = 2300, 256, (7672 if form == "p" else 7552)
    p = random_packed(K, N, 128, dtype, seed=95)
    dev = [to_dev(p["qweight"]), to_dev(p["qscales"], dtype), to_dev(p["qzeros"])]
    xb = make_x(M, K, dtype, seed=96)
    xd = to_dev(xb, dtype)
    bias = np.linspace(-1, 1, N).astype(np.float32)
    bd = to_dev(o.to_bits16(bias, dtype), dtype)
    y1 = awq_gemm_variant(xd, *dev, whole, 1, bias=bd)
    _check(y1, xb, p, dtype, o.to_dtype_f32(bias, dtype))
    for split in (2, 4):
        print(f"gemm tail {form} split={split} {dtype}", flush=True)
        y = awq_gemm_variant(xd, *dev, tail, split, bias=bd)
        torch.cuda.synchronize()
        _check(y, xb, p, dtype, o.to_dtype_f32(bias, dtype))
        assert torch.equal(y, awq_gemm_variant(xd, *dev, tail, split, bias=bd))
        # tiles 0..255 in n-fastest order: tile rows 0..7 entirely (8 x 30 = 240) and 16 tiles of row 8
        assert torch.equal(y[:2048], y1[:2048])
        assert torch.equal(y[2048:, :16 * 256], y1[2048:, :16 * 256])


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("K,N,g", [(1024, 1032, 128), (256, 8, 64), (512, 264, 32), (128, 4096, 128), (1024, 520, 1024)])
def test_dequantize_transposed_bit_exact(dtype, K, N, g):
    # out [N, K] must be awq_dequantize's [K, N] transposed, bit for bit (and so the oracle's RN((q - z) * s))
    print(f"dequantize transposed {dtype} K={K} N={N} g={g}", flush=True)
    p = random_packed(K, N, g, dtype, seed=K + N + g)
    dev = [to_dev(p["qweight"]), to_dev(p["qscales"], dtype), to_dev(p["qzeros"])]
    wt = nq.awq_dequantize_transposed(*dev)
    assert tuple(wt.shape) == (N, K)
    assert torch.equal(wt, nq.awq_dequantize(*dev).t())
    ref_bits = o.dequant(p["qweight"], p["qzeros"], p["qscales"], dtype)
    assert np.array_equal(to_bits(wt).T, ref_bits)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M,K,N,g", [(1024, 1024, 1032, 128), (1500, 512, 2048, 64), (2048, 256, 264, 32)])
def test_linear_large_m_equals_dequantise_then_matmul(dtype, M, K, N, g):
    # 1024 rows and more, the regime of the reference's awq_dequantize + torch.matmul (layers/gemm.py:558-561): the
    # default dispatch (fused kernel) against the fp32 oracle, with and without bias, against the forced whole-tile
    # variant, and against that two-step structure built from awq_dequantize_transposed + a dense matmul
    from nanoquantization_amd.layers.gemm import _linear
    print(f"large-M linear {dtype} M={M} K={K} N={N} g={g}", flush=True)
    p = make_case(K, N, g, dtype, seed=M + N)
    xb = make_x(M, K, dtype, seed=M)
    dev = [to_dev(p["qweight"]), to_dev(p["qscales"], dtype), to_dev(p["qzeros"])]
    xd = to_dev(xb, dtype)
    y = nq.awq_gemm(xd, *dev, 8)
    _check(y, xb, p, dtype)
    bias = np.linspace(-1, 1, N).astype(np.float32)
    yb = _linear("awq_linear", xd, *dev, to_dev(o.to_bits16(bias, dtype), dtype))
    _check(yb, xb, p, dtype, o.to_dtype_f32(bias, dtype))
    L = _lib.lib()
    names = [L.awq_gemm_variant_name(i).decode() for i in range(L.awq_gemm_variant_count())]
    fused = awq_gemm_variant(xd, *dev, names.index("256x256p"), 1)
    fused_r = awq_gemm_variant(xd, *dev, names.index("256x256r"), 1)
    two_step = torch.matmul(xd, nq.awq_dequantize_transposed(*dev).t())
    for other in (fused, fused_r, two_step):
        err = (y.float() - other.float()).abs().max().item() / other.float().abs().max().item()
        assert err <= (2e-3 if dtype == "f16" else 1.6e-2), err     # both round an fp32 sum of the same products once


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M,K,N,g,split", [(300, 1024, 520, 128, 1), (777, 2048, 1032, 64, 3), (256, 64, 256, 64, 1),
                                            (1000, 768, 2048, 768, 2), (513, 512, 264, 32, 1)])
def test_gemm_register_b_kernel_equals_pipelined(dtype, M, K, N, g, split):
    # the two 256 x 256 kernels multiply the same rounded weights (on MFMAs of different depth, so the fp32 sums may
    # differ in their last bits): ragged M and N, K of one step, odd K slices, every group size (g = 32 runs the
    # pipelined kernel under the r names, bit for bit), with bias
    print(f"gemm r vs p {dtype} M={M} K={K} N={N} g={g} split={split}", flush=True)
    L = _lib.lib()
    names = [L.awq_gemm_variant_name(i).decode() for i in range(L.awq_gemm_variant_count())]
    p = random_packed(K, N, g, dtype, seed=K + N + g)
    dev = [to_dev(p["qweight"]), to_dev(p["qscales"], dtype), to_dev(p["qzeros"])]
    xb = make_x(M, K, dtype, seed=M)
    xd = to_dev(xb, dtype)
    bias = np.linspace(-1, 1, N).astype(np.float32)
    bd = to_dev(o.to_bits16(bias, dtype), dtype)
    for form in ("", "t"):
        yp = awq_gemm_variant(xd, *dev, names.index("256x256p" + form), split, bias=bd)
        yr = awq_gemm_variant(xd, *dev, names.index("256x256r" + form), split, bias=bd)
        torch.cuda.synchronize()
        if g % 64 != 0:
            assert torch.equal(yp, yr), form
        diff = (yp.float() - yr.float()).abs().max().item() / yp.float().abs().max().item()
        assert diff <= (1e-3 if dtype == "f16" else 8e-3), (form, diff)
        _check(yr, xb, p, dtype, o.to_dtype_f32(bias, dtype))


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M,K,N", [(4096, 512, 4352), (4096, 1024, 4096), (2048, 1024, 4096), (4096, 4096, 4096),
                                   (1024, 1024, 4096)])
def test_gemm_default_kernel_by_work_items(dtype, M, K, N):
    # The default entry point runs the register-operand kernel (r) where the plan's work items -- whole tiles plus the
    # K slices of the tail tiles -- outnumber the 256 CUs (16 x 17 = 272 tiles); at exactly 256 items (16 x 16 tiles, or
    # 8 x 16 cut in two) in fp16, and in bf16 if an item has 64 K steps at least; the pipelined kernel (p) otherwise
    # (4 x 16 tiles cut in two).  awq_gemm_plan names that kernel, and forcing the planned pair gives the same bits.
    import ctypes
    L = _lib.lib()
    names = [L.awq_gemm_variant_name(i).decode() for i in range(L.awq_gemm_variant_count())]
    v, sp = ctypes.c_int(), ctypes.c_int()
    dt = _lib.AWQ_F16 if dtype == "f16" else _lib.AWQ_BF16
    assert L.awq_gemm_plan(M, N, K, 128, dt, ctypes.byref(v), ctypes.byref(sp)) == 0
    name = names[v.value]
    tiles = (M // 256) * (N // 256)
    tail = tiles % 256 if name.endswith("t") else (tiles if sp.value > 1 else 0)
    items = tiles - tail + tail * sp.value
    print(f"gemm default {dtype} M={M} K={K} N={N}: plan {name} split {sp.value}, {items} items", flush=True)
    steps = K // 64 // (sp.value if tail == tiles else 1)
    use_r = items > 256 or (items == 256 and (dtype == "f16" or steps >= 64))
    assert name in (("256x256r", "256x256rt") if use_r else ("256x256p", "256x256pt")), (name, items, steps)
    p = random_packed(K, N, 128, dtype, seed=123)
    dev = [to_dev(p["qweight"]), to_dev(p["qscales"], dtype), to_dev(p["qzeros"])]
    xd = to_dev(make_x(M, K, dtype, seed=124), dtype)
    y = nq.awq_gemm(xd, *dev, 8)
    assert torch.equal(y, awq_gemm_variant(xd, *dev, v.value, sp.value)), name
    rows = torch.arange(0, M, 97, device="cuda")
    ref = xd[rows].float() @ nq.awq_dequantize(*dev).float()
    assert ((y[rows].float() - ref).abs().max() / ref.abs().max()).item() <= TIGHT[dtype]


def test_gemm_prefill_full_size_bf16():
    # Qwen3-8B MLP gate/up at M=512, its real size (oracle: numpy float64 matmul, a few seconds)
    print("gemm full size M=512 4096x12288 bf16", flush=True)
    M, K, N = 512, 4096, 12288
    p = random_packed(K, N, 128, "bf16", seed=90)
    xb = make_x(M, K, "bf16", seed=91)
    y = nq.awq_gemm(to_dev(xb, "bf16"), to_dev(p["qweight"]), to_dev(p["qscales"], "bf16"), to_dev(p["qzeros"]), 8)
    _check(y, xb, p, "bf16")


@pytest.mark.parametrize("M,K,N", [(8192, 4096, 12288), (8192, 12288, 4096), (2048, 4096, 12288), (2048, 12288, 4096),
                                   (512, 12288, 4096), (4096, 8192, 5120), (300, 5120, 25600)])
def test_gemm_largest_shapes_properties(M, K, N):
    """The prefill shapes at their real sizes (Qwen3-8B MLP at M = 512 / 2048 / 8192, Qwen3-32B o_proj at a 4096-token
    prefill and gate/up at a ragged M), too big for the CPU oracle: checked through size-independent properties, on
    the default dispatch and on both 256 x 256 fused kernels (the pipelined one, p, and the one that builds its B
    operands in registers, r) forced in both of their forms (every tile whole; the tiles of the last round cut along K
    with the plan's split).  (1) rows sampled across every workgroup tile equal the
    fp32 matmul of those rows with the dequantised weight (itself bit-exact against the oracle); (2) the same rows
    pushed through alone (another tile shape) agree too; (3) run-to-run bit-stable; (4) a zero row gives exact zeros."""
    print(f"gemm properties M={M} K={K} N={N} bf16", flush=True)
    L = _lib.lib()
    names = [L.awq_gemm_variant_name(i).decode() for i in range(L.awq_gemm_variant_count())]
    import ctypes
    v, sp = ctypes.c_int(), ctypes.c_int()
    assert L.awq_gemm_plan(M, N, K, 128, _lib.AWQ_BF16, ctypes.byref(v), ctypes.byref(sp)) == 0
    g = torch.Generator(device="cuda").manual_seed(M + K)
    qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (K, N // 8), dtype=torch.int32, device="cuda", generator=g)
    qz = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 128, N // 8), dtype=torch.int32, device="cuda", generator=g)
    sc = (torch.rand(K // 128, N, device="cuda", generator=g) * 0.01 + 0.002).to(torch.bfloat16)
    x = torch.randn(M, K, device="cuda", generator=g).to(torch.bfloat16)
    x[5] = 0
    rows = torch.arange(3, M, max(1, M // 61), device="cuda")[:64]          # one or two rows of every 256-row tile
    w = nq.awq_dequantize(qw, sc, qz).float()
    ref = x[rows].float() @ w
    runs = [("default " + names[v.value] + f" split {sp.value}", lambda: nq.awq_gemm(x, qw, sc, qz, 8)),
            ("256x256p split 1", lambda: awq_gemm_variant(x, qw, sc, qz, names.index("256x256p"), 1)),
            (f"256x256pt split {max(sp.value, 2)}",
             lambda: awq_gemm_variant(x, qw, sc, qz, names.index("256x256pt"), max(sp.value, 2))),
            ("256x256r split 1", lambda: awq_gemm_variant(x, qw, sc, qz, names.index("256x256r"), 1)),
            (f"256x256rt split {max(sp.value, 2)}",
             lambda: awq_gemm_variant(x, qw, sc, qz, names.index("256x256rt"), max(sp.value, 2)))]
    for what, run in runs:
        print(f"  {what}", flush=True)
        y = run()
        torch.cuda.synchronize()
        assert torch.equal(y, run()), what
        assert torch.count_nonzero(y[5]) == 0, what
        err = ((y[rows].float() - ref).abs().max() / ref.abs().max()).item()
        assert err <= TIGHT["bf16"], (what, err)
        del y
    sub = nq.awq_gemm(x[rows].contiguous(), qw, sc, qz, 8).float()          # another kernel / tile shape
    assert ((sub - ref).abs().max() / ref.abs().max()).item() <= TIGHT["bf16"]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M,K,N,g", [(48, 288, 512, 32), (200, 224, 384, 32), (65, 544, 1280, 32), (32, 32, 256, 32)])
def test_linear_k_not_a_multiple_of_64(dtype, M, K, N, g):
    """K = 32 * odd (the reference admits any multiple of its 32-row K block) above 16 rows: awq_linear serves it
    with the GEMV, 16 rows at a time."""
    from nanoquantization_amd.layers import gemm as gemm_layer
    print(f"linear K%64!=0 M={M} K={K} N={N} g={g} {dtype}", flush=True)
    p = make_case(K, N, g, dtype, seed=M + K)
    xb = make_x(M, K, dtype, seed=M)
    bias = np.random.default_rng(M).standard_normal(N).astype(np.float32)
    bias_bits = o.to_bits16(bias, dtype)
    y = gemm_layer._linear("awq_linear", to_dev(xb, dtype), to_dev(p["qweight"]), to_dev(p["qscales"], dtype),
                           to_dev(p["qzeros"]), to_dev(bias_bits, dtype))
    _check(y, xb, p, dtype, o.from_bits16(bias_bits, dtype))


def test_linear_random_shapes_default_dispatch():
    """Seeded sweep over odd shape combinations (row counts either side of every dispatch boundary, K = group x small
    and large factors, N with and without whole 128-column tiles, three group sizes, optional bias): whatever kernel
    the default dispatch picks must meet the tight error bound and be bit-stable run to run."""
    import random
    from nanoquantization_amd.layers import gemm as gemm_layer
    rnd = random.Random(1234)
    cases = 0
    while cases < 60:
        tdt = rnd.choice([torch.float16, torch.bfloat16])
        g = rnd.choice([128, 128, 128, 64, 32])
        K = g * rnd.choice([1, 2, 3, 4, 5, 7, 8, 9, 12, 16, 17, 24, 31, 32, 40, 48, 64, 100])
        N = 8 * rnd.choice([1, 3, 16, 17, 32, 48, 64, 96, 128, 136, 160, 256, 272, 384, 512, 640, 1000, 1024, 1280])
        M = rnd.choice([1, 2, 3, 4, 5, 7, 8, 15, 16, 17, 24, 31, 32, 33, 48, 63, 64, 65, 100, 128, 129, 200, 256, 300, 1024, 1100])
        if K % 32 or K * N * max(M, 64) > 2e10:
            continue
        cases += 1
        gen = torch.Generator(device="cuda").manual_seed(cases)
        qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (K, N // 8), dtype=torch.int32, device="cuda", generator=gen)
        qz = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // g, N // 8), dtype=torch.int32, device="cuda", generator=gen)
        qs = (torch.rand(K // g, N, device="cuda", generator=gen) * 0.02 + 0.001).to(tdt)
        x = torch.randn(M, K, device="cuda", generator=gen).to(tdt)
        bias = torch.randn(N, device="cuda", generator=gen).to(tdt) if rnd.random() < 0.3 else None
        print(f"random linear {cases}: M={M} K={K} N={N} g={g} {tdt} bias={bias is not None}", flush=True)
        y = gemm_layer._linear("awq_linear", x, qw, qs, qz, bias)
        ref = x.float() @ nq.awq_dequantize(qw, qs, qz).float()
        if bias is not None:
            ref = ref + bias.float()
        err = ((y.float() - ref).abs().max() / ref.abs().max().clamp_min(1e-6)).item()
        assert err <= (1.5e-3 if tdt == torch.float16 else 6e-3), err
        assert torch.equal(y, gemm_layer._linear("awq_linear", x, qw, qs, qz, bias))
