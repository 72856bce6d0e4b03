"""Pins the CPU oracle (oracle/) without the reference: known-answer words derived by hand from the
packing rule, closed forms, brute force on small inputs, library conversions, and the independent
plain-C restatement."""
import numpy as np
import pytest
import torch

from oracle import awq_oracle as o
from oracle import c_oracle as c


# ---- pack / unpack ---------------------------------------------------------------------------
def _word(vals):
    return int(o.pack_awq(np.array([vals], dtype=np.int32))[0, 0])


def test_pack_known_answer_words():
    # nibble j <- column [0,2,4,6,1,3,5,7][j]  (layers/gemm.py:504-519)
    assert _word(list(range(8))) == 0x75316420 == 1966171168
    assert _word(list(range(8, 16))) == -38146904            # 0xFDB9ECA8 as int32
    assert _word([15] * 8) == -1
    assert _word([0, 1, 0, 0, 0, 0, 0, 0]) == 0x00010000       # column 1 -> nibble 4
    assert _word([0, 0, 0, 0, 0, 0, 0, 1]) == 0x10000000       # column 7 -> nibble 7
    assert _word([0, 0, 0, 0, 0, 0, 0, 8]) == -(2 ** 31)       # sign bit


def test_pack_matches_nibble_by_nibble_python():
    rng = np.random.default_rng(3)
    iw = rng.integers(0, 16, size=(5, 24))
    expect = np.zeros((5, 3), dtype=np.int64)
    order = [0, 2, 4, 6, 1, 3, 5, 7]
    for r in range(5):
        for i in range(3):
            w = 0
            for j in range(8):
                w |= int(iw[r, 8 * i + order[j]]) << (4 * j)
            expect[r, i] = w - (1 << 32) if w >= (1 << 31) else w
    assert (o.pack_awq(iw) == expect).all()


def test_unpack_every_value_at_every_position():
    for col in range(8):
        for val in range(16):
            v = [0] * 8
            v[col] = val
            packed = o.pack_awq(np.array([v], dtype=np.int32))
            assert (o.unpack_awq(packed)[0] == v).all()
            # shift table of layers/gemm.py:52-69
            assert ((int(packed.view(np.uint32)[0, 0]) >> o.AWQ_SHIFT[col]) & 0xF) == val


def test_pack_unpack_roundtrip_and_c_restatement():
    rng = np.random.default_rng(4)
    iw = rng.integers(0, 16, size=(64, 256), dtype=np.int32)
    p = o.pack_awq(iw)
    assert p.dtype == np.int32 and p.shape == (64, 32)
    assert (o.unpack_awq(p) == iw).all()
    assert (c.pack(iw) == p).all()
    assert (c.unpack(p) == iw).all()


def test_pair_trick_identity():
    # (word >> 4i) & 0x000F000F == col 2i | col (2i+1) << 16 -- the identity the kernels rely on
    rng = np.random.default_rng(5)
    iw = rng.integers(0, 16, size=(16, 8), dtype=np.int32)
    w = o.pack_awq(iw).view(np.uint32)[:, 0]
    for i in range(4):
        assert (((w >> np.uint32(4 * i)) & np.uint32(0x000F000F)) == (iw[:, 2 * i] | (iw[:, 2 * i + 1] << 16))).all()


# ---- 16-bit float helpers ----------------------------------------------------------------------
def test_bf16_conversion_matches_torch():
    rng = np.random.default_rng(6)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * 10.0 ** rng.integers(-30, 30, 20000),
                        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, 1e-40, -1e-40], np.float32)])
    x = x.astype(np.float32)   # one rounding only: the helpers take fp32
    t = torch.from_numpy(x).to(torch.bfloat16)
    expect = t.view(torch.int16).numpy().view(np.uint16)
    assert (o.f32_to_bf16_bits(x) == expect).all()
    assert (o.bf16_bits_to_f32(expect) == t.float().numpy()).all()


def test_c_f16_conversion_matches_numpy():
    rng = np.random.default_rng(7)
    x = np.concatenate([rng.standard_normal(50000).astype(np.float32) * 10.0 ** rng.integers(-9, 5, 50000),
                        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e6, 6.1e-5, 6.0e-8, 2.98e-8, 2.99e-8, 1e-9],
                                 np.float32)])
    x = x.astype(np.float32)
    bits, back = c.f16_roundtrip(x)
    h = x.astype(np.float16)
    assert (bits == h.view(np.uint16)).all()
    assert (back == h.astype(np.float32)).all()


# ---- quantiser ---------------------------------------------------------------------------------
def test_quantize_closed_forms():
    rng = np.random.default_rng(8)
    w = (rng.standard_normal((32, 512)) * 0.02).astype(np.float32)
    dq, s, z = o.quantize_minmax(w, 128)
    g = w.reshape(-1, 128)
    hi, lo = g.max(1), g.min(1)
    assert (s.reshape(-1) == (np.maximum(hi - lo, np.float32(1e-5)) / np.float32(15))).all()
    assert ((z >= 0) & (z <= 15) & (z == np.rint(z))).all()
    q = dq.reshape(-1, 128) / s.reshape(-1, 1) + z.reshape(-1, 1)
    assert np.abs(q - np.rint(q)).max() < 1e-3 and q.min() > -0.01 and q.max() < 15.01
    # min < 0 < max in every group here: min maps to q = 0 and max to q = 15
    qi = np.rint(q).astype(int)
    assert (qi.min(1) == 0).all() and (qi.max(1) == 15).all()
    # error bound of round-to-nearest: |w - dq| <= s/2 (+ rounding slack)
    assert (np.abs(g - dq.reshape(-1, 128)) <= s.reshape(-1, 1) * 0.5001).all()


def test_quantize_hand_computed_group():
    # linspace(-1, 2, 16) tiled to a group of 16: s = 3/15 = 0.2, z = 5, q = 0..15, dq = (q-5)*0.2
    x = np.linspace(-1.0, 2.0, 16, dtype=np.float32)[None, :]
    dq, s, z = o.quantize_minmax(x, 16)
    assert z[0, 0] == 5.0
    assert abs(s[0, 0] - 0.2) < 1e-7
    assert np.allclose(dq[0], (np.arange(16) - 5) * s[0, 0], atol=1e-7)


def test_quantize_half_to_even_and_constant_group():
    # x/s = 2.5 must round to 2 (ties to even), 3.5 to 4: s = 1 when max - min = 15
    x = np.array([[0.0, 15.0, 2.5, 3.5, 0.5, 1.5, 7.0, 8.0]], dtype=np.float32)
    dq, s, z = o.quantize_minmax(x, 8)
    assert s[0, 0] == 1.0 and z[0, 0] == 0.0
    assert (dq[0] == np.array([0, 15, 2, 4, 0, 2, 7, 8], np.float32)).all()
    # constant group: range clamps to 1e-5
    xc = np.full((1, 8), 0.25, np.float32)
    dq, s, z = o.quantize_minmax(xc, 8)
    assert s[0, 0] == np.float32(1e-5) / np.float32(15)
    assert z[0, 0] == 0.0            # -round(0.25/s) is hugely negative -> clamps to 0
    assert (dq[0] == np.float32(15) * s[0, 0]).all()  # q clamps to 15


def test_quantize_idempotent_and_matches_c_and_torch():
    rng = np.random.default_rng(9)
    w = (rng.standard_normal((48, 384)) * 0.02).astype(np.float32)
    dq, s, z = o.quantize_minmax(w, 128)
    dq2, s2, z2 = o.quantize_minmax(dq, 128)
    assert np.allclose(s2, s, rtol=1e-6) and (z2 == z).all() and np.allclose(dq2, dq, atol=1e-7)
    cdq, cs, cz = c.quantize_f32(w, 128)
    assert (cdq == dq).all() and (cs == s).all() and (cz == z).all()
    # same formula in torch CPU arithmetic (library cross-check of rounding/division semantics)
    t = torch.from_numpy(w).view(-1, 128)
    ts = (t.amax(1, keepdim=True) - t.amin(1, keepdim=True)).clamp(min=1e-5) / 15
    tz = (-torch.round(t.amin(1, keepdim=True) / ts)).clamp(0, 15)
    tdq = ((torch.round(t / ts) + tz).clamp(0, 15) - tz) * ts
    assert (ts.view(48, -1).numpy() == s).all() and (tz.view(48, -1).numpy() == z).all()
    assert (tdq.view(48, 384).numpy() == dq).all()


def test_quantize_symmetric():
    rng = np.random.default_rng(10)
    w = rng.standard_normal((4, 64)).astype(np.float32)
    dq, s, z = o.quantize_minmax(w, 32, 4, zero_point=False)
    assert z is None
    assert np.allclose(s.reshape(-1), np.abs(w.reshape(-1, 32)).max(1) / 7)
    q = dq.reshape(-1, 32) / s.reshape(-1, 1)
    assert q.min() >= -8.001 and q.max() <= 7.001


def test_int_quantize_recovers_codes():
    rng = np.random.default_rng(11)
    w = (rng.standard_normal((64, 256)) * 0.02).astype(np.float32)
    p = o.make_packed(w, 128, "f16")
    iw = p["intweight"]
    assert iw.min() >= 0 and iw.max() <= 15
    # (iw - z) * s reproduces the fake-quantised weight
    s = np.repeat(p["scales_gn"], 128, 0)
    z = np.repeat(p["zeros_gn"], 128, 0)
    assert np.allclose(((iw - z) * s).T, p["w_dq"], atol=1e-8)


# ---- dequant -----------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_dequant_bruteforce_and_c(dtype):
    rng = np.random.default_rng(12)
    K, N, g = 64, 16, 32
    iw = rng.integers(0, 16, (K, N), dtype=np.int32)
    z = rng.integers(0, 16, (K // g, N), dtype=np.int32)
    s32 = rng.uniform(1e-3, 3e-2, (K // g, N)).astype(np.float32)
    sb = o.to_bits16(s32, dtype)
    qw, qz = o.pack_awq(iw), o.pack_awq(z)
    got = o.dequant(qw, qz, sb, dtype)
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    st = torch.from_numpy(sb.view(np.int16)).view(tdt)
    for k in range(K):
        for n in range(N):
            # native 16-bit multiply in torch == exact product rounded once
            d = torch.tensor(float(iw[k, n] - z[k // g, n]), dtype=tdt)
            e = (d * st[k // g, n]).view(torch.int16).item() & 0xFFFF
            assert got[k, n] == e
    assert (c.dequant(qw, qz, sb, dtype) == got).all()


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_dequant_equals_fake_quant_when_weights_are_16bit(dtype):
    # weights and scales already representable in dtype -> dequant(pack(w)) == w_dq bit for bit
    rng = np.random.default_rng(13)
    w16 = o.to_dtype_f32((rng.standard_normal((32, 256)) * 0.02).astype(np.float32), dtype)
    if dtype == "f16":
        w_in = w16.astype(np.float16)
        dq, s, z = o.quantize_minmax(w_in, 128)
        s_gn, z_gn = np.ascontiguousarray(s.T), np.ascontiguousarray(z.T)
        iw = o.int_quantize(dq, s_gn, z_gn, 128)
        got = o.dequant(o.pack_awq(iw), o.pack_awq(z_gn.astype(np.int32)), s_gn.view(np.uint16), dtype)
        assert (got.view(np.float16) == dq.T).all()
    else:
        tw = torch.from_numpy(w16).to(torch.bfloat16).view(-1, 128)
        ts = (tw.amax(1, keepdim=True) - tw.amin(1, keepdim=True)).clamp(min=1e-5) / 15
        tz = (-torch.round(tw.amin(1, keepdim=True) / ts)).clamp(0, 15)
        tq = (torch.round(tw / ts) + tz).clamp(0, 15)
        tdq = ((tq - tz) * ts).view(32, 256)
        s_gn = ts.view(32, -1).t().contiguous()
        z_gn = tz.view(32, -1).t().contiguous()
        iw = tq.view(32, 256).t().contiguous().to(torch.int32).numpy()
        got = o.dequant(o.pack_awq(iw), o.pack_awq(z_gn.to(torch.int32).numpy()),
                        s_gn.view(torch.int16).numpy().view(np.uint16), dtype)
        assert (got == tdq.t().contiguous().view(torch.int16).numpy().view(np.uint16)).all()


# ---- linear ------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_linear_fp32_is_library_matmul_and_matches_c(dtype):
    from conftest import make_case, make_x
    p = make_case(256, 64, 128, dtype, seed=14)
    xb = make_x(5, 256, dtype, seed=15)
    y = o.linear_fp32(xb, p["qweight"], p["qzeros"], p["qscales"], dtype)
    w = o.dequant_f32(p["qweight"], p["qzeros"], p["qscales"], dtype)
    yt = torch.from_numpy(o.from_bits16(xb, dtype)).double() @ torch.from_numpy(w).double()
    assert np.abs(y - yt.numpy()).max() <= 1e-6 * np.abs(yt.numpy()).max()
    bias = np.linspace(-1, 1, 64, dtype=np.float32)
    yc = c.linear(xb, p["qweight"], p["qzeros"], p["qscales"], dtype, bias)
    yb = o.linear_fp32(xb, p["qweight"], p["qzeros"], p["qscales"], dtype, bias)
    assert np.abs(yc - yb).max() <= 1e-6 * np.abs(yb).max()
    # the reference's own schedule (8 rounded partials) stays inside the 1e-2 bound too
    ys = o.from_bits16(o.linear_splitk_ref(xb, p["qweight"], p["qzeros"], p["qscales"], dtype), dtype)
    assert o.max_rel_err(ys, y) < 1e-2


def test_packed_weight_bytes_table():
    assert o.packed_weight_bytes(1024, 1024) == 544768
    assert o.packed_weight_bytes(1024, 2048) == 1089536
    assert o.packed_weight_bytes(1024, 3072) == 1634304
    assert o.packed_weight_bytes(4096, 12288) == 26148864
    assert o.packed_weight_bytes(5120, 25600) == 68096000


# ---- linear_splitk_ref: the reference's own split-K rounding schedule ---------------------------------------------
def _exact_case(dtype, K=512, N=16, M=4, seed=5):
    """Integer-valued x and power-of-two scales: every fp32 partial sum is an exact integer (no dependence on the
    summation order) large enough that the roundings to 16 bits change it."""
    rng = np.random.default_rng(seed)
    q = rng.integers(0, 16, size=(K, N))
    z = rng.integers(0, 16, size=(K // 128, N))
    qweight, qzeros = o.pack_awq(q), o.pack_awq(z)
    scales = o.to_bits16(np.full((K // 128, N), 1.0, np.float32), dtype)
    x = rng.integers(-128, 129, size=(M, K)).astype(np.float32)
    return o.to_bits16(x, dtype), qweight, qzeros, scales


def _splitk_scalar_walk(x_bits, qweight, qzeros, scales, dtype, split_k, block_k, contiguous=False):
    """Scalar walk of nanoquantization/layers/gemm.py:217,251-326,378: program pid_k starts at row pid_k * BLOCK_K,
    takes BLOCK_K rows, then jumps BLOCK_K * SPLIT_K rows, cdiv(K, BLOCK_K * SPLIT_K) times, rows past K masked; the
    fp32 accumulator is stored rounded to the output type and the partials are summed and rounded once more."""
    x = o.from_bits16(x_bits, dtype)
    w = o.dequant_f32(qweight, qzeros, scales, dtype)
    M, K = x.shape
    N = w.shape[1]
    out = np.zeros((M, N), np.float32)
    iters = -(-K // (block_k * split_k))
    for m in range(M):
        for n in range(N):
            total = np.float32(0.0)
            for pid_k in range(split_k):
                acc = np.float32(0.0)
                start = pid_k * (iters * block_k) if contiguous else pid_k * block_k
                for it in range(iters):
                    for kk in range(block_k):
                        k = start + kk
                        if k < K:
                            acc = np.float32(acc + np.float32(x[m, k] * w[k, n]))
                    start += block_k if contiguous else block_k * split_k
                total = np.float32(total + o.to_dtype_f32(np.array([acc], np.float32), dtype)[0])
            out[m, n] = total
    return o.to_bits16(out, dtype)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_splitk_ref_matches_scalar_walk_of_the_kernel_schedule(dtype):
    xb, qw, qz, sc = _exact_case(dtype)
    for split_k, block_k in ((8, 32), (4, 32), (2, 64), (8, 16)):
        got = o.linear_splitk_ref(xb, qw, qz, sc, dtype, split_k, block_k)
        want = _splitk_scalar_walk(xb, qw, qz, sc, dtype, split_k, block_k)
        assert np.array_equal(got, want), (split_k, block_k)
    # the data discriminates: partial roundings are active, and a contiguous assignment of K blocks to splits
    # (a plausible slip) gives other bits
    one = o.linear_splitk_ref(xb, qw, qz, sc, dtype, 1, 512)
    assert not np.array_equal(o.linear_splitk_ref(xb, qw, qz, sc, dtype, 8, 32), one)
    wrong = _splitk_scalar_walk(xb, qw, qz, sc, dtype, 8, 32, contiguous=True)
    assert not np.array_equal(o.linear_splitk_ref(xb, qw, qz, sc, dtype, 8, 32), wrong)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_splitk_ref_closed_forms(dtype):
    from conftest import make_case, make_x
    # one split of one block = the fp32 product rounded once (exact data: no summation-order freedom)
    xb, qw, qz, sc = _exact_case(dtype, seed=9)
    x, w = o.from_bits16(xb, dtype), o.dequant_f32(qw, qz, sc, dtype)
    assert np.array_equal(o.linear_splitk_ref(xb, qw, qz, sc, dtype, 1, 512), o.to_bits16(x @ w, dtype))
    # one-hot activations return one row of the dequantised weight, bit for bit, whatever the split count: every K
    # row is owned by exactly one split, the other partials are zero
    p = make_case(256, 64, 128, dtype, seed=21)
    wbits = o.dequant(p["qweight"], p["qzeros"], p["qscales"], dtype)
    rows = [0, 31, 32, 100, 223, 255]
    eye = np.zeros((len(rows), 256), np.float32)
    eye[np.arange(len(rows)), rows] = 1.0
    for split_k in (1, 2, 4, 8):
        got = o.linear_splitk_ref(o.to_bits16(eye, dtype), p["qweight"], p["qzeros"], p["qscales"], dtype, split_k, 32)
        assert np.array_equal(got & 0x7FFF, wbits[rows] & 0x7FFF) and np.array_equal(got, np.where(
            (wbits[rows] & 0x7FFF) == 0, got, wbits[rows]))     # equal up to the sign of zero
    # more splits than blocks: the surplus splits own nothing
    xr = make_x(2, 256, dtype, seed=3)
    a = o.linear_splitk_ref(xr, p["qweight"], p["qzeros"], p["qscales"], dtype, 8, 32)
    b = o.linear_splitk_ref(xr, p["qweight"], p["qzeros"], p["qscales"], dtype, 16, 32)
    assert a.shape == b.shape == (2, 64)
    # linearity that survives the roundings: scaling x by 2 scales y by 2 exactly
    x2 = o.to_bits16(o.from_bits16(xr, dtype) * 2.0, dtype)
    y1 = o.from_bits16(a, dtype)
    y2 = o.from_bits16(o.linear_splitk_ref(x2, p["qweight"], p["qzeros"], p["qscales"], dtype, 8, 32), dtype)
    assert np.array_equal(y2, 2.0 * y1)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("g", [32, 128])
def test_torch_cpu_path_equals_the_oracle(dtype, g):
    """oracle/torch_cpu_path.py -- the restatement timed as the CPU baseline -- against the pinned numpy oracle: its
    dequantised weight is the oracle's bit for bit, its product (fp32-upcast matmul) is the fp32-accumulation oracle's
    up to the rounding of the output and the summation order."""
    import torch
    from conftest import make_case, make_x, random_packed
    from oracle import torch_cpu_path as cpu
    tdt = {"f16": torch.float16, "bf16": torch.bfloat16}[dtype]
    bits = lambda t: t.contiguous().view(torch.int16).numpy().view(np.uint16)
    for p in (make_case(256, 72, g, dtype, seed=3), random_packed(384, 64, g, dtype, seed=4)):
        qw, qz = torch.from_numpy(p["qweight"]), torch.from_numpy(p["qzeros"])
        qs = torch.from_numpy(p["qscales"].view(np.int16)).view(tdt)
        assert np.array_equal(cpu.unpack(qw).numpy(), o.unpack_awq(p["qweight"]))
        w = cpu.dequant(qw, qs, qz)
        assert w.dtype == tdt and np.array_equal(bits(w), o.dequant(p["qweight"], p["qzeros"], p["qscales"], dtype))
        K = p["qweight"].shape[0]
        xb = make_x(5, K, dtype, seed=6)
        x = torch.from_numpy(xb.view(np.int16)).view(tdt)
        ref = o.linear_fp32(xb, p["qweight"], p["qzeros"], p["qscales"], dtype)
        y = cpu.linear(x, qw, qs, qz, upcast=True)
        assert y.dtype == tdt
        # the output is rounded to 16 bits (half an ulp: 2^-11 / 2^-8 of the value); 1e-3 with fp16
        tol = 1e-3 if dtype == "f16" else 4e-3
        assert o.max_rel_err(y.float().numpy(), ref) <= tol
        # the native 16-bit matmul agrees with the reference's tolerance for the product (1e-2)
        assert o.max_rel_err(cpu.linear(x, qw, qs, qz, upcast=False).float().numpy(), ref) <= 1e-2
