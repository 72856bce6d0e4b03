"""Kernel (a): awq_dequantize through the C ABI, bit-exact against the oracle."""
import numpy as np
import pytest
import torch

import nanoquantization_amd as nq
from conftest import make_case, random_packed, to_bits, to_dev
from oracle import awq_oracle as o

pytestmark = pytest.mark.gpu


def _run(p, dtype):
    out = nq.awq_dequantize(to_dev(p["qweight"]), to_dev(p["qscales"], dtype), to_dev(p["qzeros"]))
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("K,N,g", [(1024, 3072, 128), (1024, 2048, 32), (256, 8, 128), (384, 1000, 64),
                                   (128, 2056, 128), (512, 512, 512)])
def test_dequant_bit_exact_random_codes(dtype, K, N, g):
    print(f"dequant case {dtype} K={K} N={N} g={g}", flush=True)
    p = random_packed(K, N, g, dtype, seed=K + N)
    out = _run(p, dtype)
    assert tuple(out.shape) == (K, N) and out.dtype == (torch.float16 if dtype == "f16" else torch.bfloat16)
    expect = o.dequant(p["qweight"], p["qzeros"], p["qscales"], dtype)
    assert (to_bits(out) == expect).all()


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_dequant_matches_fake_quantised_weight(dtype):
    # the reference's own test: dequant(pack(w)) ~ w_dq.T within atol 1e-2 (awq/tests/dequantization_kernel.py:106)
    print(f"dequant vs w_dq {dtype}", flush=True)
    p = make_case(1024, 2048, 32, dtype, seed=2, w_std=1.0)
    out = _run(p, dtype).float().cpu().numpy()
    if dtype == "f16":
        assert np.abs(out - p["w_dq"].T).max() <= 1e-2
    else:   # bf16 scales carry 8 significant bits: the bound is relative (two roundings of 2^-9 each)
        assert (np.abs(out - p["w_dq"].T) <= np.abs(p["w_dq"].T) * 2.0 ** -7 + 1e-6).all()
    assert (to_bits(_run(p, dtype)) == o.dequant(p["qweight"], p["qzeros"], p["qscales"], dtype)).all()


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_dequant_tiny_and_huge_scales(dtype):
    # subnormal fp16 products, the 1e-5/15 scale of a constant group, large scales, all-15 words (negative int32)
    print(f"dequant scale extremes {dtype}", flush=True)
    K, N, g = 256, 64, 128
    rng = np.random.default_rng(5)
    iw = rng.integers(0, 16, (K, N), dtype=np.int32)
    iw[:, :8] = 15
    z = rng.integers(0, 16, (K // g, N), dtype=np.int32)
    s = np.empty((K // g, N), np.float32)
    s[0] = np.float32(1e-5) / np.float32(15)
    s[1] = np.geomspace(1e-7, 3000.0, N).astype(np.float32)
    p = {"qweight": o.pack_awq(iw), "qzeros": o.pack_awq(z), "qscales": o.to_bits16(s, dtype)}
    assert (p["qweight"][:, 0] == -1).all()
    out = _run(p, dtype)
    assert (to_bits(out) == o.dequant(p["qweight"], p["qzeros"], p["qscales"], dtype)).all()


def test_dequant_full_size_checksum():
    # Qwen3-8B MLP shape: too slow to compare element-wise against the scalar C oracle, so compare with the
    # vectorised oracle and through a size-independent property: rows of one group differ only through q
    print("dequant full size 4096x12288 bf16", flush=True)
    K, N, g = 4096, 12288, 128
    p = random_packed(K, N, g, "bf16", seed=9)
    out = _run(p, "bf16")
    expect = o.dequant(p["qweight"], p["qzeros"], p["qscales"], "bf16")
    assert (to_bits(out) == expect).all()


def test_dequant_errors():
    p = random_packed(256, 64, 128, "f16")
    qw, qs, qz = to_dev(p["qweight"]), to_dev(p["qscales"], "f16"), to_dev(p["qzeros"])
    with pytest.raises(AssertionError):
        nq.awq_dequantize(qw[:, :4], qs, qz)
    with pytest.raises(AssertionError):
        nq.awq_dequantize(qw, qs, qz[:1])
