"""The device quantise+pack kernel against the CPU oracle's quantise -> transpose -> int-quantise -> pack
chain (utils/quantization.py:5-58, awq/quantizer.py:156-158, layers/gemm.py:474-548 of the reference):
packed words, zero words and scales must be bit-identical."""
import numpy as np
import pytest
import torch

from oracle import awq_oracle as o

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("N,K,g", [(3072, 1024, 128), (64, 256, 32), (8, 128, 128), (1000, 384, 64), (40, 512, 512)])
def test_quantize_pack_bit_exact(dtype, N, K, g):
    import nanoquantization_amd as nq
    rng = np.random.default_rng(N * 7 + K + g)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    w[0, :g] = 0.125            # a constant group: max == min, scale = 1e-5 / 15
    w[1 % N, g - 1] = 3.0       # an outlier that stretches one group
    w[2 % N, :g] = np.linspace(-1.0, 2.0, g, dtype=np.float32)
    ref = o.make_packed(w, g, dtype)
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    print(f"quantize_pack N={N} K={K} g={g} {dtype}", flush=True)
    qw, qs, qz = nq.quantize_pack(torch.from_numpy(w).cuda(), g, tdt)
    assert np.array_equal(qw.cpu().numpy(), ref["qweight"])
    assert np.array_equal(qz.cpu().numpy(), ref["qzeros"])
    assert np.array_equal(qs.cpu().view(torch.int16).numpy().view(np.uint16), ref["qscales"])


def test_quantize_pack_feeds_the_linear():
    import nanoquantization_amd as nq
    torch.manual_seed(0)
    w = torch.randn(512, 256) * 0.02
    x = torch.randn(5, 256).half()
    qw, qs, qz = nq.quantize_pack(w.cuda(), 128, torch.float16)
    y = nq.awq_gemm(x.cuda(), qw, qs, qz, 8).float().cpu()
    dq, _, _ = nq.pseudo_quantize(w, 128, 4, True)
    ref = x.float() @ dq.t()
    assert (y - ref).abs().max() <= 1e-2 * ref.abs().max()


def test_quantize_pack_rejects_bad_input():
    import nanoquantization_amd as nq
    from nanoquantization_amd import _lib
    with pytest.raises(_lib.AwqHipError, match="HIP device only"):
        nq.quantize_pack(torch.zeros(8, 128), 128)
    with pytest.raises(AssertionError, match="nan"):
        nq.quantize_pack(torch.full((8, 128), float("nan")).cuda(), 128)
