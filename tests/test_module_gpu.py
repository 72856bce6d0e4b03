"""WQLinear_GEMM.forward on the GPU: shapes, dtype, bias, regime switch, state_dict round trip."""
import numpy as np
import pytest
import torch

import nanoquantization_amd as nq
from conftest import to_bits
from oracle import awq_oracle as o

pytestmark = pytest.mark.gpu


def _module(K, N, g, tdt, bias, seed=0):
    torch.manual_seed(seed)
    w = torch.randn(N, K) * 0.02
    dq, s, z = nq.pseudo_quantize(w, g, 4, True)
    lin = torch.nn.Linear(K, N, bias=bias)
    lin.weight.data = dq
    return nq.WQLinear_GEMM.from_linear(lin, 4, g, s.t().contiguous(), z.t().contiguous(), tdt).to("cuda")


@pytest.mark.parametrize("tdt,dt", [(torch.float16, "f16"), (torch.bfloat16, "bf16")])
@pytest.mark.parametrize("bias", [False, True])
def test_forward_matches_oracle_all_regimes(tdt, dt, bias):
    K, N, g = 1024, 3072, 128
    m = _module(K, N, g, tdt, bias)
    qw, qz = m.qweight.cpu().numpy(), m.qzeros.cpu().numpy()
    qs = to_bits(m.qscales)
    b = m.bias.float().cpu().numpy() if bias else None
    for shape in [(16, K), (1, K), (2, 3, K), (4, 40, K), (300, K)]:   # cfg1 is the first
        print(f"forward {dt} bias={bias} x{shape}", flush=True)
        torch.manual_seed(sum(shape))
        x = torch.randn(*shape).to(tdt).cuda()
        y = m(x)
        assert y.shape == x.shape[:-1] + (N,) and y.dtype == tdt
        ref = o.linear_fp32(to_bits(x.reshape(-1, K)), qw, qz, qs, dt, b)
        err = o.max_rel_err(y.float().cpu().numpy().reshape(-1, N), ref)
        assert err <= 1e-2 and err <= (1.5e-3 if dt == "f16" else 6e-3), err


def test_forward_casts_x_to_scale_dtype():
    # the reference's test runs fp16 activations through bf16 scales: x is cast on load (layers/gemm.py:259)
    m = _module(512, 256, 128, torch.bfloat16, False)
    x = torch.randn(8, 512, dtype=torch.float16, device="cuda")
    y = m(x)
    assert y.dtype == torch.bfloat16
    assert torch.equal(y, m(x.to(torch.bfloat16)))


def test_state_dict_roundtrip_keeps_outputs():
    m = _module(512, 256, 128, torch.float16, False)
    m2 = nq.WQLinear_GEMM(4, 128, 512, 256, bias=False, output_dtype=torch.float16)
    m2.load_state_dict({k: v.cpu() for k, v in m.state_dict().items()})
    m2 = m2.to("cuda")
    x = torch.randn(5, 512, dtype=torch.float16, device="cuda")
    assert torch.equal(m(x), m2(x))
    # with a bias the constructor's buffer is bf16 whatever the output dtype (layers/gemm.py:435-443),
    # so a loaded fp16 bias is rounded to bf16: equal only to bf16 precision
    mb = _module(512, 256, 128, torch.float16, True)
    mb2 = nq.WQLinear_GEMM(4, 128, 512, 256, bias=True, output_dtype=torch.float16)
    mb2.load_state_dict({k: v.cpu() for k, v in mb.state_dict().items()})
    mb2 = mb2.to("cuda")
    assert mb2.bias.dtype == torch.bfloat16
    assert (mb(x).float() - mb2(x).float()).abs().max().item() <= 2.0 ** -8 * mb.bias.abs().max().item() + 2e-3


@pytest.mark.parametrize("bias", [False, True])
def test_forward_empty_and_boundary_row_counts(bias):
    """No rows at all, and the row counts where the dispatch changes kernel (16/17 one m-tile vs row blocks, 64/65
    and 128/129 GEMV vs GEMM -- 128 rows on small weights like this one --, 1023/1024 where the reference's own structure
    changes): shape, dtype and the fp32 oracle at every one of them."""
    K, N, g = 512, 384, 128
    m = _module(K, N, g, torch.bfloat16, bias, seed=3)
    for shape in [(0, K), (2, 0, K)]:
        y = m(torch.zeros(*shape, dtype=torch.bfloat16, device="cuda"))
        assert y.shape == tuple(shape[:-1]) + (N,) and y.dtype == torch.bfloat16 and y.numel() == 0
    qw, qz, qs = m.qweight.cpu().numpy(), m.qzeros.cpu().numpy(), to_bits(m.qscales)
    b = m.bias.float().cpu().numpy() if bias else None
    for M in (16, 17, 64, 65, 128, 129, 1023, 1024):
        print(f"forward boundary M={M} bias={bias}", flush=True)
        torch.manual_seed(M)
        x = torch.randn(M, K).to(torch.bfloat16).cuda()
        ref = o.linear_fp32(to_bits(x), qw, qz, qs, "bf16", b)
        err = o.max_rel_err(m(x).float().cpu().numpy(), ref)
        assert err <= 6e-3, (M, err)


@pytest.mark.parametrize("K,N,g", [(1024, 151936, 128), (65536, 1024, 128), (128, 8, 128), (64, 8, 64), (32, 4096, 32),
                                   (256, 262144, 128)])
def test_linear_extreme_widths_default_dispatch(K, N, g):
    """Widths at the ends of what the entry point takes -- a vocabulary-sized N (a quantised lm_head), one packed word
    of N, one group of K, a K of 512 chunks -- at row counts on both sides of every regime switch, through the default
    dispatch.  Reference: x @ awq_dequantize(...) in fp32 on the device (the dequantise kernel is bit-exact against the
    oracle, tests/test_dequant_gpu.py; the CPU oracle would need minutes at these sizes).  Bound: the 1e-2 of the
    task, and the rounding-only bound the other GEMV tests use."""
    from nanoquantization_amd.layers.gemm import _linear
    torch.manual_seed(K + N)
    for tdt, tight in ((torch.float16, 1.5e-3), (torch.bfloat16, 6e-3)):
        qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (K, N // 8), dtype=torch.int32, device="cuda")
        qz = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // g, N // 8), dtype=torch.int32, device="cuda")
        qs = (torch.rand(K // g, N, device="cuda") * 0.02 + 0.001).to(tdt)
        W = nq.awq_dequantize(qw, qs, qz).float()
        for M in (1, 5, 16, 17, 64, 65, 129):
            print(f"extreme widths K={K} N={N} g={g} {tdt} M={M}", flush=True)
            x = (torch.randn(M, K, device="cuda") * 0.5).to(tdt)
            y = _linear("awq_linear", x, qw, qs, qz, None)
            ref = x.float() @ W
            err = ((y.float() - ref).abs().max() / ref.abs().max()).item()
            assert y.shape == (M, N) and y.dtype == tdt and err <= tight, (M, err)
        del W
