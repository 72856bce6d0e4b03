"""The PyTorch operator binding (csrc/torch_binding.cpp -> libawq_torch.so): torch.ops.nanoquantization_amd.* over
the C ABI.  CPU: the library loads, the schemas are registered, shape inference works on meta tensors, and host
tensors are refused.  GPU: the operators return the bits of the C entry points called directly."""
import pytest
import torch

import nanoquantization_amd as nq
from nanoquantization_amd import _lib
from nanoquantization_amd.layers.gemm import _linear
from conftest import random_packed, to_dev


def test_ops_registered_with_schemas():
    ops = _lib.torch_ops()
    assert str(ops.awq_linear.default._schema) == (
        "nanoquantization_amd::awq_linear(Tensor x, Tensor qweight, Tensor qscales, Tensor qzeros, "
        "Tensor? bias=None) -> Tensor")
    assert "awq_dequantize(Tensor qweight, Tensor qscales, Tensor qzeros) -> Tensor" in str(ops.awq_dequantize.default._schema)
    assert "awq_linear_swiglu(Tensor x, Tensor qweight, Tensor qscales, Tensor qzeros) -> Tensor" in str(
        ops.awq_linear_swiglu.default._schema)


def test_meta_shapes():
    ops = _lib.torch_ops()
    qw = torch.zeros(256, 8, dtype=torch.int32, device="meta")
    qs = torch.zeros(2, 64, dtype=torch.bfloat16, device="meta")
    qz = torch.zeros(2, 8, dtype=torch.int32, device="meta")
    x = torch.zeros(5, 256, dtype=torch.bfloat16, device="meta")
    y = ops.awq_linear(x, qw, qs, qz, None)
    assert y.shape == (5, 64) and y.dtype == torch.bfloat16 and y.device.type == "meta"
    assert ops.awq_dequantize(qw, qs, qz).shape == (256, 64)
    assert ops.awq_linear_swiglu(x, qw, qs, qz).shape == (5, 32)


def test_host_tensors_are_refused():
    ops = _lib.torch_ops()
    m = nq.WQLinear_GEMM(4, 128, 256, 64, output_dtype=torch.float16)
    with pytest.raises(NotImplementedError):   # no CPU kernel is registered: there is no fallback to fall into
        ops.awq_linear(torch.zeros(2, 256, dtype=torch.float16), m.qweight, m.qscales, m.qzeros, None)
    with pytest.raises(_lib.AwqHipError):
        m(torch.zeros(2, 256, dtype=torch.float16))


def _packed(K, N, g, dt, seed=0):
    p = random_packed(K, N, g, dt, seed=seed)
    return to_dev(p["qweight"]), to_dev(p["qscales"], dt), to_dev(p["qzeros"])


@pytest.mark.gpu
@pytest.mark.parametrize("dt,tdt", [("f16", torch.float16), ("bf16", torch.bfloat16)])
def test_op_equals_c_abi(dt, tdt):
    ops = _lib.torch_ops()
    for (M, K, N, g) in [(1, 1024, 3072, 128), (16, 1024, 3072, 128), (40, 1024, 1024, 128), (300, 512, 256, 64),
                         (7, 256, 72, 32)]:
        print(f"torch op vs C ABI {dt} M={M} K={K} N={N} g={g}", flush=True)
        qw, qs, qz = _packed(K, N, g, dt, seed=M)
        torch.manual_seed(M)
        x = torch.randn(M, K, device="cuda").to(tdt)
        bias = torch.randn(N, device="cuda").to(tdt)
        assert torch.equal(ops.awq_linear(x, qw, qs, qz, None), _linear("awq_linear", x, qw, qs, qz, None))
        assert torch.equal(ops.awq_linear(x, qw, qs, qz, bias), _linear("awq_linear", x, qw, qs, qz, bias))
        out = torch.empty(K, N, dtype=tdt, device="cuda")
        _lib.check(_lib.lib().awq_dequantize(qw.data_ptr(), qs.data_ptr(), qz.data_ptr(), out.data_ptr(), K, N, g,
                                             _lib.dtype_id(tdt), _lib.current_stream_ptr(out.device)))
        assert torch.equal(ops.awq_dequantize(qw, qs, qz), out)


@pytest.mark.gpu
def test_op_argument_checks_and_edge_cases():
    ops = _lib.torch_ops()
    qw, qs, qz = _packed(256, 64, 128, "f16")
    x = torch.randn(3, 256, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError, match=r"x must be \[M, 256\]"):
        ops.awq_linear(x[:, :128], qw, qs, qz, None)
    with pytest.raises(RuntimeError, match="int32"):
        ops.awq_linear(x, qw.float(), qs, qz, None)
    with pytest.raises(RuntimeError, match="float16 or bfloat16"):
        ops.awq_linear(x, qw, qs.float(), qz, None)
    with pytest.raises(RuntimeError, match="bias must have 64"):
        ops.awq_linear(x, qw, qs, qz, torch.zeros(8, dtype=torch.float16, device="cuda"))
    with pytest.raises(RuntimeError, match="different devices"):
        ops.awq_linear(x, qw.cpu(), qs, qz, None)
    assert ops.awq_linear(x[:0], qw, qs, qz, None).shape == (0, 64)
    # x in another 16-bit type is cast to the scales' type, a strided x is made dense
    xt = torch.randn(256, 3, dtype=torch.bfloat16, device="cuda").t()
    assert torch.equal(ops.awq_linear(xt, qw, qs, qz, None), ops.awq_linear(xt.to(torch.float16).contiguous(), qw, qs, qz, None))


@pytest.mark.gpu
def test_op_runs_on_the_current_stream_and_under_graph_capture():
    ops = _lib.torch_ops()
    qw, qs, qz = _packed(2048, 1024, 128, "f16")     # split-K shape: uses the binding's own workspace
    x = torch.randn(16, 2048, dtype=torch.float16, device="cuda")
    want = ops.awq_linear(x, qw, qs, qz, None)
    s = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    y = None
    with torch.cuda.stream(s):
        assert torch.equal(ops.awq_linear(x, qw, qs, qz, None), want)    # allocates this stream's workspace
        torch.cuda.synchronize()
        with torch.cuda.graph(g, stream=s):
            y = ops.awq_linear(x, qw, qs, qz, None)
    torch.cuda.synchronize()
    for rep in range(3):
        y.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want), rep
