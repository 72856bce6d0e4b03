"""Golden fixtures (tests/golden/): the oracle, its C restatement and the host packer reproduce them on
the CPU; the HIP kernels reproduce them on the GPU."""
import glob
import json
import os

import numpy as np
import pytest
import torch

from oracle import awq_oracle as o
from oracle import c_oracle as c

HERE = os.path.dirname(os.path.abspath(__file__))
FIXTURES = sorted(glob.glob(os.path.join(HERE, "golden", "awq_*.npz")))


def _dtype_of(path):
    return "bf16" if "_bf16_" in os.path.basename(path) else "f16"


def test_fixtures_present():
    assert len(FIXTURES) >= 3


def test_kat_words():
    kat = json.load(open(os.path.join(HERE, "golden", "kat_words.json")))
    assert tuple(kat["order"]) == o.AWQ_ORDER and tuple(kat["shifts"]) == o.AWQ_SHIFT
    from nanoquantization_amd.layers.gemm import pack_awq
    for w in kat["words"]:
        cols = np.array([w["columns"]], dtype=np.int32)
        assert int(o.pack_awq(cols)[0, 0]) == w["int32"]
        assert int(c.pack(cols)[0, 0]) == w["int32"]
        assert int(pack_awq(torch.from_numpy(cols))[0, 0]) == w["int32"]
        assert (w["int32"] & 0xFFFFFFFF) == int(w["hex"], 16)
        assert (o.unpack_awq(np.array([[w["int32"]]], dtype=np.int32))[0] == cols[0]).all()


@pytest.mark.parametrize("path", FIXTURES, ids=os.path.basename)
def test_oracle_reproduces_fixture(path):
    d = np.load(path)
    dt = _dtype_of(path)
    g = int(d["group_size"])
    p = o.make_packed(d["w"], g, dt)
    assert (p["qweight"] == d["qweight"]).all() and (p["qzeros"] == d["qzeros"]).all()
    assert (p["qscales"] == d["qscales"]).all()
    assert (o.dequant(d["qweight"], d["qzeros"], d["qscales"], dt) == d["w_dequant"]).all()
    assert (c.dequant(d["qweight"], d["qzeros"], d["qscales"], dt) == d["w_dequant"]).all()
    y = c.linear(d["x"], d["qweight"], d["qzeros"], d["qscales"], dt)
    assert np.abs(y - d["y"]).max() <= 1e-6 * np.abs(d["y"]).max()


@pytest.mark.parametrize("path", FIXTURES, ids=os.path.basename)
def test_host_quantise_and_pack_reproduce_fixture(path):
    import nanoquantization_amd as nq
    d = np.load(path)
    dt = _dtype_of(path)
    tdt = torch.float16 if dt == "f16" else torch.bfloat16
    g = int(d["group_size"])
    w = torch.from_numpy(d["w"])
    dq, s, z = nq.pseudo_quantize(w, g, 4, True)
    lin = torch.nn.Linear(w.shape[1], w.shape[0], bias=False)
    lin.weight.data = dq
    m = nq.WQLinear_GEMM.from_linear(lin, 4, g, s.t().contiguous(), z.t().contiguous(), tdt)
    assert (m.qweight.numpy() == d["qweight"]).all() and (m.qzeros.numpy() == d["qzeros"]).all()
    assert (m.qscales.view(torch.int16).numpy().view(np.uint16) == d["qscales"]).all()


@pytest.mark.gpu
@pytest.mark.parametrize("path", FIXTURES, ids=os.path.basename)
def test_hip_reproduces_fixture(path):
    import nanoquantization_amd as nq
    from conftest import to_bits, to_dev
    d = np.load(path)
    dt = _dtype_of(path)
    print(f"golden {os.path.basename(path)}", flush=True)
    qw, qs, qz = to_dev(d["qweight"]), to_dev(d["qscales"], dt), to_dev(d["qzeros"])
    assert (to_bits(nq.awq_dequantize(qw, qs, qz)) == d["w_dequant"]).all()
    y = nq.awq_gemm(to_dev(d["x"], dt), qw, qs, qz, 8)
    assert o.max_rel_err(o.from_bits16(to_bits(y), dt), d["y"]) <= 1e-2
    m = nq.WQLinear_GEMM(4, int(d["group_size"]), qw.shape[0], qs.shape[1], bias=True,
                         output_dtype=qs.dtype).to("cuda")
    m.qweight, m.qscales, m.qzeros = qw, qs, qz
    m.bias = to_dev(d["bias"], dt)
    yb = m(to_dev(d["x"], dt))
    assert o.max_rel_err(o.from_bits16(to_bits(yb), dt), d["y_bias"]) <= 1e-2
