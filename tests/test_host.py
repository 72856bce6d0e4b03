"""CPU-side checks of the product: the host mirror of the reference interface against the oracle, the
module contract, and that the C-ABI library loads and exports every declared symbol (no compute)."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import nanoquantization_amd as nq
from nanoquantization_amd import _lib
from nanoquantization_amd.layers.gemm import pack_awq
from oracle import awq_oracle as o

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _ensure_built():
    if not os.path.exists(_lib.LIB_PATH):
        from nanoquantization_amd.build import build
        build(verbose=False)


def test_library_exports_every_declared_symbol():
    _ensure_built()
    header = open(os.path.join(ROOT, "include", "awq_hip.h")).read()
    header += open(os.path.join(ROOT, "include", "nq_engine_ops.h")).read()
    declared = set(re.findall(r"\b((?:awq|nq)_[a-z0-9_]+)\s*\(", header))
    declared -= {"awq_status", "awq_dtype"}
    assert declared, "no declarations parsed"
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name in sorted(declared):
        assert hasattr(handle, name), f"{name} declared in include/*.h but not exported"
    assert declared == set(_lib.SYMBOLS), "ctypes table and header disagree"
    L = _lib.lib()
    assert L.awq_hip_version() >= 100
    assert L.awq_gemv_variant_count() >= 1 and L.awq_gemm_variant_count() >= 1
    assert L.awq_gemv_variant_name(0)
    # argument validation happens before anything touches a device
    rc = L.awq_gemv(None, None, None, None, None, None, 1, 8, 128, 128, 0, None, 0, None)
    assert rc == 1 and b"null pointer" in L.awq_hip_last_error()
    # the published packed-weight workspace rule: 0 bytes when there is nothing to split
    assert L.awq_gemv_ex_workspace_bytes(1, 1024, 1024, 0, 1) == 0
    assert L.awq_gemv_ex_workspace_bytes(4, 1024, 1024, 0, 4) == 4096 * 4 + 4 * 4 * 1024 * 4


def test_pseudo_quantize_matches_oracle_bitwise():
    torch.manual_seed(0)
    w = torch.randn(96, 512) * 0.02
    dq, s, z = nq.pseudo_quantize(w, 128, 4, True)
    odq, os_, oz = o.quantize_minmax(w.numpy(), 128)
    assert (dq.numpy() == odq).all() and (s.numpy() == os_).all() and (z.numpy() == oz).all()
    assert dq.shape == w.shape and s.shape == (96, 4) and z.shape == (96, 4)
    dq, s, z = nq.pseudo_quantize(w, 64, 4, False)
    odq, os_, oz = o.quantize_minmax(w.numpy(), 64, 4, False)
    assert z is None and oz is None and (dq.numpy() == odq).all() and (s.numpy() == os_).all()
    wh = w.half()
    dq, s, z = nq.pseudo_quantize(wh, 32, 4, True)
    odq, os_, oz = o.quantize_minmax(wh.numpy(), 32)
    assert dq.dtype == torch.float16 and (dq.numpy() == odq).all() and (z.numpy() == oz).all()


def test_pseudo_quantize_rejects_nan_and_bad_group():
    w = torch.randn(4, 128)
    w[0, 0] = float("nan")
    with pytest.raises(AssertionError):
        nq.pseudo_quantize(w, 128, 4, True)
    with pytest.raises(AssertionError):
        nq.pseudo_quantize(torch.randn(4, 100), 128, 4, True)


@pytest.mark.parametrize("dt,tdt", [("f16", torch.float16), ("bf16", torch.bfloat16)])
@pytest.mark.parametrize("g", [32, 128])
def test_from_linear_matches_oracle_words(dt, tdt, g):
    torch.manual_seed(1)
    N, K = 72, 256
    w = torch.randn(N, K) * 0.02
    dq, s, z = nq.pseudo_quantize(w, g, 4, True)
    lin = torch.nn.Linear(K, N, bias=True)
    lin.weight.data = dq
    m = nq.WQLinear_GEMM.from_linear(lin, 4, g, s.t().contiguous(), z.t().contiguous(), tdt)
    p = o.make_packed(w.numpy(), g, dt)
    assert m.qweight.dtype == torch.int32 and tuple(m.qweight.shape) == (K, N // 8)
    assert (m.qweight.numpy() == p["qweight"]).all()
    assert (m.qzeros.numpy() == p["qzeros"]).all()
    assert m.qscales.dtype == tdt
    assert (m.qscales.view(torch.int16).numpy().view(np.uint16) == p["qscales"]).all()
    assert m.bias is not None and m.bias.dtype == tdt and m.bias.shape == (N,)


def test_pack_known_words_and_sign():
    v = torch.tensor([[0, 1, 2, 3, 4, 5, 6, 7], [8, 9, 10, 11, 12, 13, 14, 15], [15] * 8, [0, 1, 0, 0, 0, 0, 0, 0]])
    assert pack_awq(v).flatten().tolist() == [1966171168, -38146904, -1, 0x00010000]
    assert pack_awq(v).dtype == torch.int32


def test_module_contract():
    m = nq.WQLinear_GEMM(4, 128, 1024, 3072)
    assert m.qweight.shape == (1024, 384) and m.qweight.dtype == torch.int32
    assert m.qscales.shape == (8, 3072) and m.qscales.dtype == torch.bfloat16
    assert m.qzeros.shape == (8, 384) and m.qzeros.dtype == torch.int32
    assert m.bias is None
    assert set(dict(m.named_buffers())) == {"qweight", "qscales", "qzeros"}
    assert (m.w_bits, m.group_size, m.in_features, m.out_features) == (4, 128, 1024, 3072)
    mb = nq.WQLinear_GEMM(4, 128, 256, 64, bias=True, output_dtype=torch.float16)
    assert mb.bias.dtype == torch.bfloat16 and mb.qscales.dtype == torch.float16
    assert "bias" in dict(mb.named_buffers())
    with pytest.raises(ValueError):
        nq.WQLinear_GEMM(8, 128, 256, 64)
    with pytest.raises(AssertionError):
        nq.WQLinear_GEMM(4, 128, 200, 64)
    with pytest.raises(AssertionError):
        nq.WQLinear_GEMM(4, 128, 256, 60)
    # state_dict keys are the checkpoint contract
    assert list(m.state_dict()) == ["qweight", "qscales", "qzeros"]


def test_no_cpu_fallback():
    m = nq.WQLinear_GEMM(4, 128, 256, 64, output_dtype=torch.float16)
    with pytest.raises(_lib.AwqHipError):
        m(torch.randn(2, 256, dtype=torch.float16))
    with pytest.raises(_lib.AwqHipError):
        nq.awq_dequantize(m.qweight, m.qscales, m.qzeros)


def test_product_does_not_import_oracle():
    pkg = os.path.join(ROOT, "nanoquantization_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, f"{f} mentions the oracle"


def _plan(fn, *args):
    v, s = ctypes.c_int(-1), ctypes.c_int(-1)
    rc = fn(*args, ctypes.byref(v), ctypes.byref(s))
    return rc, v.value, s.value


def test_dispatch_plans_are_consistent():
    """Host-only: for a sweep of shapes, the variant and K split the library would pick are valid for the shape, fit
    the workspace it asks for, and follow the documented rules (no device call is made)."""
    _ensure_built()
    L = _lib.lib()
    gemv_names = [L.awq_gemv_variant_name(i).decode() for i in range(L.awq_gemv_variant_count())]
    gemm_names = [L.awq_gemm_variant_name(i).decode() for i in range(L.awq_gemm_variant_count())]
    shapes = [(1024, 2048), (1024, 1024), (2048, 1024), (1024, 3072), (3072, 1024), (4096, 12288), (12288, 4096),
              (5120, 25600), (25600, 5120), (5120, 10240), (8192, 5120), (5120, 34816), (4096, 24576), (5120, 20480),
              (8192, 14336), (12288, 8192), (8192, 8192), (6144, 10240), (16384, 4096), (128, 128),
              (256, 8), (1024, 1032), (3072, 136)]
    for K, N in shapes:
        for M in (1, 2, 4, 5, 8, 16, 17, 32, 33, 48, 64):
            for g in (128, 32):
                rc, v, s = _plan(L.awq_gemv_plan, M, N, K, g)
                staged_ok = N % 128 == 0 and g % 128 == 0
                if M > 16 and not staged_ok:
                    assert rc != 0, (M, N, K, g)
                    continue
                assert rc == 0 and 0 <= v < len(gemv_names) and s >= 1, (M, N, K, g, rc, v, s)
                name = gemv_names[v]
                chunks = max(K // 128, 1)
                assert s <= chunks, (name, s, chunks)
                if name.startswith(("dma", "wide")):
                    assert staged_ok
                else:
                    assert M <= 16
                if name.startswith("wide"):
                    cols = 256 if name.startswith("wide2") else 512      # columns per workgroup
                    assert N % cols == 0 and K * N >= (40000000 if M > 48 else 45000000 if M > 32 else 48000000)
                    one = name.endswith(("m1", "m1t"))
                    assert one == (M <= 16) and name.endswith("m4") == (M > 32)
                    cps = -(-chunks // s)
                    wgs = N // cols * -(-chunks // cps)
                    if name.endswith("t"):                               # in-kernel tail: few rows x splits
                        assert M <= 8 and M * s <= 64 and s <= 25
                        assert wgs <= 560
                    elif one or M > 16:
                        assert wgs <= 256 + N // cols or cols == 256     # second pass: about one workgroup per CU
                    if "d3" in name:                                     # three staging buffers
                        assert (one or name == "wide2d3m2") and cps >= 6 and (wgs <= 256 or cols == 256)
                    if cols == 256 and M <= 32:
                        assert (5120 if one else 4096) <= N < 28672
                    if name == "wide2d2m4":                               # plan B from 92 % of the CUs, else about 500
                        assert N >= 3584 and chunks >= 28
                        assert (216 <= wgs <= 256 and cps <= 11) or wgs > 256 or 512 // (N // 256) >= chunks // 4
                if not staged_ok:
                    assert not name.startswith(("dma", "wide"))
                if g == 128:   # awq_gemv_workspace_bytes takes no group size: it must cover this plan
                    assert L.awq_gemv_ex_workspace_bytes(M, N, K, v, s) <= L.awq_gemv_workspace_bytes(M, N, K)
                    assert L.awq_gemv_workspace_bytes(M, N, K) <= L.awq_linear_workspace_bytes(M, N, K)
        for M in (17, 64, 65, 128, 129, 512, 1000, 2048, 8192):
            if K % 64:
                continue
            rc, v, s = _plan(L.awq_gemm_plan, M, N, K, 128, _lib.AWQ_BF16)
            assert rc == 0 and 0 <= v < len(gemm_names) and 1 <= s <= 16, (M, N, K, rc, v, s)
            assert s <= max(K // 64 // 8, 1)                         # at least 8 K steps per split
            assert (gemm_names[v].startswith("256x256")) == (M > 128)
            # the plan names the kernel that runs: the register-operand one (r) only where the work items reach the
            # 256 CUs, the group size is a multiple of 64 and N of 128; never for a group size it does not take
            tiles = -(-M // 256) * -(-N // 256)
            tail = tiles % 256 if gemm_names[v].endswith("t") else (tiles if s > 1 else 0)
            items = tiles - tail + tail * s
            if gemm_names[v] in ("256x256r", "256x256rt"):
                assert items >= 256 and N % 128 == 0, (M, N, K, gemm_names[v], s)
            elif gemm_names[v] in ("256x256p", "256x256pt") and N % 128 == 0:
                assert items <= 256, (M, N, K, gemm_names[v], s)
            rc32, v32, s32 = _plan(L.awq_gemm_plan, M, N, K, 32, _lib.AWQ_BF16)
            assert rc32 == 0 and s32 == s and gemm_names[v32] == gemm_names[v].replace("r", "p"), (M, N, K)
            assert L.awq_gemm_ex_workspace_bytes(M, N, K, v, s) == L.awq_gemm_workspace_bytes(M, N, K)
            assert L.awq_gemm_workspace_bytes(M, N, K) <= L.awq_linear_workspace_bytes(M, N, K)
    # the whole-rounds rule for 5..64 rows: 272 column tiles are cut so that the workgroups fill the 256 CUs evenly
    rc, v, s = _plan(L.awq_gemv_plan, 16, 34816, 2048, 128)
    assert rc == 0 and gemv_names[v] == "dma1x4" and s >= 3
    wgs = 34816 // 128 * s
    assert wgs / (256 * -(-wgs // 256)) >= 0.8
    # up to 16 rows on wide, large weights: the one-m-tile forms of the shared-chunk kernel
    rc, v, s = _plan(L.awq_gemv_plan, 16, 34816, 5120, 128)      # N >= 28672: 512 columns, 68 groups x 3 splits of 14 chunks
    assert rc == 0 and gemv_names[v] == "wided3m1" and s == 3
    rc, v, s = _plan(L.awq_gemv_plan, 4, 34816, 5120, 128)       # three or four rows there: ten splits would be too many
    assert rc == 0 and gemv_names[v] == "dma1x4" and s == 5
    rc, v, s = _plan(L.awq_gemv_plan, 1, 34816, 5120, 128)       # one row: 68 x 7 = 476 workgroups, two rounds of six chunks
    assert rc == 0 and gemv_names[v] == "wided2m1t" and s == 7
    rc, v, s = _plan(L.awq_gemv_plan, 4, 51200, 5120, 128)       # 100 groups x 5 splits: two full rounds, also at four rows
    assert rc == 0 and gemv_names[v] == "wided2m1t" and s == 5
    rc, v, s = _plan(L.awq_gemv_plan, 1, 25600, 5120, 128)       # N < 28672: 256 columns, 100 groups x 5 splits
    assert rc == 0 and gemv_names[v] == "wide2d2m1t" and s == 5
    rc, v, s = _plan(L.awq_gemv_plan, 8, 25600, 5120, 128)       # the tail while rows x splits <= 64
    assert rc == 0 and gemv_names[v] == "wide2d2m1t" and s == 5
    rc, v, s = _plan(L.awq_gemv_plan, 4, 8192, 12288, 128)       # eleven splits or more for 500 workgroups: one per CU instead
    assert rc == 0 and gemv_names[v] == "wide2d3m1t" and s == 8
    rc, v, s = _plan(L.awq_gemv_plan, 16, 8192, 12288, 128)      # and the second pass beyond 64 rows x splits
    assert rc == 0 and gemv_names[v] == "wide2d3m1" and s == 8
    rc, v, s = _plan(L.awq_gemv_plan, 16, 24576, 4096, 128)      # 96 groups of 256 fill 75 % of the CUs in two splits: 512 columns
    assert rc == 0 and gemv_names[v] == "wided2m1" and s == 5
    rc, v, s = _plan(L.awq_gemv_plan, 32, 8192, 8192, 128)       # 17..32 rows: 256 columns x two m-tiles, one workgroup per CU
    assert rc == 0 and gemv_names[v] == "wide2d3m2" and s == 8
    rc, v, s = _plan(L.awq_gemv_plan, 24, 17408, 5120, 128)      # 68 groups: about 500 workgroups instead
    assert rc == 0 and gemv_names[v] == "wide2d2m2" and s == 7
    rc, v, s = _plan(L.awq_gemv_plan, 64, 8192, 8192, 128)       # 33..64 rows: 256 columns x four m-tiles, 32 groups x 8 splits
    assert rc == 0 and gemv_names[v] == "wide2d2m4" and s == 8
    rc, v, s = _plan(L.awq_gemv_plan, 48, 28672, 4096, 128)      # 112 groups: two splits would fill 87 % of the CUs, four it is
    assert rc == 0 and gemv_names[v] == "wide2d2m4" and s == 4
    rc, v, s = _plan(L.awq_gemv_plan, 64, 51200, 5120, 128)      # any N
    assert rc == 0 and gemv_names[v] == "wide2d2m4" and s == 2
    assert gemv_names[_plan(L.awq_gemv_plan, 48, 5120, 8192, 128)[1]] == "dma1x4"      # below 45 M weights: row blocks
    rc, v, s = _plan(L.awq_gemv_plan, 64, 5120, 8192, 128)       # from 40 M at 49..64 rows (four row blocks otherwise)
    assert rc == 0 and gemv_names[v] == "wide2d2m4" and s == 11
    rc, v, s = _plan(L.awq_gemv_plan, 48, 19456, 2560, 128)      # 20 chunks of K: four row blocks, and unsplit at 456 workgroups
    assert rc == 0 and gemv_names[v] == "dma1x4" and s == 1
    rc, v, s = _plan(L.awq_gemv_plan, 48, 6144, 2048, 128)       # a small weight in 144 workgroups: unsplit as well
    assert rc == 0 and gemv_names[v] == "dma1x4" and s == 1
    rc, v, s = _plan(L.awq_gemv_plan, 40, 5120, 17408, 128)      # 12 chunks a split would fill the CUs: 23 splits of 6 instead
    assert rc == 0 and gemv_names[v] == "wide2d2m4" and s == 23
    assert gemv_names[_plan(L.awq_gemv_plan, 1, 4096, 16384, 128)[1]] == "dma1x8"      # narrow weights: the one-tile kernel
    assert gemv_names[_plan(L.awq_gemv_plan, 8, 12288, 4096, 128)[1]] == "dma1x4"      # and small ones
    # narrow-tile GEMM (65..128 rows): the split fills whole rounds of the 512 resident workgroups (two per CU), so
    # 200 tiles are cut in two (400 workgroups, one round) or five (1000, two full rounds), never in three (600)
    rc, v, s = _plan(L.awq_gemm_plan, 128, 25600, 5120, 128, _lib.AWQ_BF16)
    assert rc == 0 and gemm_names[v] == "128x128" and s in (2, 5), s
    rc, v, s = _plan(L.awq_gemm_plan, 96, 5120, 25600, 128, _lib.AWQ_BF16)     # 40 tiles, 400 K steps: about 12 splits, one round
    assert rc == 0 and gemm_names[v] == "128x128" and 40 * s <= 512 and s >= 8, s
    # GEMV at up to four rows on a short K: one 128-row chunk per wave of the four-wave workgroups
    rc, v, s = _plan(L.awq_gemv_plan, 1, 1024, 2048, 128)
    assert rc == 0 and gemv_names[v] == "dma1x4" and s == 4, (gemv_names[v], s)
    # shapes awq_gemv does not take are refused by the plan as well
    assert _plan(L.awq_gemv_plan, 129, 1024, 1024, 128)[0] != 0
    # 65..128 rows: blocks of 16 rows on the one-tile staged kernels, unsplit once the blocks fill the chip
    rc, v, s = _plan(L.awq_gemv_plan, 128, 2048, 2048, 128)
    assert rc == 0 and gemv_names[v] == "dma1x4" and s == 1, (gemv_names[v], s)
    assert L.awq_gemv_workspace_bytes(128, 2048, 2048) <= L.awq_linear_workspace_bytes(128, 2048, 2048)
    assert _plan(L.awq_gemv_plan, 4, 1024, 1000, 128)[0] != 0
    assert _plan(L.awq_gemm_plan, 64, 1024, 96, 32, _lib.AWQ_BF16)[0] != 0
    # which 256 x 256 kernel: more items than CUs -> r in both types; exactly 256 items -> fp16 r, bf16 r only with 64
    # K steps per item or more; fewer -> p
    for (M, N, K, f16_name, bf16_name) in ((8192, 12288, 4096, "256x256r", "256x256r"),
                                           (4096, 4096, 1024, "256x256r", "256x256p"),
                                           (4096, 4096, 4096, "256x256r", "256x256r"),
                                           (1024, 4096, 1024, "256x256p", "256x256p")):
        assert gemm_names[_plan(L.awq_gemm_plan, M, N, K, 128, _lib.AWQ_F16)[1]] == f16_name, (M, N, K)
        assert gemm_names[_plan(L.awq_gemm_plan, M, N, K, 128, _lib.AWQ_BF16)[1]] == bf16_name, (M, N, K)
    # the register-operand kernel addresses a launch with 32-bit offsets: a packed weight of 2 GiB or a K whose 256
    # rows of x reach 2 GiB stay on the pipelined kernel
    assert gemm_names[_plan(L.awq_gemm_plan, 8192, 65536, 32768, 128, _lib.AWQ_F16)[1]].startswith("256x256r")
    assert gemm_names[_plan(L.awq_gemm_plan, 8192, 65536, 65536, 128, _lib.AWQ_F16)[1]].startswith("256x256p")


def test_every_entry_point_validates_before_touching_a_device():
    """Called with null pointers, every status-returning entry point reports an error (and says which function) without
    any device call: this runs on a machine with no GPU."""
    _ensure_built()
    L = _lib.lib()
    checked = 0
    for name, (res, args) in _lib.SYMBOLS.items():
        if res is not ctypes.c_int or not args or name == "awq_prefetch_hint":   # NULL clears the pending hints
            continue
        vals = []
        for a in args:
            if a is ctypes.c_float:
                vals.append(1e-6)
            elif a in (ctypes.c_int64, ctypes.c_size_t):
                vals.append(128)
            elif a is ctypes.c_int:
                vals.append(0)
            else:
                vals.append(None)
        rc = getattr(L, name)(*vals)
        msg = L.awq_hip_last_error().decode()
        assert rc != 0 and msg.split(":")[0] in (name, "awq_gemm", "awq_gemv"), (name, rc, msg)
        checked += 1
    assert checked >= 25
    assert L.awq_prefetch_hint(None, 0) == 0


def test_prefetch_hints_never_outlive_the_next_linear_call():
    """Hints are taken on entry of every linear entry point, before argument checks: a failing call (null pointers:
    no device needed) clears them, and a full queue ignores further regions instead of failing."""
    _ensure_built()
    L = _lib.lib()
    assert L.awq_prefetch_hint(None, 0) == 0
    fake = ctypes.c_void_p(1 << 20)   # never dereferenced on the host
    for entry in ("awq_gemv", "awq_gemm", "awq_linear", "awq_gemv_swiglu", "awq_linear_swiglu", "awq_gemv_ex",
                  "awq_gemm_ex", "awq_gemv_add_residual", "awq_gemv_rmsnorm"):
        for _ in range(6):
            assert L.awq_prefetch_hint(fake, 4096) == 0
        assert L.awq_prefetch_pending() == 4
        res, args = _lib.SYMBOLS[entry]
        vals = [1e-6 if a is ctypes.c_float else 128 if a in (ctypes.c_int64, ctypes.c_size_t) else 0
                if a is ctypes.c_int else None for a in args]
        assert getattr(L, entry)(*vals) != 0
        assert L.awq_prefetch_pending() == 0, entry


def test_superseded_workspaces_stay_alive():
    """A workspace that a captured graph may still point to is retired, never freed, when a larger one replaces it
    (bookkeeping only: allocation on the CPU through the test hook)."""
    dev = torch.device("cpu", 0)
    alloc = lambda n, dtype, device: torch.zeros(n, dtype=dtype)   # noqa: E731
    key_stream = 0x5eed
    before = len(_lib._retired_workspaces)
    a = _lib.workspace(dev, key_stream, 1 << 10, _alloc=alloc)
    assert a.numel() == 8 << 20 and _lib.workspace(dev, key_stream, 4 << 20, _alloc=alloc) is a
    b = _lib.workspace(dev, key_stream, 9 << 20, _alloc=alloc)
    assert b is not a and b.numel() == 9 << 20
    assert len(_lib._retired_workspaces) == before + 1 and _lib._retired_workspaces[-1] is a
    assert _lib.workspace(dev, key_stream, 1 << 10, _alloc=alloc) is b
    assert _lib.workspace(dev, key_stream, 0) is None
    del _lib._workspaces[(0, key_stream)]
    _lib._retired_workspaces.pop()


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asked for more it says so and exits non-zero before touching a device."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=300)
    assert p.returncode != 0 and "one GPU" in p.stderr and p.stdout.strip() == ""
