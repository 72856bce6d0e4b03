"""The decode-step kernels (include/nq_engine_ops.h) against plain torch fp32 restatements of the
module code they stand in for: nanoquantization/layers/norm.py:18-32, layers/rope.py:24-45,
models/qwen3_quantized.py:79-99 and :147-152.  Tolerances: one rounding step of the tensor type
(2^-8 relative for bf16, 2^-11 for fp16) on top of fp32 reduction-order noise."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DTYPES = [torch.bfloat16, torch.float16]


def _ulp(dtype):
    return 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11


def _close(got, want, dtype, scale=1.0, what=""):
    got, want = got.float(), want.float()
    err = (got - want).abs().max().item()
    ref = max(want.abs().max().item(), 1e-6)
    assert err <= 2.5 * _ulp(dtype) * ref * scale, f"{what}: max err {err} vs max |ref| {ref}"


def _rmsnorm_ref(x, w, eps):
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).to(x.dtype) * w


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,hidden", [(1, 1024), (32, 1024), (7, 5120), (3, 8192), (5, 136)])
def test_add_rmsnorm(dtype, rows, hidden):
    from nanoquantization_amd.engine import ops
    g = torch.Generator().manual_seed(rows * 131 + hidden)
    x = torch.randn(rows, hidden, generator=g).to(dtype).cuda()
    d = torch.randn(rows, hidden, generator=g).to(dtype).cuda()
    w = (1 + 0.1 * torch.randn(hidden, generator=g)).to(dtype).cuda()
    y0 = ops.add_rmsnorm(x.clone(), None, w, 1e-6)
    _close(y0, _rmsnorm_ref(x, w, 1e-6), dtype, what="norm only")
    res = x.clone()
    y1 = ops.add_rmsnorm(res, d, w, 1e-6)
    assert torch.equal(res, x + d), "the residual sum is one rounded add: bit-exact"
    _close(y1, _rmsnorm_ref(x + d, w, 1e-6), dtype, what="add + norm")


def test_add_rmsnorm_rejects_bad_shapes():
    from nanoquantization_amd import _lib
    from nanoquantization_amd.engine import ops
    w = torch.ones(8200, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(_lib.AwqHipError, match="exceeds"):
        ops.add_rmsnorm(torch.zeros(2, 8200, dtype=torch.bfloat16, device="cuda"), None, w, 1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,hd", [(16, 8, 128), (4, 4, 64), (8, 1, 256), (64, 8, 128),
                                       (6, 2, 96)])    # 96: the scalar kernel (head dims other than 64/128/256)
def test_qk_norm_rope_store(dtype, nh, nkv, hd):
    from nanoquantization_amd.engine import ops
    from nanoquantization_amd.layers.rope import RoPE
    rows, num_slots, max_pos = 37, 256, 512
    g = torch.Generator().manual_seed(nh * 7 + hd)
    qkv = torch.randn(rows, (nh + 2 * nkv) * hd, generator=g).to(dtype).cuda()
    qw = (1 + 0.1 * torch.randn(hd, generator=g)).to(dtype).cuda()
    kw = (1 + 0.1 * torch.randn(hd, generator=g)).to(dtype).cuda()
    pos = torch.randint(0, max_pos, (rows,), generator=g).cuda()
    slots = torch.randperm(num_slots, generator=g)[:rows].cuda()
    slots[5] = -1            # a row that owns no cache slot
    rope = RoPE(hd, max_pos).cuda()
    bs = 16
    kc = torch.zeros(num_slots // bs, nkv, bs, hd, dtype=dtype, device="cuda")   # [blocks, kv heads, block, hd]
    vc = torch.zeros_like(kc)
    q = ops.qk_norm_rope_store(qkv, qw, kw, rope.cos_sin_cache, pos, slots, kc, vc, nh, nkv, hd, 1e-6)
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
    q2, kd = ops.qk_norm_rope_store(qkv, qw, kw, rope.cos_sin_cache, pos, slots, kc2, vc2, nh, nkv, hd, 1e-6,
                                    dense_k=True)
    assert torch.equal(q2, q) and torch.equal(kc2, kc) and torch.equal(vc2, vc)

    qr, kr, vr = torch.split(qkv, [nh * hd, nkv * hd, nkv * hd], dim=-1)
    qr = _rmsnorm_ref(qr.view(rows, 1, nh, hd), qw, 1e-6)
    kr = _rmsnorm_ref(kr.view(rows, 1, nkv, hd), kw, 1e-6)
    qr, kr = rope(qr, kr, pos.view(rows, 1))
    _close(q, qr.view(rows, nh, hd), dtype, what="q")
    _close(kd, kr.view(rows, nkv, hd), dtype, what="dense k (every row, also the one without a slot)")
    keep = slots >= 0
    by_slot = lambda c: c.permute(0, 2, 1, 3).reshape(num_slots, nkv, hd)      # slot = block * bs + offset
    _close(by_slot(kc)[slots[keep]], kr.view(rows, nkv, hd)[keep], dtype, what="k cache")
    assert torch.equal(by_slot(vc)[slots[keep]], vr.reshape(rows, nkv, hd)[keep]), "v is copied bit for bit"
    untouched = torch.ones(num_slots, dtype=torch.bool, device="cuda")
    untouched[slots[keep]] = False
    assert not by_slot(kc)[untouched].any() and not by_slot(vc)[untouched].any(), "other slots must stay untouched"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,K,nh,nkv", [(1, 1024, 16, 8), (32, 1024, 16, 8), (64, 1024, 16, 8), (5, 3072, 4, 2),
                                        (40, 5120, 64, 8), (16, 2048, 8, 8), (64, 5120, 64, 8), (24, 5120, 64, 8),
                                        (16, 5120, 64, 8), (33, 4096, 32, 8)])
def test_gemv_qkv_rope_store_equals_unfused(dtype, M, K, nh, nkv):
    """Projection + q/k norm + rotary + cache write in one launch (the epilogue of the one-tile kernel or, from 17
    rows on the largest weights, of the shared-chunk kernel's second pass) against the GEMV followed by the
    stand-alone kernel: bit for bit (same summation order and rounding points), except where the plain projection
    runs another kernel with another summation order (up to 16 rows on the largest weights)."""
    import nanoquantization_amd as nq
    from nanoquantization_amd.engine import ops
    from nanoquantization_amd.layers.rope import RoPE
    hd, bs, max_pos = 128, 16, 512
    num_slots = 256
    N = (nh + 2 * nkv) * hd
    g = torch.Generator(device="cuda").manual_seed(M * 131 + K + nh)
    qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (K, N // 8), dtype=torch.int32, device="cuda", generator=g)
    qs = (torch.rand(K // 128, N, device="cuda", generator=g) * 0.02 + 0.001).to(dtype)
    qz = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 128, N // 8), dtype=torch.int32, device="cuda", generator=g)
    x = (torch.randn(M, K, device="cuda", generator=g) * 0.3).to(dtype)
    nqw = (1 + 0.1 * torch.randn(hd, device="cuda", generator=g)).to(dtype)
    nkw = (1 + 0.1 * torch.randn(hd, device="cuda", generator=g)).to(dtype)
    pos = torch.randint(0, max_pos, (M,), device="cuda", generator=g)
    slots = torch.randperm(num_slots, device="cuda", generator=g)[:M]
    if M > 3:
        slots[3] = -1
    rope = RoPE(hd, max_pos).cuda()
    print(f"gemv_qkv_rope_store M={M} K={K} nh={nh} nkv={nkv} {dtype}", flush=True)
    kc = torch.zeros(num_slots // bs, nkv, bs, hd, dtype=dtype, device="cuda")
    vc = torch.zeros_like(kc)
    q = ops.awq_gemv_qkv_rope_store(x, qw, qs, qz, nqw, nkw, rope.cos_sin_cache, pos, slots, kc, vc, nh, nkv, 1e-6)
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
    q2 = ops.qk_norm_rope_store(nq.awq_gemm(x, qw, qs, qz, 8), nqw, nkw, rope.cos_sin_cache, pos, slots, kc2, vc2,
                                nh, nkv, hd, 1e-6)
    import ctypes
    from nanoquantization_amd import _lib
    L = _lib.lib()
    pv, ps = ctypes.c_int(), ctypes.c_int()
    assert L.awq_gemv_plan(M, N, K, 128, ctypes.byref(pv), ctypes.byref(ps)) == 0
    plan = L.awq_gemv_variant_name(pv.value).decode()
    if plan.startswith("wide") and (M <= 16 or plan.endswith("t") or ps.value < 2):
        # the plain projection runs a shared-chunk kernel whose form the fused entry point does not take: another sum order
        assert (M, K) == (16, 5120)
        _close(vc, vc2.float(), dtype, what="v cache")
        _close(q, q2.float(), dtype, what="q")
        _close(kc, kc2.float(), dtype, what="k cache")
    else:
        assert torch.equal(vc, vc2), "v is the projection itself"
        assert torch.equal(q, q2) and torch.equal(kc, kc2)
    assert torch.equal(q, ops.awq_gemv_qkv_rope_store(x, qw, qs, qz, nqw, nkw, rope.cos_sin_cache, pos, slots,
                                                      torch.zeros_like(kc), torch.zeros_like(vc), nh, nkv, 1e-6))


def _attn_ref(q, kc, vc, table, ctx, scale):
    B, nh, hd = q.shape
    nb, nkv, bs, _ = kc.shape
    G = nh // nkv
    out = torch.empty(B, nh, hd, dtype=torch.float32, device=q.device)
    for b in range(B):
        n = int(ctx[b])
        t = torch.arange(n, device=q.device)
        blk, off = table[b, t // bs].long(), t % bs
        k = kc[blk, :, off].float().repeat_interleave(G, dim=1)               # [n, nh, hd]
        v = vc[blk, :, off].float().repeat_interleave(G, dim=1)
        s = torch.einsum("hd,nhd->hn", q[b].float(), k) * scale
        out[b] = torch.einsum("hn,nhd->hd", torch.softmax(s, dim=-1), v)
    return out.view(B, nh * hd)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,nh,nkv,hd,bs,max_blocks", [
    (32, 16, 8, 128, 64, 12),     # Qwen3-0.6B decode, context splits
    (3, 16, 8, 128, 16, 5),       # tiny context: fewer tokens than lanes
    (64, 64, 8, 128, 64, 4),      # 8 query heads per kv head
    (5, 4, 4, 64, 32, 9),         # head_dim 64, no grouping
    (130, 8, 8, 128, 64, 1),      # one block per sequence, single split
    (2, 4, 1, 128, 48, 7),        # block size that is not a power of two
    (8, 32, 8, 128, 64, 6),       # 4 query heads per kv head
    (4, 64, 8, 128, 64, 40),      # 8 per kv head, long context, context splits
    (9, 16, 2, 128, 16, 11),      # 8 per kv head, one tile per block
    (3, 8, 1, 128, 24, 5),        # 8 per kv head, block size not a multiple of the tile: the general kernel
    (6, 40, 8, 128, 64, 5),       # 5 per kv head (Qwen3-14B): the matrix-core kernel with the ratio at run time
    (3, 12, 4, 128, 32, 7),       # 3 per kv head
    (2, 16, 1, 128, 64, 4),       # 16 per kv head
    (5, 20, 4, 128, 16, 9),       # 5 per kv head, 16-token blocks: every tile of 32 tokens spans two blocks
    (4, 24, 4, 128, 48, 6),       # 6 per kv head, 48-token blocks: every third tile does
    (7, 64, 8, 128, 80, 5),       # 8 per kv head, 80-token blocks
])
def test_paged_attention_decode(dtype, B, nh, nkv, hd, bs, max_blocks):
    from nanoquantization_amd.engine import ops
    g = torch.Generator().manual_seed(B * 1000 + nh)
    nb = B * max_blocks + 3
    kc = torch.randn(nb, nkv, bs, hd, generator=g).to(dtype).cuda()
    vc = torch.randn(nb, nkv, bs, hd, generator=g).to(dtype).cuda()
    q = torch.randn(B, nh, hd, generator=g).to(dtype).cuda()
    table = torch.randperm(nb, generator=g)[: B * max_blocks].view(B, max_blocks).to(torch.int32).cuda()
    ctx = torch.randint(1, bs * max_blocks + 1, (B,), generator=g).to(torch.int32)
    ctx[0] = 1
    ctx[-1] = bs * max_blocks
    ctx = ctx.cuda()
    scale = 1.0 / math.sqrt(hd)
    out = ops.paged_attention_decode(q, kc, vc, table, ctx, scale)
    _close(out, _attn_ref(q, kc, vc, table, ctx, scale), dtype, scale=2.0, what="attention")
    assert torch.equal(out, ops.paged_attention_decode(q, kc, vc, table, ctx, scale)), "run-to-run bit-stable"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,bs", [(16, 8, 32), (64, 8, 32), (16, 4, 32), (40, 8, 32), (64, 8, 16), (40, 8, 48)])
def test_paged_attention_ignores_rows_past_the_context(dtype, nh, nkv, bs):
    """Cache rows past a sequence's context (and unused blocks) hold whatever was there before: NaNs planted there
    must not reach the output."""
    from nanoquantization_amd.engine import ops
    B, hd, max_blocks = 6, 128, -(-160 // bs)
    g = torch.Generator().manual_seed(nh)
    nb = B * max_blocks + 2
    table = torch.randperm(nb, generator=g)[: B * max_blocks].view(B, max_blocks).to(torch.int32)
    ctx = torch.tensor([1, 17, 32, 33, 100, 159], dtype=torch.int32)
    kc = torch.full((nb, nkv, bs, hd), float("nan"))
    vc = torch.full((nb, nkv, bs, hd), float("nan"))
    for b in range(B):
        t = torch.arange(int(ctx[b]))
        blk, off = table[b, t // bs].long(), t % bs
        kc[blk, :, off] = torch.randn(len(t), nkv, hd, generator=g)
        vc[blk, :, off] = torch.randn(len(t), nkv, hd, generator=g)
    kc, vc, table, ctx = kc.to(dtype).cuda(), vc.to(dtype).cuda(), table.cuda(), ctx.cuda()
    q = torch.randn(B, nh, hd, generator=g).to(dtype).cuda()
    scale = 1.0 / math.sqrt(hd)
    out = ops.paged_attention_decode(q, kc, vc, table, ctx, scale)
    assert torch.isfinite(out.float()).all()
    _close(out, _attn_ref(q, kc, vc, table, ctx, scale), dtype, scale=2.0, what="attention")


def test_paged_attention_rejects_unsupported():
    from nanoquantization_amd import _lib
    from nanoquantization_amd.engine import ops
    kc = torch.zeros(4, 1, 24, 128, dtype=torch.bfloat16, device="cuda")   # 3 per kv head needs 16 | block size
    q = torch.zeros(1, 3, 128, dtype=torch.bfloat16, device="cuda")
    tb = torch.zeros(1, 2, dtype=torch.int32, device="cuda")
    cx = torch.ones(1, dtype=torch.int32, device="cuda")
    with pytest.raises(_lib.AwqHipError, match="1, 2, 4 or 8"):
        ops.paged_attention_decode(q, kc, kc, tb, cx, 1.0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,inter", [(1, 3072), (32, 3072), (9, 25600), (3, 8)])
def test_silu_mul(dtype, rows, inter):
    import torch.nn.functional as F
    from nanoquantization_amd.engine import ops
    g = torch.Generator().manual_seed(rows + inter)
    gu = (2 * torch.randn(rows, 2 * inter, generator=g)).to(dtype).cuda()
    _close(ops.silu_mul(gu), F.silu(gu[:, :inter]) * gu[:, inter:], dtype, what="silu*up")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,K,inter", [(1, 1024, 3072), (32, 1024, 3072), (16, 2048, 1024), (64, 5120, 1280), (3, 4096, 64),
                                           (48, 4096, 3072), (24, 8192, 2560), (64, 8192, 4096), (40, 5120, 8704)])
# (from 24 rows x 8192 on: the shared-chunk kernel, whose second pass applies the gate)
def test_gemv_swiglu_equals_unfused(dtype, M, K, inter):
    """Gate and up interleaved + gated epilogue must give, bit for bit, what the plain GEMV over gate|up side by
    side followed by the SiLU*up kernel gives (a column's sum does not depend on where the column sits)."""
    import nanoquantization_amd as nq
    from nanoquantization_amd.engine import ops
    g = torch.Generator(device="cuda").manual_seed(M * 31 + K + inter)
    def packed(n):
        return (torch.randint(-2 ** 31, 2 ** 31 - 1, (K, n // 8), dtype=torch.int32, device="cuda", generator=g),
                (torch.rand(K // 128, n, device="cuda", generator=g) * 0.02 + 0.001).to(dtype),
                torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 128, n // 8), dtype=torch.int32, device="cuda", generator=g))
    gate, up = packed(inter), packed(inter)
    x = torch.randn(M, K, device="cuda", generator=g).to(dtype)
    print(f"gemv_swiglu M={M} K={K} inter={inter} {dtype}", flush=True)
    fused = ops.awq_gemv_swiglu(x, *ops.interleave_gate_up(gate, up))
    side = [torch.cat([a, b], dim=1).contiguous() for a, b in zip(gate, up)]
    ref = ops.silu_mul(nq.awq_gemm(x, side[0], side[1], side[2], 8))
    assert fused.shape == (M, inter)
    assert torch.equal(fused, ref)


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul_interleaved_equals_side_by_side(dtype):
    from nanoquantization_amd.engine import ops
    g = torch.Generator(device="cuda").manual_seed(5)
    rows, inter = 37, 3072
    gate = torch.randn(rows, inter, device="cuda", generator=g).to(dtype)
    up = torch.randn(rows, inter, device="cuda", generator=g).to(dtype)
    il = torch.stack([gate.view(rows, inter // 8, 8), up.view(rows, inter // 8, 8)], dim=2).reshape(rows, 2 * inter)
    assert torch.equal(ops.silu_mul(il.contiguous(), interleaved=True), ops.silu_mul(torch.cat([gate, up], dim=1)))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,K,inter", [(65, 1024, 3072), (300, 1024, 3072), (1000, 2048, 1032), (4100, 1024, 8192),
                                       (130, 256, 8)])
def test_gemm_swiglu_equals_unfused(dtype, M, K, inter):
    """Above the GEMV regime the gate runs in the GEMM's epilogue (whole tiles and K-split tiles alike): bit for bit
    what the plain GEMM over gate|up side by side followed by the SiLU*up kernel gives."""
    import nanoquantization_amd as nq
    from nanoquantization_amd.engine import ops
    g = torch.Generator(device="cuda").manual_seed(M * 31 + K + inter)
    def packed(n):
        return (torch.randint(-2 ** 31, 2 ** 31 - 1, (K, n // 8), dtype=torch.int32, device="cuda", generator=g),
                (torch.rand(K // 128, n, device="cuda", generator=g) * 0.02 + 0.001).to(dtype),
                torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 128, n // 8), dtype=torch.int32, device="cuda", generator=g))
    gate, up = packed(inter), packed(inter)
    x = torch.randn(M, K, device="cuda", generator=g).to(dtype)
    print(f"gemm_swiglu M={M} K={K} inter={inter} {dtype}", flush=True)
    fused = ops.awq_linear_swiglu(x, *ops.interleave_gate_up(gate, up))
    side = [torch.cat([a, b], dim=1).contiguous() for a, b in zip(gate, up)]
    if M > 128:
        ref_lin = nq.awq_gemm(x, side[0], side[1], side[2], 8)      # same kernel and K split as the fused call
    else:
        # up to 128 rows the plain dispatch takes a narrower tile; force the pipelined kernel with its split rule
        from nanoquantization_amd import _lib
        from nanoquantization_amd.layers.gemm import awq_gemm_variant
        L = _lib.lib()
        names = [L.awq_gemm_variant_name(i).decode() for i in range(L.awq_gemm_variant_count())]
        tiles = (2 * inter + 255) // 256
        split = max(1, min(256 // tiles, max(1, K // 64 // 8), 16))
        ref_lin = awq_gemm_variant(x, side[0], side[1], side[2], names.index("256x256p"), split)
    ref = ops.silu_mul(ref_lin)
    assert fused.shape == (M, inter)
    assert torch.equal(fused, ref)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,vocab", [(1, 8), (3, 1000), (32, 151936), (5, 151943), (2, 7)])
def test_argmax_rows(dtype, rows, vocab):
    from nanoquantization_amd.engine import ops
    print(f"argmax_rows {dtype} rows={rows} vocab={vocab}", flush=True)
    g = torch.Generator(device="cuda").manual_seed(rows + vocab)
    logits = torch.randn(rows, vocab, device="cuda", generator=g).to(dtype)
    out = ops.argmax_rows(logits)
    assert out.dtype == torch.int64 and tuple(out.shape) == (rows,)
    # 16-bit logits tie often: the winner must hold the maximum and be the first to do so
    mx = logits.float().max(dim=1).values
    first = (logits.float() == mx[:, None]).float().argmax(dim=1)
    assert torch.equal(out, first)
    # planted ties and extremes
    logits[0, :] = -float("inf")
    assert ops.argmax_rows(logits)[0].item() == 0
    logits[0, vocab - 1] = 3.0
    logits[0, vocab // 2] = 3.0
    assert ops.argmax_rows(logits)[0].item() == vocab // 2


def _packed(K, N, dtype, g):
    qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (K, N // 8), dtype=torch.int32, device="cuda", generator=g)
    qs = (torch.rand(K // 128, N, device="cuda", generator=g) * 0.02 + 0.001).to(dtype)
    qz = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 128, N // 8), dtype=torch.int32, device="cuda", generator=g)
    return qw, qs, qz


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,hidden", [(1, 1024), (32, 1024), (7, 5120), (3, 8192), (5, 136)])
def test_row_ssq(dtype, rows, hidden):
    """Tile sums of squares against torch (fp32, a few ulps: another summation order)."""
    from nanoquantization_amd.engine import ops
    g = torch.Generator(device="cuda").manual_seed(rows + hidden)
    x = torch.randn(rows, hidden, device="cuda", generator=g).to(dtype)
    ssq = ops.row_ssq(x)
    tiles = (hidden + 127) // 128
    assert ssq.shape == (tiles, rows) and ssq.dtype == torch.float32
    pad = torch.zeros(rows, tiles * 128, device="cuda")
    pad[:, :hidden] = x.float()
    want = pad.view(rows, tiles, 128).double().pow(2).sum(-1).t()
    assert torch.allclose(ssq.double(), want, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,K,N", [(1, 2048, 1024), (32, 2048, 1024), (16, 3072, 1024), (64, 1024, 5120),
                                   (5, 8192, 256), (33, 25600, 1024)])
def test_gemv_add_residual_equals_unfused(dtype, M, K, N):
    """o_proj / down_proj with the residual addition and the RMSNorm statistics in the epilogue against the GEMV
    followed by the add + norm kernel: residual stream and statistics bit for bit."""
    import nanoquantization_amd as nq
    from nanoquantization_amd.engine import ops
    g = torch.Generator(device="cuda").manual_seed(M * 7 + K + N)
    qw, qs, qz = _packed(K, N, dtype, g)
    x = (torch.randn(M, K, device="cuda", generator=g) * 0.3).to(dtype)
    res = torch.randn(M, N, device="cuda", generator=g).to(dtype)
    print(f"gemv_add_residual M={M} K={K} N={N} {dtype}", flush=True)
    want = res.clone()
    w = torch.ones(N, dtype=dtype, device="cuda")
    ops.add_rmsnorm(want, nq.awq_gemm(x, qw, qs, qz, 8), w, 1e-6)     # updates `want` in place
    got = res.clone()
    ssq = torch.full((N // 128, M), float("nan"), device="cuda")
    ops.awq_gemv_add_residual(x, qw, qs, qz, got, ssq)
    assert torch.equal(got, want)
    assert torch.equal(ssq, ops.row_ssq(want))
    again = res.clone()
    ssq2 = torch.empty_like(ssq)
    ops.awq_gemv_add_residual(x, qw, qs, qz, again, ssq2)              # workspace counters were left clean
    assert torch.equal(again, got) and torch.equal(ssq2, ssq)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,K,N", [(64, 8192, 5120), (64, 25600, 5120), (33, 12288, 4096), (17, 12288, 4096),
                                   (64, 8192, 8192), (48, 16384, 3584)])
def test_gemv_add_rmsnorm_equals_unfused(dtype, M, K, N):
    """The residual add and the RMSNorm after o_proj / down_proj inside the second pass of a K-split shared-chunk
    GEMV (Qwen3-32B and 8B shapes at 17..64 rows) against the GEMV, then the add + norm kernel: residual stream and
    normalised output bit for bit, twice in a row; shapes without such a plan are refused."""
    import nanoquantization_amd as nq
    from nanoquantization_amd import _lib
    from nanoquantization_amd.engine import ops
    g = torch.Generator(device="cuda").manual_seed(M * 11 + K + N)
    qw, qs, qz = _packed(K, N, dtype, g)
    x = (torch.randn(M, K, device="cuda", generator=g) * 0.3).to(dtype)
    res = torch.randn(M, N, device="cuda", generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(N, device="cuda", generator=g)).to(dtype)
    print(f"gemv_add_rmsnorm M={M} K={K} N={N} {dtype}", flush=True)
    assert ops.gemv_add_rmsnorm_supported(M, N, K, 128)
    want_res = res.clone()
    want = ops.add_rmsnorm(want_res, nq.awq_gemm(x, qw, qs, qz, 8), w, 1e-6)     # updates `want_res` in place
    for _ in range(2):
        got_res = res.clone()
        got = ops.awq_gemv_add_rmsnorm(x, qw, qs, qz, got_res, w, 1e-6)
        assert torch.equal(got_res, want_res)
        assert torch.equal(got, want)
    # one row on the same weight: the in-kernel tail or the one-tile kernel, no second pass to put the norm in
    assert not ops.gemv_add_rmsnorm_supported(1, N, K, 128)
    with pytest.raises(_lib.AwqHipError, match="second pass"):
        ops.awq_gemv_add_rmsnorm(x[:1].contiguous(), qw, qs, qz, res[:1].clone(), w, 1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,K,N,gated", [(1, 1024, 4096, False), (32, 1024, 6144, True), (16, 2048, 2048, True),
                                         (64, 1024, 4096, False), (7, 5120, 1280, True), (40, 4096, 512, False)])
def test_gemv_rmsnorm_equals_unfused(dtype, M, K, N, gated):
    """RMSNorm in the GEMV's prologue against the norm kernel followed by the plain (or gated) GEMV: bit for bit."""
    import nanoquantization_amd as nq
    from nanoquantization_amd.engine import ops
    g = torch.Generator(device="cuda").manual_seed(M * 11 + K + N)
    qw, qs, qz = _packed(K, N, dtype, g)
    x = torch.randn(M, K, device="cuda", generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(K, device="cuda", generator=g)).to(dtype)
    print(f"gemv_rmsnorm M={M} K={K} N={N} gated={gated} {dtype}", flush=True)
    h = ops.add_rmsnorm(x.clone(), None, w, 1e-6)
    want = ops.awq_gemv_swiglu(h, qw, qs, qz) if gated else nq.awq_gemm(h, qw, qs, qz, 8)
    got = ops.awq_gemv_rmsnorm(x, ops.row_ssq(x), w, 1e-6, qw, qs, qz, gated=gated)
    assert torch.equal(got, want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,K,nh,nkv", [(1, 1024, 16, 8), (32, 1024, 16, 8), (64, 2048, 4, 2)])
def test_gemv_rmsnorm_qkv_rope_store_equals_unfused(dtype, M, K, nh, nkv):
    from nanoquantization_amd.engine import ops
    from nanoquantization_amd.layers.rope import RoPE
    hd, bs, max_pos, num_slots = 128, 16, 512, 256
    N = (nh + 2 * nkv) * hd
    g = torch.Generator(device="cuda").manual_seed(M * 17 + K + nh)
    qw, qs, qz = _packed(K, N, dtype, g)
    x = torch.randn(M, K, device="cuda", generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(K, device="cuda", generator=g)).to(dtype)
    nqw = (1 + 0.1 * torch.randn(hd, device="cuda", generator=g)).to(dtype)
    nkw = (1 + 0.1 * torch.randn(hd, device="cuda", generator=g)).to(dtype)
    pos = torch.randint(0, max_pos, (M,), device="cuda", generator=g)
    slots = torch.randperm(num_slots, device="cuda", generator=g)[:M]
    rope = RoPE(hd, max_pos).cuda()
    print(f"gemv_rmsnorm_qkv_rope_store M={M} K={K} nh={nh} nkv={nkv} {dtype}", flush=True)
    kc = torch.zeros(num_slots // bs, nkv, bs, hd, dtype=dtype, device="cuda")
    vc, kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(kc), torch.zeros_like(kc)
    h = ops.add_rmsnorm(x.clone(), None, w, 1e-6)
    q2 = ops.awq_gemv_qkv_rope_store(h, qw, qs, qz, nqw, nkw, rope.cos_sin_cache, pos, slots, kc2, vc2, nh, nkv, 1e-6)
    q = ops.awq_gemv_rmsnorm_qkv_rope_store(x, ops.row_ssq(x), w, 1e-6, qw, qs, qz, nqw, nkw, rope.cos_sin_cache, pos,
                                            slots, kc, vc, nh, nkv, 1e-6)
    assert torch.equal(q, q2) and torch.equal(kc, kc2) and torch.equal(vc, vc2)


def test_norm_fused_entry_points_reject_unsupported():
    from nanoquantization_amd import _lib
    from nanoquantization_amd.engine import ops
    g = torch.Generator(device="cuda").manual_seed(5)
    K, N = 256, 136                                     # N is not a multiple of 128: no staged kernel
    qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (K, N // 8), dtype=torch.int32, device="cuda", generator=g)
    qs = torch.rand(K // 128, N, device="cuda", generator=g).half()
    qz = torch.zeros(K // 128, N // 8, dtype=torch.int32, device="cuda")
    x = torch.randn(4, K, device="cuda", generator=g).half()
    with pytest.raises(_lib.AwqHipError):
        ops.awq_gemv_rmsnorm(x, ops.row_ssq(x), torch.ones(K, dtype=torch.half, device="cuda"), 1e-6, qw, qs, qz)


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_fused_forms_on_largest_decode_shapes(dtype):
    """Qwen3-32B widths at 64 rows, where the plain GEMV runs the shared-chunk kernel (another summation order) and
    the fused forms stay on the row-block kernel: results within one rounding step of the separate kernels, the
    statistics exactly those of the residual that was stored."""
    import nanoquantization_amd as nq
    from nanoquantization_amd.engine import ops
    M = 64
    g = torch.Generator(device="cuda").manual_seed(64)
    # down_proj 25600 -> 5120 with the residual epilogue
    K, N = 25600, 5120
    qw, qs, qz = _packed(K, N, dtype, g)
    x = (torch.randn(M, K, device="cuda", generator=g) * 0.1).to(dtype)
    res = torch.randn(M, N, device="cuda", generator=g).to(dtype)
    print(f"norm-fused forms at 32B widths {dtype}", flush=True)
    want = res.clone()
    ops.add_rmsnorm(want, nq.awq_gemm(x, qw, qs, qz, 8), torch.ones(N, dtype=dtype, device="cuda"), 1e-6)
    got = res.clone()
    ssq = torch.empty(N // 128, M, device="cuda")
    ops.awq_gemv_add_residual(x, qw, qs, qz, got, ssq)
    _close(got, want.float(), dtype, what="residual")
    assert torch.equal(ssq, ops.row_ssq(got))
    # fused gate|up 5120 -> 2 x 25600 with the RMSNorm prologue
    K, N = 5120, 51200
    qw, qs, qz = _packed(K, N, dtype, g)
    xr = torch.randn(M, K, device="cuda", generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(K, device="cuda", generator=g)).to(dtype)
    want = ops.awq_gemv_swiglu(ops.add_rmsnorm(xr.clone(), None, w, 1e-6), qw, qs, qz)
    got = ops.awq_gemv_rmsnorm(xr, ops.row_ssq(xr), w, 1e-6, qw, qs, qz, gated=True)
    _close(got, want.float(), dtype, what="gated product")


def test_decode_prepare_and_advance():
    """The step's bookkeeping kernels against the torch expressions they stand in for."""
    from nanoquantization_amd.engine import ops
    g = torch.Generator().manual_seed(9)
    rows, max_blocks, bs = 37, 6, 16
    pos = torch.randint(0, max_blocks * bs, (rows,), generator=g).cuda()
    active = (torch.rand(rows, generator=g) > 0.3).cuda()
    table = torch.randint(0, 500, (rows, max_blocks), generator=g).to(torch.int32).cuda()
    slots, ctx = ops.decode_prepare(pos, active, table, bs)
    blk = table.gather(1, (pos // bs).unsqueeze(1)).squeeze(1).long()
    assert torch.equal(slots, torch.where(active, blk * bs + pos % bs, torch.full_like(pos, -1)))
    assert torch.equal(ctx, (pos + 1).to(torch.int32))
    out = torch.full((5, rows), -7, dtype=torch.long, device="cuda")
    ids = torch.zeros(rows, dtype=torch.long, device="cuda")
    step = torch.tensor([3], device="cuda")
    nxt = torch.randint(0, 1000, (rows,), generator=g).cuda()
    pos0 = pos.clone()
    ops.decode_advance(nxt, active, out, ids, pos, step)
    assert torch.equal(out[3], nxt) and (out[[0, 1, 2, 4]] == -7).all()
    assert torch.equal(ids, nxt) and torch.equal(pos, pos0 + active.long()) and step.item() == 4
    ops.decode_advance(nxt, active, out, ids, pos, step)
    ops.decode_advance(nxt, active, out, ids, pos, step)          # step 5 is past the log: nothing is written there
    assert step.item() == 6 and torch.equal(out[4], nxt) and torch.equal(pos, pos0 + 3 * active.long())


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed_row_ssq(dtype):
    from nanoquantization_amd.engine import ops
    g = torch.Generator(device="cuda").manual_seed(21)
    table = torch.randn(1000, 1024, device="cuda", generator=g).to(dtype)
    ids = torch.randint(0, 1000, (33,), device="cuda", generator=g)
    x, ssq = ops.embed_row_ssq(ids, table)
    assert torch.equal(x, table[ids]) and torch.equal(ssq, ops.row_ssq(table[ids].contiguous()))
