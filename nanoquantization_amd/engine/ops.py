"""torch-tensor wrappers of the decode-step kernels declared in include/nq_engine_ops.h.

Each function checks shapes on the host, allocates its output with torch (graph-capture safe:
the caching allocator) and launches on the current stream.  HIP device tensors only."""
from __future__ import annotations

from typing import Optional

import torch

from .. import _lib


def _dev(*ts: torch.Tensor) -> torch.device:
    dev = ts[0].device
    if dev.type != "cuda":
        raise _lib.AwqHipError(f"engine kernels run on a HIP device only (tensor is on {dev})")
    for t in ts:
        if t is not None and t.device != dev:
            raise _lib.AwqHipError(f"tensors on different devices: {t.device} vs {dev}")
        if t is not None and not t.is_contiguous():
            raise _lib.AwqHipError("engine kernels take contiguous tensors")
    return dev


def _stream(dev: torch.device) -> int:
    return _lib.current_stream_ptr(dev)


def add_rmsnorm(residual: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float) -> torch.Tensor:
    """residual [rows, hidden] += delta IN PLACE (if given); returns RMSNorm(residual) * weight."""
    dev = _dev(residual, weight) if delta is None else _dev(residual, delta, weight)
    rows, hidden = residual.shape
    assert weight.shape == (hidden,) and weight.dtype == residual.dtype
    assert delta is None or (delta.shape == residual.shape and delta.dtype == residual.dtype)
    y = torch.empty_like(residual)
    with _lib.on_device(dev):
        _lib.check(_lib.lib().nq_add_rmsnorm(residual.data_ptr(), None if delta is None else delta.data_ptr(),
                                             weight.data_ptr(), y.data_ptr(), rows, hidden, eps,
                                             _lib.dtype_id(residual.dtype), _stream(dev)))
    return y


def qk_norm_rope_store(qkv: torch.Tensor, q_weight: torch.Tensor, k_weight: torch.Tensor, cos_sin: torch.Tensor,
                       positions: torch.Tensor, slots: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                       num_heads: int, num_kv_heads: int, head_dim: int, eps: float, dense_k: bool = False):
    """qkv [rows, (nh + 2 nkv) * hd]; caches [blocks, nkv, block_size, hd]; returns q [rows, nh, hd], or
    (q, k [rows, nkv, hd]) with dense_k."""
    dev = _dev(qkv, q_weight, k_weight, cos_sin, positions, slots, k_cache, v_cache)
    rows = qkv.shape[0]
    assert qkv.shape[1] == (num_heads + 2 * num_kv_heads) * head_dim
    assert q_weight.shape == (head_dim,) and k_weight.shape == (head_dim,)
    assert q_weight.dtype == qkv.dtype and k_weight.dtype == qkv.dtype
    assert k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype and k_cache.shape == v_cache.shape
    assert k_cache.dim() == 4 and k_cache.shape[1] == num_kv_heads and k_cache.shape[3] == head_dim
    block_size = k_cache.shape[2]
    assert cos_sin.dtype == torch.float32 and cos_sin.numel() % head_dim == 0
    assert positions.dtype == torch.int64 and slots.dtype == torch.int64
    assert positions.numel() == rows and slots.numel() == rows
    num_slots = k_cache.numel() // (num_kv_heads * head_dim)
    q = torch.empty(rows, num_heads, head_dim, dtype=qkv.dtype, device=dev)
    k = torch.empty(rows, num_kv_heads, head_dim, dtype=qkv.dtype, device=dev) if dense_k else None
    with _lib.on_device(dev):
        _lib.check(_lib.lib().nq_qk_norm_rope_store(
            qkv.data_ptr(), q_weight.data_ptr(), k_weight.data_ptr(), cos_sin.data_ptr(), positions.data_ptr(),
            slots.data_ptr(), q.data_ptr(), None if k is None else k.data_ptr(), k_cache.data_ptr(),
            v_cache.data_ptr(), rows, num_heads, num_kv_heads,
            head_dim, cos_sin.numel() // head_dim, num_slots, block_size, eps, _lib.dtype_id(qkv.dtype), _stream(dev)))
    return (q, k) if dense_k else q


def awq_gemv_qkv_rope_store(x: torch.Tensor, qweight: torch.Tensor, qscales: torch.Tensor, qzeros: torch.Tensor,
                            q_weight: torch.Tensor, k_weight: torch.Tensor, cos_sin: torch.Tensor,
                            positions: torch.Tensor, slots: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                            num_heads: int, num_kv_heads: int, eps: float) -> torch.Tensor:
    """Fused q|k|v projection of x [M <= 64, K] + q/k RMSNorm + rotary + cache write (head_dim 128): returns
    q [M, nh, 128]; k and v go to their cache slots."""
    dev = _dev(x, qweight, qscales, qzeros, q_weight, k_weight, cos_sin, positions, slots, k_cache, v_cache)
    M, K = x.shape
    N = qscales.shape[1]
    g = K // qscales.shape[0]
    hd = 128
    assert N == (num_heads + 2 * num_kv_heads) * hd
    assert qweight.shape == (K, N // 8) and qzeros.shape == (K // g, N // 8) and x.dtype == qscales.dtype
    assert q_weight.shape == (hd,) and k_weight.shape == (hd,) and q_weight.dtype == x.dtype and k_weight.dtype == x.dtype
    assert k_cache.dtype == x.dtype and v_cache.dtype == x.dtype and k_cache.shape == v_cache.shape
    assert k_cache.dim() == 4 and k_cache.shape[1] == num_kv_heads and k_cache.shape[3] == hd
    assert cos_sin.dtype == torch.float32 and cos_sin.numel() % hd == 0
    assert positions.dtype == torch.int64 and slots.dtype == torch.int64 and positions.numel() == M and slots.numel() == M
    block_size = k_cache.shape[2]
    num_slots = k_cache.numel() // (num_kv_heads * hd)
    q = torch.empty(M, num_heads, hd, dtype=x.dtype, device=dev)
    L = _lib.lib()
    with _lib.on_device(dev):
        stream = _stream(dev)
        nbytes = L.awq_gemv_workspace_bytes(M, N, K)
        ws = _lib.workspace(dev, stream, nbytes)
        _lib.check(L.awq_gemv_qkv_rope_store(
            x.data_ptr(), qweight.data_ptr(), qscales.data_ptr(), qzeros.data_ptr(), q_weight.data_ptr(),
            k_weight.data_ptr(), cos_sin.data_ptr(), positions.data_ptr(), slots.data_ptr(), q.data_ptr(),
            k_cache.data_ptr(), v_cache.data_ptr(), M, N, K, g, num_heads, num_kv_heads, cos_sin.numel() // hd,
            num_slots, block_size, eps, _lib.dtype_id(x.dtype), None if ws is None else ws.data_ptr(),
            0 if ws is None else ws.numel(), stream))
    return q


def row_ssq(x: torch.Tensor) -> torch.Tensor:
    """x [rows, hidden] -> fp32 [ceil(hidden / 128), rows]: the sum of squares of every 128-column tile of every row,
    the RMSNorm statistics awq_gemv_rmsnorm reads."""
    dev = _dev(x)
    rows, hidden = x.shape
    ssq = torch.empty((hidden + 127) // 128, rows, dtype=torch.float32, device=dev)
    with _lib.on_device(dev):
        _lib.check(_lib.lib().nq_row_ssq(x.data_ptr(), ssq.data_ptr(), rows, hidden, _lib.dtype_id(x.dtype), _stream(dev)))
    return ssq


def embed_row_ssq(ids: torch.Tensor, table: torch.Tensor):
    """ids int64 [rows], table [vocab, hidden] -> (x [rows, hidden] = table[ids], its row_ssq)."""
    dev = _dev(ids, table)
    rows, (vocab, hidden) = ids.numel(), table.shape
    assert ids.dtype == torch.int64
    x = torch.empty(rows, hidden, dtype=table.dtype, device=dev)
    ssq = torch.empty((hidden + 127) // 128, rows, dtype=torch.float32, device=dev)
    with _lib.on_device(dev):
        _lib.check(_lib.lib().nq_embed_row_ssq(ids.data_ptr(), table.data_ptr(), x.data_ptr(), ssq.data_ptr(), rows, hidden,
                                               vocab, _lib.dtype_id(table.dtype), _stream(dev)))
    return x, ssq


def _gemv_ws(dev, M, N, K):
    stream = _stream(dev)
    ws = _lib.workspace(dev, stream, _lib.lib().awq_gemv_workspace_bytes(M, N, K))
    return (None if ws is None else ws.data_ptr()), (0 if ws is None else ws.numel()), stream


def awq_gemv_add_residual(x: torch.Tensor, qweight: torch.Tensor, qscales: torch.Tensor, qzeros: torch.Tensor,
                          residual: torch.Tensor, ssq: torch.Tensor) -> None:
    """residual [M <= 64, N] += x @ W IN PLACE (rounded like a linear followed by an addition); ssq [N / 128, M]
    receives the tile sums of squares of the new residual."""
    dev = _dev(x, qweight, qscales, qzeros, residual, ssq)
    M, K = x.shape
    N = qscales.shape[1]
    g = K // qscales.shape[0]
    assert qweight.shape == (K, N // 8) and qzeros.shape == (K // g, N // 8) and x.dtype == qscales.dtype
    assert residual.shape == (M, N) and residual.dtype == x.dtype
    assert ssq.shape == (N // 128, M) and ssq.dtype == torch.float32 and N % 128 == 0
    with _lib.on_device(dev):
        ws, ws_bytes, stream = _gemv_ws(dev, M, N, K)
        _lib.check(_lib.lib().awq_gemv_add_residual(x.data_ptr(), qweight.data_ptr(), qscales.data_ptr(),
                                                    qzeros.data_ptr(), residual.data_ptr(), ssq.data_ptr(), M, N, K, g,
                                                    _lib.dtype_id(x.dtype), ws, ws_bytes, stream))


def gemv_add_rmsnorm_supported(M: int, N: int, K: int, group_size: int) -> bool:
    """Whether awq_gemv_add_rmsnorm takes this problem: its GEMV plan is a shared-chunk variant whose K splits a
    second pass adds (that pass is what does the residual add and the norm), and N <= 8192."""
    import ctypes
    L = _lib.lib()
    v, s = ctypes.c_int(-1), ctypes.c_int(-1)
    if N > 8192 or N % 128 or L.awq_gemv_plan(M, N, K, group_size, ctypes.byref(v), ctypes.byref(s)) != 0:
        return False
    name = L.awq_gemv_variant_name(v.value).decode()
    return name.startswith("wide") and not name.endswith("t") and s.value > 1


def awq_gemv_add_rmsnorm(x: torch.Tensor, qweight: torch.Tensor, qscales: torch.Tensor, qzeros: torch.Tensor,
                         residual: torch.Tensor, norm_weight: torch.Tensor, eps: float) -> torch.Tensor:
    """residual [M <= 64, N] += x @ W IN PLACE and returns RMSNorm(residual) * norm_weight: a linear, the residual add
    and the norm that follow it in a Qwen3 block, the last two inside the GEMV's second pass (the bits of the three
    separate launches).  Only where gemv_add_rmsnorm_supported."""
    dev = _dev(x, qweight, qscales, qzeros, residual, norm_weight)
    M, K = x.shape
    N = qscales.shape[1]
    g = K // qscales.shape[0]
    assert qweight.shape == (K, N // 8) and qzeros.shape == (K // g, N // 8) and x.dtype == qscales.dtype
    assert residual.shape == (M, N) and residual.dtype == x.dtype and residual.is_contiguous()
    assert norm_weight.shape == (N,) and norm_weight.dtype == x.dtype
    out = torch.empty_like(residual)
    with _lib.on_device(dev):
        ws, ws_bytes, stream = _gemv_ws(dev, M, N, K)
        _lib.check(_lib.lib().awq_gemv_add_rmsnorm(x.data_ptr(), qweight.data_ptr(), qscales.data_ptr(), qzeros.data_ptr(),
                                                   residual.data_ptr(), norm_weight.data_ptr(), eps, out.data_ptr(), M, N,
                                                   K, g, _lib.dtype_id(x.dtype), ws, ws_bytes, stream))
    return out


def awq_gemv_rmsnorm(x: torch.Tensor, ssq: torch.Tensor, norm_weight: torch.Tensor, eps: float, qweight: torch.Tensor,
                     qscales: torch.Tensor, qzeros: torch.Tensor, gated: bool = False) -> torch.Tensor:
    """(RMSNorm(x) * norm_weight) @ W for the residual stream x [M <= 64, K] with its statistics ssq [K / 128, M];
    gated: interleaved gate|up buffers, returns SiLU(gate) * up [M, N / 2]."""
    dev = _dev(x, ssq, norm_weight, qweight, qscales, qzeros)
    M, K = x.shape
    N = qscales.shape[1]
    g = K // qscales.shape[0]
    assert qweight.shape == (K, N // 8) and qzeros.shape == (K // g, N // 8) and x.dtype == qscales.dtype
    assert K % 128 == 0 and ssq.shape == (K // 128, M) and ssq.dtype == torch.float32
    assert norm_weight.shape == (K,) and norm_weight.dtype == x.dtype
    out = torch.empty(M, N // 2 if gated else N, dtype=x.dtype, device=dev)
    with _lib.on_device(dev):
        ws, ws_bytes, stream = _gemv_ws(dev, M, N, K)
        _lib.check(_lib.lib().awq_gemv_rmsnorm(x.data_ptr(), ssq.data_ptr(), norm_weight.data_ptr(), eps,
                                               qweight.data_ptr(), qscales.data_ptr(), qzeros.data_ptr(), out.data_ptr(),
                                               M, N, K, g, 1 if gated else 0, _lib.dtype_id(x.dtype), ws, ws_bytes, stream))
    return out


def awq_gemv_rmsnorm_qkv_rope_store(x: torch.Tensor, ssq: torch.Tensor, norm_weight: torch.Tensor, norm_eps: float,
                                    qweight: torch.Tensor, qscales: torch.Tensor, qzeros: torch.Tensor,
                                    q_weight: torch.Tensor, k_weight: torch.Tensor, cos_sin: torch.Tensor,
                                    positions: torch.Tensor, slots: torch.Tensor, k_cache: torch.Tensor,
                                    v_cache: torch.Tensor, num_heads: int, num_kv_heads: int, eps: float) -> torch.Tensor:
    """awq_gemv_qkv_rope_store on RMSNorm(x) * norm_weight, x [M <= 64, K] the residual stream, ssq [K / 128, M]."""
    dev = _dev(x, ssq, norm_weight, qweight, qscales, qzeros, q_weight, k_weight, cos_sin, positions, slots, k_cache,
               v_cache)
    M, K = x.shape
    N = qscales.shape[1]
    g = K // qscales.shape[0]
    hd = 128
    assert N == (num_heads + 2 * num_kv_heads) * hd
    assert qweight.shape == (K, N // 8) and qzeros.shape == (K // g, N // 8) and x.dtype == qscales.dtype
    assert K % 128 == 0 and ssq.shape == (K // 128, M) and ssq.dtype == torch.float32
    assert norm_weight.shape == (K,) and norm_weight.dtype == x.dtype
    assert q_weight.shape == (hd,) and k_weight.shape == (hd,) and q_weight.dtype == x.dtype and k_weight.dtype == x.dtype
    assert k_cache.dtype == x.dtype and v_cache.dtype == x.dtype and k_cache.shape == v_cache.shape
    assert k_cache.dim() == 4 and k_cache.shape[1] == num_kv_heads and k_cache.shape[3] == hd
    assert cos_sin.dtype == torch.float32 and cos_sin.numel() % hd == 0
    assert positions.dtype == torch.int64 and slots.dtype == torch.int64 and positions.numel() == M and slots.numel() == M
    block_size = k_cache.shape[2]
    num_slots = k_cache.numel() // (num_kv_heads * hd)
    q = torch.empty(M, num_heads, hd, dtype=x.dtype, device=dev)
    with _lib.on_device(dev):
        ws, ws_bytes, stream = _gemv_ws(dev, M, N, K)
        _lib.check(_lib.lib().awq_gemv_rmsnorm_qkv_rope_store(
            x.data_ptr(), ssq.data_ptr(), norm_weight.data_ptr(), norm_eps, qweight.data_ptr(), qscales.data_ptr(),
            qzeros.data_ptr(), q_weight.data_ptr(), k_weight.data_ptr(), cos_sin.data_ptr(), positions.data_ptr(),
            slots.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), M, N, K, g, num_heads, num_kv_heads,
            cos_sin.numel() // hd, num_slots, block_size, eps, _lib.dtype_id(x.dtype), ws, ws_bytes, stream))
    return q


def paged_attention_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                           context_lens: torch.Tensor, scale: float) -> torch.Tensor:
    """q [batch, nh, hd]; caches [num_blocks, nkv, block_size, hd]; block_table int32 [batch, max_blocks];
    context_lens int32 [batch].  Returns [batch, nh * hd]."""
    dev = _dev(q, k_cache, v_cache, block_table, context_lens)
    batch, nh, hd = q.shape
    num_blocks, nkv, block_size, hd2 = k_cache.shape
    assert hd2 == hd and v_cache.shape == k_cache.shape and k_cache.dtype == q.dtype and v_cache.dtype == q.dtype
    assert block_table.dtype == torch.int32 and context_lens.dtype == torch.int32
    assert block_table.shape[0] == batch and context_lens.shape == (batch,)
    max_blocks = block_table.shape[1]
    out = torch.empty(batch, nh * hd, dtype=q.dtype, device=dev)
    L = _lib.lib()
    with _lib.on_device(dev):
        nbytes = L.nq_paged_attention_workspace_bytes(batch, nh, nkv, hd, block_size * max_blocks)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev) if nbytes else None
        _lib.check(L.nq_paged_attention_decode(
            q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(), context_lens.data_ptr(),
            out.data_ptr(), batch, nh, nkv, hd, block_size, max_blocks, num_blocks, scale, _lib.dtype_id(q.dtype),
            None if ws is None else ws.data_ptr(), nbytes, _stream(dev)))
    return out


def silu_mul(gate_up: torch.Tensor, interleaved: bool = False) -> torch.Tensor:
    """gate_up [rows, 2*inter] -> SiLU(gate) * up [rows, inter]; gate | up side by side, or interleaved in words
    of 8 columns (the layout of interleave_gate_up)."""
    dev = _dev(gate_up)
    rows, two = gate_up.shape
    inter = two // 2
    assert two == 2 * inter and gate_up.is_contiguous()
    out = torch.empty(rows, inter, dtype=gate_up.dtype, device=dev)
    fn = _lib.lib().nq_silu_mul_interleaved if interleaved else _lib.lib().nq_silu_mul
    with _lib.on_device(dev):
        _lib.check(fn(gate_up.data_ptr(), out.data_ptr(), rows, inter, _lib.dtype_id(gate_up.dtype), _stream(dev)))
    return out


def argmax_rows(logits: torch.Tensor) -> torch.Tensor:
    """Greedy sampler: int64 [rows] index of the largest logit per row (lowest index among equal maxima)."""
    dev = _dev(logits)
    rows, vocab = logits.shape
    assert logits.is_contiguous()
    out = torch.empty(rows, dtype=torch.int64, device=dev)
    with _lib.on_device(dev):
        _lib.check(_lib.lib().nq_argmax_rows(logits.data_ptr(), out.data_ptr(), rows, vocab,
                                             _lib.dtype_id(logits.dtype), _stream(dev)))
    return out


def decode_prepare(positions: torch.Tensor, active: torch.Tensor, block_table: torch.Tensor, block_size: int):
    """positions int64 [rows], active bool [rows], block_table int32 [rows, max_blocks] -> (slots int64 [rows] with -1
    for idle rows, context_lens int32 [rows] = positions + 1)."""
    dev = _dev(positions, active, block_table)
    rows = positions.numel()
    assert positions.dtype == torch.int64 and active.dtype == torch.bool and block_table.dtype == torch.int32
    assert active.numel() == rows and block_table.dim() == 2 and block_table.shape[0] == rows
    slots = torch.empty(rows, dtype=torch.int64, device=dev)
    ctx = torch.empty(rows, dtype=torch.int32, device=dev)
    with _lib.on_device(dev):
        _lib.check(_lib.lib().nq_decode_prepare(positions.data_ptr(), active.data_ptr(), block_table.data_ptr(),
                                                slots.data_ptr(), ctx.data_ptr(), rows, block_table.shape[1], block_size,
                                                _stream(dev)))
    return slots, ctx


def decode_advance(next_tokens: torch.Tensor, active: torch.Tensor, out_log: torch.Tensor, ids: torch.Tensor,
                   positions: torch.Tensor, step: torch.Tensor) -> None:
    """IN PLACE: out_log[step[0]] = next_tokens, ids = next_tokens, positions += active, step += 1."""
    dev = _dev(next_tokens, active, out_log, ids, positions, step)
    rows = next_tokens.numel()
    assert all(t.dtype == torch.int64 for t in (next_tokens, out_log, ids, positions, step)) and active.dtype == torch.bool
    assert out_log.dim() == 2 and out_log.shape[1] == rows and ids.numel() == rows and positions.numel() == rows
    assert active.numel() == rows and step.numel() == 1
    with _lib.on_device(dev):
        _lib.check(_lib.lib().nq_decode_advance(next_tokens.data_ptr(), active.data_ptr(), out_log.data_ptr(),
                                                ids.data_ptr(), positions.data_ptr(), step.data_ptr(), rows,
                                                out_log.shape[0], _stream(dev)))


def interleave_gate_up(gate, up):
    """Packed buffers (qweight, qscales, qzeros) of the gate and the up projection -> one set with the word
    columns interleaved (word 2t = gate word t, word 2t+1 = up word t), the layout awq_gemv_swiglu takes."""
    gq, gs, gz = gate
    uq, us, uz = up
    K, W = gq.shape
    G = gz.shape[0]
    qweight = torch.stack([gq, uq], dim=2).reshape(K, 2 * W).contiguous()
    qzeros = torch.stack([gz, uz], dim=2).reshape(G, 2 * W).contiguous()
    qscales = torch.stack([gs.view(G, W, 8), us.view(G, W, 8)], dim=2).reshape(G, 16 * W).contiguous()
    return qweight, qscales, qzeros


def awq_linear_swiglu(x: torch.Tensor, qweight: torch.Tensor, qscales: torch.Tensor, qzeros: torch.Tensor) -> torch.Tensor:
    """x [M, K] (any M) and interleaved gate|up buffers [K, 2*inter/8] -> SiLU(x @ Wgate) * (x @ Wup) [M, inter]."""
    dev = _dev(x, qweight, qscales, qzeros)
    M, K = x.shape
    N = qscales.shape[1]
    g = K // qscales.shape[0]
    assert qweight.shape == (K, N // 8) and qzeros.shape == (K // g, N // 8) and x.dtype == qscales.dtype
    out = torch.empty(M, N // 2, dtype=x.dtype, device=dev)
    L = _lib.lib()
    with _lib.on_device(dev):
        stream = _stream(dev)
        nbytes = L.awq_linear_swiglu_workspace_bytes(M, N, K)
        ws = _lib.workspace(dev, stream, nbytes)
        _lib.check(L.awq_linear_swiglu(x.data_ptr(), qweight.data_ptr(), qscales.data_ptr(), qzeros.data_ptr(),
                                       out.data_ptr(), M, N, K, g, _lib.dtype_id(x.dtype),
                                       None if ws is None else ws.data_ptr(), 0 if ws is None else ws.numel(), stream))
    return out


def awq_gemv_swiglu(x: torch.Tensor, qweight: torch.Tensor, qscales: torch.Tensor, qzeros: torch.Tensor) -> torch.Tensor:
    """x [M <= 64, K] and interleaved gate|up buffers [K, 2*inter/8] -> SiLU(x @ Wgate) * (x @ Wup) [M, inter]."""
    dev = _dev(x, qweight, qscales, qzeros)
    M, K = x.shape
    N = qscales.shape[1]
    g = K // qscales.shape[0]
    assert qweight.shape == (K, N // 8) and qzeros.shape == (K // g, N // 8) and x.dtype == qscales.dtype
    out = torch.empty(M, N // 2, dtype=x.dtype, device=dev)
    L = _lib.lib()
    with _lib.on_device(dev):
        stream = _stream(dev)
        nbytes = L.awq_gemv_workspace_bytes(M, N, K)
        ws = _lib.workspace(dev, stream, nbytes)
        _lib.check(L.awq_gemv_swiglu(x.data_ptr(), qweight.data_ptr(), qscales.data_ptr(), qzeros.data_ptr(),
                                     out.data_ptr(), M, N, K, g, _lib.dtype_id(x.dtype),
                                     None if ws is None else ws.data_ptr(), 0 if ws is None else ws.numel(), stream))
    return out
