"""Paged-KV greedy generation for Qwen3QuantizedForCausalLM on one MI355X.

Layout.  One K and one V tensor per model: [layers, blocks, kv_heads, block_size, head_dim] in the
model dtype (a head's tokens of one block are contiguous: 16 KiB runs for the attention kernel); a sequence owns a list of blocks (its row of the block table); token t of a sequence
lives in slot block_table[t // block_size] * block_size + t % block_size.

Weights.  q/k/v (same input) and gate/up (same input) are concatenated along N into one packed AWQ
linear each -- legal because a packed word holds 8 consecutive output columns and every width is a
multiple of 8 -- so a block costs 4 AWQ launches instead of 7.  The fused buffers are derived at
start-up; the checkpoint layout is untouched.

Decode.  One step = embedding, then per block: add+RMSNorm kernel, fused q|k|v AWQ GEMV, a kernel that
does per-head q/k RMSNorm + rotary and writes k/v into their cache slots, paged attention (flash
decoding over the block table), o_proj GEMV, add+RMSNorm, fused gate|up GEMV, SiLU*up kernel, down GEMV
(include/nq_engine_ops.h + include/awq_hip.h).  Where the shapes allow (head_dim 128, hidden a multiple of 128, gate|up
interleaved) the two add+RMSNorm kernels disappear as well: the o_proj and down_proj GEMVs add into the residual
stream and leave its RMSNorm statistics, the q|k|v and gate|up GEMVs normalise their input on the way in -- five
launches per block, same bits.  All per-step state lives in fixed device buffers (token
ids, positions, active mask, block table, step counter, output tokens) and the step advances that
state itself, so it is captured once in a HIP graph and replayed with no host work between steps.

Scheduling.  `generate` runs one static batch of equal-length prompts.  `serve` is continuous batching over
the same decode graph: requests of any length wait in a queue, are admitted whenever a batch row and enough
cache blocks are free (their prompt is prefilled on its own), decode together with whatever else is running,
and give their row and blocks back when they reach their token budget or the end-of-sequence token.
"""
from __future__ import annotations

from typing import List, Optional

import torch
import torch.nn.functional as F

from ..layers.gemm import _linear, prefetch_hint
from . import ops
from ..models.qwen3_quantized import Qwen3QuantizedForCausalLM


class PagedKVCache:
    def __init__(self, num_layers: int, num_blocks: int, block_size: int, num_kv_heads: int, head_dim: int,
                 dtype: torch.dtype, device: torch.device):
        self.block_size = block_size
        self.num_blocks = num_blocks
        shape = (num_layers, num_blocks, num_kv_heads, block_size, head_dim)
        self.k = torch.zeros(shape, dtype=dtype, device=device)
        self.v = torch.zeros(shape, dtype=dtype, device=device)
        self.free: List[int] = list(range(num_blocks - 1, -1, -1))

    def allocate(self, n: int) -> List[int]:
        if n > len(self.free):
            raise RuntimeError(f"KV cache exhausted: {n} blocks wanted, {len(self.free)} free")
        return [self.free.pop() for _ in range(n)]

    def release(self, blocks: List[int]) -> None:
        self.free.extend(reversed(blocks))


class _FusedLinear:
    """Packed buffers of several WQLinear_GEMM with a common input, concatenated along N."""

    def __init__(self, mods):
        self.qweight = torch.cat([m.qweight for m in mods], dim=1).contiguous()
        self.qzeros = torch.cat([m.qzeros for m in mods], dim=1).contiguous()
        self.qscales = torch.cat([m.qscales for m in mods], dim=1).contiguous()
        assert all(m.bias is None for m in mods), "fused AWQ linears carry no bias in Qwen3"

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        return _linear("awq_linear", x, self.qweight, self.qscales, self.qzeros, None)


class LLMEngine:
    def __init__(self, model: Qwen3QuantizedForCausalLM, max_batch: int, max_seq_len: int, block_size: int = 64,
                 num_blocks: Optional[int] = None, use_graph: bool = True, fuse_norm: bool = True):
        self.model = model.eval()
        p = next(model.parameters())
        self.device, self.dtype = p.device, p.dtype
        if self.device.type != "cuda":
            raise RuntimeError("LLMEngine needs the model on a HIP device")
        layers = model.model.layers
        a0 = layers[0].self_attn
        self.nh, self.nkv, self.hd = a0.num_heads, a0.num_kv_heads, a0.head_dim
        self.inter = layers[0].mlp.intermediate_size
        self.max_batch, self.block_size = max_batch, block_size
        self.max_blocks = (max_seq_len + block_size - 1) // block_size
        self.max_ctx = self.max_blocks * block_size
        if num_blocks is None:
            num_blocks = max_batch * self.max_blocks
        self.cache = PagedKVCache(len(layers), num_blocks, block_size, self.nkv, self.hd, self.dtype, self.device)
        self.qkv = [_FusedLinear([l.self_attn.q_proj, l.self_attn.k_proj, l.self_attn.v_proj]) for l in layers]
        # gate and up interleaved word by word, SiLU(gate) * up applied in the epilogue of the GEMV (decode) or
        # the GEMM (prefill); shapes that form does not take keep the two projections side by side + silu_mul
        g0 = layers[0].mlp.gate_proj
        self.swiglu_ok = (2 * self.inter) % 128 == 0 and g0.group_size % 128 == 0 and g0.in_features % 64 == 0
        self.gate_up = None if self.swiglu_ok else [_FusedLinear([l.mlp.gate_proj, l.mlp.up_proj]) for l in layers]
        self.gate_up_il = [ops.interleave_gate_up((l.mlp.gate_proj.qweight, l.mlp.gate_proj.qscales, l.mlp.gate_proj.qzeros),
                                                  (l.mlp.up_proj.qweight, l.mlp.up_proj.qscales, l.mlp.up_proj.qzeros))
                           for l in layers] if self.swiglu_ok else None
        q0 = layers[0].self_attn.q_proj
        self.qkv_fused_ok = (self.hd == 128 and max_batch <= 64 and q0.group_size % 128 == 0 and q0.bias is None)
        # residual add + RMSNorm folded into the neighbouring GEMVs (statistics handed from one to the next); not for
        # models whose MLP weights at this batch run faster on the shared-chunk GEMV, which has no such form
        hidden = q0.in_features
        self.norm_fused_ok = (fuse_norm and self.qkv_fused_ok and self.swiglu_ok and hidden % 128 == 0
                              and (max_batch <= 16 or 2 * self.inter * hidden < (50 << 20)))
        # in the plain decode step: the residual add + RMSNorm after o_proj / down_proj inside the GEMV's second pass,
        # where that GEMV has one at this batch (the large models at 33..64 rows)
        o0, d0 = layers[0].self_attn.o_proj, layers[0].mlp.down_proj
        self.o_add_norm = o0.bias is None and ops.gemv_add_rmsnorm_supported(
            max_batch, o0.out_features, o0.in_features, o0.group_size)
        self.down_add_norm = d0.bias is None and ops.gemv_add_rmsnorm_supported(
            max_batch, d0.out_features, d0.in_features, d0.group_size)
        self.use_graph = use_graph
        self._graph = None
        B, dev = max_batch, self.device
        # static decode state, advanced on the device by the step itself
        self.s_ids = torch.zeros(B, dtype=torch.long, device=dev)       # token fed at this step
        self.s_pos = torch.zeros(B, dtype=torch.long, device=dev)       # its position
        self.s_active = torch.zeros(B, dtype=torch.bool, device=dev)    # rows that own cache blocks
        self.s_table = torch.zeros(B, self.max_blocks, dtype=torch.int32, device=dev)
        self.s_step = torch.zeros(1, dtype=torch.long, device=dev)      # row of s_out the step writes
        self.s_out = torch.zeros(self.max_ctx + 1, B, dtype=torch.long, device=dev)
        self.eps = layers[0].input_layernorm.eps
        self.scale = float(self.hd) ** -0.5

    # ---- prefill: full causal attention over the prompt itself ------------------------------------
    @torch.no_grad()
    def _prefill(self, ids: torch.Tensor, tables: List[List[int]]) -> torch.Tensor:
        """ids: [b, s] (equal-length prompts). Returns the next token of every sequence [b].  Same kernels as
        the decode step around the AWQ linears (which take the MFMA GEMM at these row counts); the causal
        attention over the prompt is torch's scaled_dot_product_attention."""
        b, s = ids.shape
        m, bs, eps = self.model.model, self.block_size, self.eps
        pos = torch.arange(s, device=self.device).unsqueeze(0).expand(b, s)
        tbl = torch.tensor([t[: (s + bs - 1) // bs] for t in tables], device=self.device)
        slots = (tbl[:, pos[0] // bs] * bs + pos % bs).reshape(-1).contiguous()
        pos_flat = pos.reshape(-1).contiguous()
        gqa = self.nh != self.nkv
        kvw = self.nkv * self.hd
        x = m.embed_tokens(ids).reshape(b * s, -1)                       # residual stream [b*s, hidden]
        delta = None
        for li, layer in enumerate(m.layers):
            attn = layer.self_attn
            h = ops.add_rmsnorm(x, delta, layer.input_layernorm.weight, eps)
            qkv = self.qkv[li](h)
            q, k = ops.qk_norm_rope_store(qkv, attn.q_norm.weight, attn.k_norm.weight, attn.rope.cos_sin_cache,
                                          pos_flat, slots, self.cache.k[li], self.cache.v[li], self.nh, self.nkv,
                                          self.hd, attn.q_norm.eps, dense_k=True)
            v = qkv[:, -kvw:].view(b, s, self.nkv, self.hd)
            o = F.scaled_dot_product_attention(q.view(b, s, self.nh, self.hd).transpose(1, 2),
                                               k.view(b, s, self.nkv, self.hd).transpose(1, 2), v.transpose(1, 2),
                                               is_causal=True, enable_gqa=gqa)
            o = o.transpose(1, 2).reshape(b * s, self.nh * self.hd)
            h = ops.add_rmsnorm(x, attn.o_proj(o), layer.post_attention_layernorm.weight, eps)
            act = (ops.awq_linear_swiglu(h, *self.gate_up_il[li]) if self.swiglu_ok
                   else ops.silu_mul(self.gate_up[li](h)))
            delta = layer.mlp.down_proj(act)
        last = x.view(b, s, -1)[:, -1].contiguous()
        dlast = delta.view(b, s, -1)[:, -1].contiguous()
        h = ops.add_rmsnorm(last, dlast, m.norm.weight, m.norm.eps)
        return ops.argmax_rows(self.model.lm_head(h))

    @torch.no_grad()
    def _prefill_ragged(self, prompts: List[List[int]], tables: List[List[int]]) -> torch.Tensor:
        """Prompts of any lengths in one pass: every per-token operation (norms, AWQ linears, rotary, cache write)
        runs once over the concatenated tokens, the causal attention once per prompt over its own slice.  Returns the
        next token of every prompt [len(prompts)]."""
        m, bs, eps = self.model.model, self.block_size, self.eps
        dev = self.device
        lens = [len(p) for p in prompts]
        starts = [0]
        for n in lens:
            starts.append(starts[-1] + n)
        total = starts[-1]
        ids = torch.tensor([t for p in prompts for t in p], dtype=torch.long, device=dev)
        pos_flat = torch.cat([torch.arange(n, device=dev) for n in lens]).contiguous()
        slot_list = []
        for n, tbl in zip(lens, tables):
            t = torch.tensor(tbl[: (n + bs - 1) // bs], device=dev)
            p = torch.arange(n, device=dev)
            slot_list.append(t[p // bs] * bs + p % bs)
        slots = torch.cat(slot_list).contiguous()
        gqa = self.nh != self.nkv
        kvw = self.nkv * self.hd
        x = m.embed_tokens(ids)                                          # residual stream [total, hidden]
        delta = None
        for li, layer in enumerate(m.layers):
            attn = layer.self_attn
            h = ops.add_rmsnorm(x, delta, layer.input_layernorm.weight, eps)
            qkv = self.qkv[li](h)
            q, k = ops.qk_norm_rope_store(qkv, attn.q_norm.weight, attn.k_norm.weight, attn.rope.cos_sin_cache,
                                          pos_flat, slots, self.cache.k[li], self.cache.v[li], self.nh, self.nkv,
                                          self.hd, attn.q_norm.eps, dense_k=True)
            v = qkv[:, -kvw:].view(total, self.nkv, self.hd)
            o = torch.empty(total, self.nh * self.hd, dtype=self.dtype, device=dev)
            for a, n in zip(starts, lens):
                oi = F.scaled_dot_product_attention(q[a:a + n].transpose(0, 1).unsqueeze(0),
                                                    k[a:a + n].transpose(0, 1).unsqueeze(0),
                                                    v[a:a + n].transpose(0, 1).unsqueeze(0),
                                                    is_causal=True, enable_gqa=gqa)
                o[a:a + n] = oi[0].transpose(0, 1).reshape(n, self.nh * self.hd)
            h = ops.add_rmsnorm(x, attn.o_proj(o), layer.post_attention_layernorm.weight, eps)
            act = (ops.awq_linear_swiglu(h, *self.gate_up_il[li]) if self.swiglu_ok
                   else ops.silu_mul(self.gate_up[li](h)))
            delta = layer.mlp.down_proj(act)
        last = torch.tensor([a + n - 1 for a, n in zip(starts, lens)], device=dev)
        h = ops.add_rmsnorm(x[last].contiguous(), delta[last].contiguous(), m.norm.weight, m.norm.eps)
        return ops.argmax_rows(self.model.lm_head(h))

    # ---- decode: one token per sequence, attention over the paged cache --------------------------
    def _decode_step(self) -> None:
        m, bs, eps = self.model.model, self.block_size, self.eps
        pos = self.s_pos
        # idle rows read row 0's table but write nothing: slot -1 is skipped by the kernels
        slots, ctx = ops.decode_prepare(pos, self.s_active, self.s_table, bs)
        nl = len(m.layers)
        if self.norm_fused_ok:
            # five launches per block: the o_proj and down_proj GEMVs add into the residual stream and leave its
            # RMSNorm statistics, the q|k|v and gate|up GEMVs normalise their input on the way in
            x, ssq = ops.embed_row_ssq(self.s_ids, m.embed_tokens.weight)   # residual stream [B, hidden]
            for li, layer in enumerate(m.layers):
                attn, lin, mlp = layer.self_attn, self.qkv[li], layer.mlp
                prefetch_hint(attn.o_proj.qweight, attn.o_proj.qscales)
                q = ops.awq_gemv_rmsnorm_qkv_rope_store(
                    x, ssq, layer.input_layernorm.weight, eps, lin.qweight, lin.qscales, lin.qzeros,
                    attn.q_norm.weight, attn.k_norm.weight, attn.rope.cos_sin_cache, pos, slots, self.cache.k[li],
                    self.cache.v[li], self.nh, self.nkv, attn.q_norm.eps)
                o = ops.paged_attention_decode(q, self.cache.k[li], self.cache.v[li], self.s_table, ctx, self.scale)
                prefetch_hint(*self.gate_up_il[li][:2])
                ops.awq_gemv_add_residual(o, attn.o_proj.qweight, attn.o_proj.qscales, attn.o_proj.qzeros, x, ssq)
                prefetch_hint(mlp.down_proj.qweight, mlp.down_proj.qscales)
                act = ops.awq_gemv_rmsnorm(x, ssq, layer.post_attention_layernorm.weight, eps, *self.gate_up_il[li],
                                           gated=True)
                if li + 1 < nl:
                    prefetch_hint(self.qkv[li + 1].qweight, self.qkv[li + 1].qscales)
                ops.awq_gemv_add_residual(act, mlp.down_proj.qweight, mlp.down_proj.qscales, mlp.down_proj.qzeros, x, ssq)
            self._finish_step(ops.add_rmsnorm(x, None, m.norm.weight, m.norm.eps))
            return
        x = m.embed_tokens(self.s_ids)                                   # residual stream [B, hidden]

        def lin_add_norm(lin, fused, inp, w, e):   # x += lin(inp) in place; returns RMSNorm(x) * w
            if fused:
                return ops.awq_gemv_add_rmsnorm(inp, lin.qweight, lin.qscales, lin.qzeros, x, w, e)
            return ops.add_rmsnorm(x, lin(inp), w, e)

        h = ops.add_rmsnorm(x, None, m.layers[0].input_layernorm.weight, eps)
        for li, layer in enumerate(m.layers):
            attn = layer.self_attn
            gu = self.gate_up_il[li][:2] if self.swiglu_ok else (self.gate_up[li].qweight, self.gate_up[li].qscales)
            # every AWQ launch also pulls the next launch's packed weights and scales towards the Infinity Cache
            # (the small zero-point tensor measured as a net loss)
            prefetch_hint(attn.o_proj.qweight, attn.o_proj.qscales)
            if self.qkv_fused_ok:   # projection, q/k norm, rotary and cache write in one launch
                lin = self.qkv[li]
                q = ops.awq_gemv_qkv_rope_store(h, lin.qweight, lin.qscales, lin.qzeros, attn.q_norm.weight,
                                                attn.k_norm.weight, attn.rope.cos_sin_cache, pos, slots,
                                                self.cache.k[li], self.cache.v[li], self.nh, self.nkv, attn.q_norm.eps)
            else:
                q = ops.qk_norm_rope_store(self.qkv[li](h), attn.q_norm.weight, attn.k_norm.weight,
                                           attn.rope.cos_sin_cache, pos, slots, self.cache.k[li], self.cache.v[li],
                                           self.nh, self.nkv, self.hd, attn.q_norm.eps)
            o = ops.paged_attention_decode(q, self.cache.k[li], self.cache.v[li], self.s_table, ctx, self.scale)
            prefetch_hint(*gu)
            h = lin_add_norm(attn.o_proj, self.o_add_norm, o, layer.post_attention_layernorm.weight, eps)
            prefetch_hint(layer.mlp.down_proj.qweight, layer.mlp.down_proj.qscales)
            act = (ops.awq_linear_swiglu(h, *self.gate_up_il[li]) if self.swiglu_ok
                   else ops.silu_mul(self.gate_up[li](h)))
            if li + 1 < nl:
                nq_ = self.qkv[li + 1]
                prefetch_hint(nq_.qweight, nq_.qscales)
            nw, ne = (m.layers[li + 1].input_layernorm.weight, eps) if li + 1 < nl else (m.norm.weight, m.norm.eps)
            h = lin_add_norm(layer.mlp.down_proj, self.down_add_norm, act, nw, ne)
        self._finish_step(h)

    def _finish_step(self, h: torch.Tensor) -> None:
        nxt = ops.argmax_rows(self.model.lm_head(h))
        # log the tokens, feed them back, move the active rows on (idle rows stay where they are), count the step
        ops.decode_advance(nxt, self.s_active, self.s_out, self.s_ids, self.s_pos, self.s_step)

    def _state(self):
        return [self.s_ids, self.s_pos, self.s_step]

    def _run_decode(self) -> None:
        if not self.use_graph:
            self._decode_step()
            return
        if self._graph is None:
            saved = [t.clone() for t in self._state()]
            s = torch.cuda.Stream()
            s.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(s):
                for _ in range(2):          # warm-up: workspaces and library handles exist before capture
                    self._decode_step()
                    for t, v in zip(self._state(), saved):   # the step advanced the state: put it back
                        t.copy_(v)
                torch.cuda.synchronize()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=s):
                    self._decode_step()
            torch.cuda.current_stream().wait_stream(s)
            self._graph = g
        self._graph.replay()

    @torch.no_grad()
    def generate(self, prompts: List[List[int]], max_new_tokens: int, stats: Optional[dict] = None) -> List[List[int]]:
        """Greedy continuation of each prompt (token-id lists of equal length), `max_new_tokens` each.
        If `stats` is given it receives prefill_s / decode_s wall times (device-synchronised)."""
        import time
        n = len(prompts)
        if n == 0:
            return []
        if n > self.max_batch:
            raise ValueError(f"{n} prompts exceed max_batch={self.max_batch}")
        plen = len(prompts[0])
        if any(len(p) != plen for p in prompts):
            raise ValueError("this engine batches prompts of equal length only")
        if plen + max_new_tokens > self.max_ctx:
            raise ValueError("prompt + max_new_tokens exceeds max_seq_len")
        tables = [self.cache.allocate(self.max_blocks) for _ in range(n)]
        try:
            ids = torch.tensor(prompts, dtype=torch.long, device=self.device)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            nxt = self._prefill(ids, tables)
            out = [nxt.tolist()]
            t1 = time.perf_counter()
            # batch rows beyond n mirror row 0 (same token, position and table) but are marked idle:
            # they recompute row 0's token and write nothing to the cache
            rows = list(range(n)) + [0] * (self.max_batch - n)
            self.s_table.copy_(torch.tensor(tables, dtype=torch.int32)[rows])
            self.s_active.copy_(torch.tensor([True] * n + [False] * (self.max_batch - n)))
            self.s_ids.copy_(nxt[rows] if n < self.max_batch else nxt)
            self.s_pos.fill_(plen)                                   # position of the token being fed
            self.s_step.zero_()
            steps = max_new_tokens - 1
            for _ in range(steps):
                self._run_decode()
            toks = self.s_out[:steps, :n].tolist()                   # one synchronisation for the whole run
            out.extend(toks)
            if stats is not None:
                torch.cuda.synchronize()
                stats.update(prefill_s=t1 - t0, decode_s=time.perf_counter() - t1, decode_steps=max_new_tokens - 1,
                             batch=n, prompt_len=plen)
            return [[out[s][i] for s in range(len(out))] for i in range(n)]
        finally:
            for t in tables:
                self.cache.release(t)

    # ---- continuous batching ---------------------------------------------------------------------------
    @torch.no_grad()
    def serve(self, requests, eos_token_id: Optional[int] = None, stats: Optional[dict] = None,
              batch_prefill: bool = False, max_prefill_tokens: int = 8192) -> List[List[int]]:
        """requests: sequence of (prompt token ids, max_new_tokens), any lengths.  Returns the greedy continuation
        of each request, in request order (cut after `eos_token_id` if one is given).  Without an end-of-sequence
        token the host reads tokens back only when the output buffer fills up or at the end; with one it reads
        them after every step.

        By default every admitted request is prefilled on its own, so its tokens do not depend on what else is
        queued or running (decode rows are independent as well).  `batch_prefill` prefills all requests admitted at
        the same moment in one pass (up to `max_prefill_tokens` prompt tokens): fewer, larger launches, but the row
        count of the prefill linears -- and with it their kernel and summation order -- then depends on the
        company a request arrives in."""
        import time
        from collections import deque
        bs = self.block_size
        for prompt, max_new in requests:
            if len(prompt) < 1 or max_new < 1:
                raise ValueError("every request needs a non-empty prompt and max_new_tokens >= 1")
            if len(prompt) + max_new > self.max_ctx:
                raise ValueError("prompt + max_new_tokens exceeds max_seq_len")
        out: List[List[int]] = [[] for _ in requests]
        waiting = deque(range(len(requests)))
        free_rows = list(range(self.max_batch - 1, -1, -1))
        running = {}                      # row -> [request index, tokens still to decode, blocks]
        step_log = []                     # per decode step since the last read-back: [(row, request index)]
        self.s_active.zero_(); self.s_pos.zero_(); self.s_ids.zero_(); self.s_table.zero_(); self.s_step.zero_()
        torch.cuda.synchronize()
        t_start, n_steps, n_prefill, n_prefill_calls = time.perf_counter(), 0, 0, 0
        prefill_log = []                  # per prefill pass: (prompt tokens, requests, decode steps so far, seconds)

        def retire(row):
            _, _, blocks = running.pop(row)
            self.cache.release(blocks)
            free_rows.append(row)
            self.s_active[row] = False
            self.s_pos[row] = 0

        def read_back():
            """Tokens of the logged steps -> their requests; returns the rows whose request ended with eos."""
            ended = []
            if step_log:
                toks = self.s_out[:len(step_log)].tolist()
                for i, entries in enumerate(step_log):
                    for row, ri in entries:
                        if out[ri] and eos_token_id is not None and out[ri][-1] == eos_token_id:
                            continue            # already ended on an earlier step of this batch of steps
                        out[ri].append(toks[i][row])
                        if eos_token_id is not None and toks[i][row] == eos_token_id and row in running \
                                and running[row][0] == ri:
                            ended.append(row)
                step_log.clear()
                self.s_step.zero_()
            return ended

        try:
            while waiting or running:
                # admit while a row and the blocks for the whole request are free
                admitted = []                 # (request index, blocks), prefilled together if batch_prefill
                tokens_admitted = 0
                while waiting and len(admitted) < len(free_rows):
                    ri = waiting[0]
                    prompt, max_new = requests[ri]
                    need = (len(prompt) + max_new + bs - 1) // bs
                    if need > len(self.cache.free):
                        if not running and not admitted:
                            raise RuntimeError(f"KV cache too small for request {ri}: {need} blocks wanted, "
                                               f"{len(self.cache.free)} exist free with nothing running")
                        break
                    if admitted and (not batch_prefill or tokens_admitted + len(prompt) > max_prefill_tokens):
                        break
                    waiting.popleft()
                    admitted.append((ri, self.cache.allocate(need)))
                    tokens_admitted += len(prompt)
                if admitted:
                    if stats is not None:
                        torch.cuda.synchronize()
                        t_pf = time.perf_counter()
                    try:
                        if len(admitted) == 1:
                            ids = torch.tensor([requests[admitted[0][0]][0]], dtype=torch.long, device=self.device)
                            toks = self._prefill(ids, [admitted[0][1]]).tolist()
                        else:
                            toks = self._prefill_ragged([requests[ri][0] for ri, _ in admitted],
                                                        [b for _, b in admitted]).tolist()
                    except Exception:
                        for _, blocks in admitted:
                            self.cache.release(blocks)
                        raise
                    n_prefill += len(admitted)
                    n_prefill_calls += 1
                    if stats is not None:       # toks.tolist() above has waited for the pass
                        prefill_log.append((tokens_admitted, len(admitted), n_steps, time.perf_counter() - t_pf))
                    for (ri, blocks), tok in zip(admitted, toks):
                        prompt, max_new = requests[ri]
                        out[ri].append(tok)
                        if max_new == 1 or tok == eos_token_id:
                            self.cache.release(blocks)
                            continue
                        row = free_rows.pop()
                        running[row] = [ri, max_new - 1, blocks]
                        self.s_table[row] = torch.tensor(blocks + [0] * (self.max_blocks - len(blocks)), dtype=torch.int32)
                        self.s_ids[row] = tok
                        self.s_pos[row] = len(prompt)
                        self.s_active[row] = True
                    if waiting and free_rows and len(admitted) > 0 and not batch_prefill:
                        continue              # one prefill per pass: admit the next request before decoding
                if not running:
                    continue
                self._run_decode()
                n_steps += 1
                step_log.append([(row, r[0]) for row, r in running.items()])
                done = []
                for row, r in running.items():
                    r[1] -= 1
                    if r[1] == 0:
                        done.append(row)
                if eos_token_id is not None or len(step_log) == self.s_out.shape[0]:
                    done.extend(row for row in read_back() if row not in done)
                for row in done:
                    retire(row)
            read_back()
        finally:
            for row in list(running):
                retire(row)
        if stats is not None:
            torch.cuda.synchronize()
            wall = time.perf_counter() - t_start
            prefill_s = sum(p[3] for p in prefill_log)
            stats.update(wall_s=wall, decode_steps=n_steps, prefills=n_prefill, prefill_calls=n_prefill_calls,
                         tokens=sum(len(o) for o in out), prefill_s=prefill_s, decode_s=wall - prefill_s,
                         prefill_log=prefill_log)
        return out

