"""Paged-KV greedy generation for Qwen3QuantizedForCausalLM on one MI355X.

Layout.  One K and one V tensor per model: [layers, blocks, block_size, kv_heads, head_dim] in the
model dtype; a sequence owns a list of blocks (its row of the block table); token t of a sequence
lives in slot block_table[t // block_size] * block_size + t % block_size.

Weights.  q/k/v (same input) and gate/up (same input) are concatenated along N into one packed AWQ
linear each -- legal because a packed word holds 8 consecutive output columns and every width is a
multiple of 8 -- so a block costs 4 AWQ launches instead of 7.  The fused buffers are derived at
start-up; the checkpoint layout is untouched.

Decode.  All per-step inputs live in fixed device buffers (token ids, positions, slots, context
lengths, block table), attention always spans the table's full width under a length mask, so the
step has static shapes and is captured once in a HIP graph and replayed.
"""
from __future__ import annotations

from typing import List, Optional

import torch
import torch.nn.functional as F

from ..layers.gemm import _linear
from ..models.qwen3_quantized import Qwen3QuantizedForCausalLM


class PagedKVCache:
    def __init__(self, num_layers: int, num_blocks: int, block_size: int, num_kv_heads: int, head_dim: int,
                 dtype: torch.dtype, device: torch.device):
        self.block_size = block_size
        self.num_blocks = num_blocks
        shape = (num_layers, num_blocks, block_size, num_kv_heads, head_dim)
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
                 num_blocks: Optional[int] = None, use_graph: bool = True):
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
        self.gate_up = [_FusedLinear([l.mlp.gate_proj, l.mlp.up_proj]) for l in layers]
        self.use_graph = use_graph
        self._graph = None
        B, dev = max_batch, self.device
        # static decode inputs / outputs
        self.s_ids = torch.zeros(B, dtype=torch.long, device=dev)
        self.s_pos = torch.zeros(B, dtype=torch.long, device=dev)
        self.s_slots = torch.zeros(B, dtype=torch.long, device=dev)
        self.s_ctx = torch.ones(B, dtype=torch.long, device=dev)
        self.s_table = torch.zeros(B, self.max_blocks, dtype=torch.long, device=dev)
        self.s_next = torch.zeros(B, dtype=torch.long, device=dev)
        self._arange_ctx = torch.arange(self.max_ctx, device=dev)

    # ---- one transformer block on the cache --------------------------------------------------------
    def _block(self, li: int, x: torch.Tensor, pos: torch.Tensor, slots: torch.Tensor, attend):
        """x: [b, s, hidden]; pos: [b, s]; slots: [b*s] flat cache slots of these tokens;
        attend(q, k, v, li) -> [b, s, heads*head_dim] given this call's q [b,s,h,d], k, v [b,s,kv,d]."""
        layer = self.model.model.layers[li]
        attn = layer.self_attn
        b, s, _ = x.shape
        h = layer.input_layernorm(x)
        qkv = self.qkv[li](h.reshape(b * s, -1))
        q, k, v = torch.split(qkv, [self.nh * self.hd, self.nkv * self.hd, self.nkv * self.hd], dim=-1)
        q = q.view(b, s, self.nh, self.hd)
        k = k.view(b, s, self.nkv, self.hd)
        v = v.view(b, s, self.nkv, self.hd)
        q, k = attn.rope(attn.q_norm(q), attn.k_norm(k), pos)
        self.cache.k[li].view(-1, self.nkv, self.hd).index_copy_(0, slots, k.reshape(b * s, self.nkv, self.hd))
        self.cache.v[li].view(-1, self.nkv, self.hd).index_copy_(0, slots, v.reshape(b * s, self.nkv, self.hd))
        o = attend(q, k, v, li)
        x = x + attn.o_proj(o).view(b, s, -1)
        h = layer.post_attention_layernorm(x)
        gu = self.gate_up[li](h.reshape(b * s, -1))
        act = F.silu(gu[:, : self.inter]) * gu[:, self.inter:]
        return x + layer.mlp.down_proj(act).view(b, s, -1)

    # ---- prefill: full causal attention over the prompt itself ------------------------------------
    @torch.no_grad()
    def _prefill(self, ids: torch.Tensor, tables: List[List[int]]) -> torch.Tensor:
        """ids: [b, s] (equal-length prompts). Returns the next token of every sequence [b]."""
        b, s = ids.shape
        pos = torch.arange(s, device=self.device).unsqueeze(0).expand(b, s)
        tbl = torch.tensor([t[: (s + self.block_size - 1) // self.block_size] for t in tables], device=self.device)
        slots = (tbl[:, pos[0] // self.block_size] * self.block_size + pos % self.block_size).reshape(-1)
        gqa = self.nh != self.nkv

        def attend(q, k, v, li):
            o = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2),
                                               is_causal=True, enable_gqa=gqa)
            return o.transpose(1, 2).reshape(b * s, self.nh * self.hd)

        x = self.model.model.embed_tokens(ids)
        for li in range(len(self.model.model.layers)):
            x = self._block(li, x, pos, slots, attend)
        x = self.model.model.norm(x[:, -1])
        return self.model.lm_head(x).argmax(dim=-1)

    # ---- decode: one token per sequence, attention over the paged cache --------------------------
    def _decode_step(self) -> None:
        B = self.max_batch
        mask = (self._arange_ctx.unsqueeze(0) < self.s_ctx.unsqueeze(1)).view(B, 1, 1, self.max_ctx)
        gqa = self.nh != self.nkv

        def attend(q, k, v, li):
            kk = self.cache.k[li][self.s_table].view(B, self.max_ctx, self.nkv, self.hd)
            vv = self.cache.v[li][self.s_table].view(B, self.max_ctx, self.nkv, self.hd)
            o = F.scaled_dot_product_attention(q.transpose(1, 2), kk.transpose(1, 2), vv.transpose(1, 2),
                                               attn_mask=mask, enable_gqa=gqa)
            return o.transpose(1, 2).reshape(B, self.nh * self.hd)

        x = self.model.model.embed_tokens(self.s_ids).unsqueeze(1)
        pos = self.s_pos.unsqueeze(1)
        for li in range(len(self.model.model.layers)):
            x = self._block(li, x, pos, self.s_slots, attend)
        x = self.model.model.norm(x[:, 0])
        self.s_next.copy_(self.model.lm_head(x).argmax(dim=-1))

    def _run_decode(self) -> None:
        if not self.use_graph:
            self._decode_step()
            return
        if self._graph is None:
            s = torch.cuda.Stream()
            s.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(s):
                for _ in range(2):          # warm-up: workspaces and library handles exist before capture
                    self._decode_step()
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
            # batch rows beyond n mirror row 0 (same token, slot and table): they recompute and rewrite
            # row 0's values, so the step keeps its static shape without touching any other state
            rows = list(range(n)) + [0] * (self.max_batch - n)
            tbl_cpu = torch.tensor(tables)[rows]
            self.s_table.copy_(tbl_cpu)
            bs = self.block_size
            for step in range(1, max_new_tokens):
                t = plen + step - 1                                  # position of the token being fed
                self.s_ids.copy_(nxt[rows] if n < self.max_batch else nxt)
                self.s_pos.fill_(t)
                self.s_slots.copy_(tbl_cpu[:, t // bs] * bs + t % bs)
                self.s_ctx.fill_(t + 1)
                self._run_decode()
                nxt = self.s_next[:n].clone()
                out.append(nxt.tolist())
            if stats is not None:
                torch.cuda.synchronize()
                stats.update(prefill_s=t1 - t0, decode_s=time.perf_counter() - t1, decode_steps=max_new_tokens - 1,
                             batch=n, prompt_len=plen)
            return [[out[s][i] for s in range(len(out))] for i in range(n)]
        finally:
            for t in tables:
                self.cache.release(t)
