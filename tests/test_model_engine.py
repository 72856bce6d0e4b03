"""The callers of the hot path: Qwen3 model contract (CPU), checkpoint round trip (CPU), and on the GPU
the paged-KV engine against the model's own no-cache forward (the reference semantics)."""
import json
import os

import numpy as np
import pytest
import torch

import nanoquantization_amd as nq
from nanoquantization_amd.layers.norm import RMSNorm
from nanoquantization_amd.layers.rope import RoPE
from nanoquantization_amd.models.qwen3_quantized import Qwen3QuantizedForCausalLM
from nanoquantization_amd.utils.loader import load_model, model_from_config, save_quantized_model

TINY = dict(num_hidden_layers=2, vocab_size=512, hidden_size=256, total_num_heads=4, total_num_kv_heads=2,
            max_position_embeddings=256, intermediate_size=512, head_dim=64, tie_word_embeddings=True,
            rope_theta=10000.0, rms_norm_eps=1e-6)


def test_rmsnorm_and_rope_closed_forms():
    torch.manual_seed(0)
    x = torch.randn(3, 5, 64)
    n = RMSNorm(64, 1e-6)
    n.weight.data = torch.linspace(0.5, 1.5, 64)
    expect = x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-6) * n.weight
    assert torch.allclose(n(x), expect, atol=1e-6)
    r = RoPE(64, 128, 10000.0)
    q, k = torch.randn(2, 7, 4, 64), torch.randn(2, 7, 2, 64)
    pos = torch.arange(7).unsqueeze(0).expand(2, 7)
    q2, k2 = r(q, k, pos)
    # rotation preserves the norm of each (i, i+32) pair and position 0 is the identity
    assert torch.allclose(q2[:, 0], q[:, 0], atol=1e-6)
    pair = lambda t: t[..., :32] ** 2 + t[..., 32:] ** 2
    assert torch.allclose(pair(q2), pair(q), atol=1e-4) and torch.allclose(pair(k2), pair(k), atol=1e-4)
    # angle of pair i at position p is p * base^(-2i/d)
    ang = torch.atan2(q2[0, 3, 0, 32:] * q[0, 3, 0, :32] - q2[0, 3, 0, :32] * q[0, 3, 0, 32:],
                      q2[0, 3, 0, :32] * q[0, 3, 0, :32] + q2[0, 3, 0, 32:] * q[0, 3, 0, 32:])
    inv = 1.0 / (10000.0 ** (torch.arange(0, 64, 2).float() / 64))
    assert torch.allclose(torch.remainder(ang, 2 * np.pi), torch.remainder(3 * inv, 2 * np.pi), atol=1e-3)
    # the angle table survives model.to(bfloat16) in fp32
    assert r.to(torch.bfloat16).cos_sin_cache.dtype == torch.float32


def test_model_state_dict_keys_match_reference_contract():
    m = Qwen3QuantizedForCausalLM(**TINY)
    keys = set(m.state_dict())
    for i in range(2):
        for proj in ("q_proj", "k_proj", "v_proj", "o_proj"):
            for buf in ("qweight", "qscales", "qzeros"):
                assert f"model.layers.{i}.self_attn.{proj}.{buf}" in keys
        for proj in ("gate_proj", "up_proj", "down_proj"):
            for buf in ("qweight", "qscales", "qzeros"):
                assert f"model.layers.{i}.mlp.{proj}.{buf}" in keys
        for nrm in ("input_layernorm", "post_attention_layernorm", "self_attn.q_norm", "self_attn.k_norm"):
            assert f"model.layers.{i}.{nrm}.weight" in keys
    assert {"model.norm.weight", "model.embed_tokens.weight", "lm_head.weight", "lm_head.bias"} <= keys
    assert not any("cos_sin_cache" in k for k in keys)       # non-persistent, as in the reference
    assert m.model.layers[0].self_attn.q_proj.qscales.dtype == torch.bfloat16
    assert m.lm_head.weight.data_ptr() == m.model.embed_tokens.weight.data_ptr()   # tied


def test_checkpoint_roundtrip(tmp_path):
    torch.manual_seed(1)
    m = Qwen3QuantizedForCausalLM(**TINY).to(torch.bfloat16)
    for name, buf in m.named_buffers():
        if buf.dtype == torch.int32:
            buf.copy_(torch.randint(-2 ** 31, 2 ** 31 - 1, buf.shape, dtype=torch.int32))
        elif "qscales" in name:
            buf.copy_(torch.rand(buf.shape) * 0.01)
    cfg = dict(num_hidden_layers=2, vocab_size=512, hidden_size=256, num_attention_heads=4, num_key_value_heads=2,
               max_position_embeddings=256, intermediate_size=512, head_dim=64, tie_word_embeddings=True,
               rope_theta=10000.0, rms_norm_eps=1e-6)
    save_quantized_model(m, str(tmp_path), cfg, 4, 128)
    saved = json.load(open(tmp_path / "config.json"))
    assert saved["quantization_config"]["quant_method"] == "awq" and saved["quantization_config"]["version"] == "gemm"
    assert os.path.exists(tmp_path / "model.safetensors") and os.path.exists(tmp_path / "model.safetensors.index.json")
    m2 = model_from_config(str(tmp_path))
    for (k1, v1), (k2, v2) in zip(m.state_dict().items(), m2.state_dict().items()):
        assert k1 == k2 and torch.equal(v1, v2), k1
    m3 = Qwen3QuantizedForCausalLM(**TINY).to(torch.bfloat16)
    load_model(m3, str(tmp_path))
    assert torch.equal(m3.model.layers[1].mlp.down_proj.qweight, m.model.layers[1].mlp.down_proj.qweight)
    with pytest.raises(AttributeError):
        from safetensors.torch import save_file
        save_file({"no.such.tensor": torch.zeros(1)}, str(tmp_path / "extra.safetensors"))
        load_model(m3, str(tmp_path))


@pytest.mark.gpu
def test_engine_greedy_matches_full_recompute():
    from nanoquantization_amd.engine import LLMEngine
    from nanoquantization_amd.models.random_init import random_awq_qwen3
    print("engine vs recompute", flush=True)
    model = random_awq_qwen3(TINY, seed=3, std=0.05)
    torch.manual_seed(4)
    prompts = torch.randint(0, 512, (3, 19)).tolist()
    new = 12
    for use_graph in (False, True):
        eng = LLMEngine(model, max_batch=4, max_seq_len=64, block_size=16, use_graph=use_graph)
        got = eng.generate(prompts, new)
        # reference semantics: full-sequence causal forward, no cache.  Teacher-force the engine's own
        # continuation through it: every token the engine chose must be the recompute's argmax up to the
        # bf16 noise of a near-tie, and where the logits are not near-tied the tokens must be identical.
        seqs = torch.tensor([p + g for p, g in zip(prompts, got)], device="cuda")
        pos = torch.arange(seqs.shape[1], device="cuda").unsqueeze(0)
        logits = model.lm_head(model(seqs, pos)).float()[:, 18:-1]            # predictions for the new tokens
        chosen = torch.tensor(got, device="cuda")
        top = logits.max(-1).values
        gap = top - logits.gather(-1, chosen.unsqueeze(-1)).squeeze(-1)
        scale = logits.abs().max().item()
        assert gap.max().item() <= 2e-2 * scale, (use_graph, gap.max().item(), scale)
        top2 = logits.topk(2, dim=-1).values
        clear = (top2[..., 0] - top2[..., 1]) > 4e-2 * scale
        assert torch.equal(chosen[clear], logits.argmax(-1)[clear])
        assert clear.float().mean().item() > 0.5
        assert [g[0] for g in got] == logits[:, 0].argmax(-1).tolist() or not clear[:, 0].all()
        # a second call reuses the freed blocks and the captured graph
        assert eng.generate(prompts, new) == got


@pytest.mark.gpu
def test_model_forward_matches_dequantised_torch_model():
    from nanoquantization_amd.models.random_init import random_awq_qwen3
    print("model forward vs dequantised linears", flush=True)
    model = random_awq_qwen3(TINY, seed=5, std=0.05)
    ids = torch.randint(0, 512, (2, 24), device="cuda")
    pos = torch.arange(24, device="cuda").unsqueeze(0)
    h = model(ids, pos).float()
    # same network with every AWQ linear replaced by x @ dequant(W) in fp32
    import torch.nn.functional as F

    class Deq(torch.nn.Module):
        def __init__(self, m):
            super().__init__()
            self.w = nq.awq_dequantize(m.qweight, m.qscales, m.qzeros).float()
        def forward(self, x):
            return (x.float() @ self.w).to(x.dtype)

    import copy
    ref = copy.deepcopy(model)
    for blk in ref.model.layers:
        for parent, names in ((blk.self_attn, ("q_proj", "k_proj", "v_proj", "o_proj")), (blk.mlp, ("gate_proj", "up_proj", "down_proj"))):
            for nme in names:
                setattr(parent, nme, Deq(getattr(parent, nme)))
    h_ref = ref(ids, pos).float()
    err = (h - h_ref).abs().max().item() / h_ref.abs().max().item()
    assert err <= 3e-2, err


@pytest.mark.gpu
def test_engine_at_qwen3_32b_widths():
    """Two blocks of the Qwen3-32B architecture at its real widths (hidden 5120, 64 q / 8 kv heads,
    intermediate 25600, vocabulary 151936): batch-64 decode shapes (idle rows included), 8 query heads per kv
    head in the paged attention, the pipelined GEMM in the recompute.  Same check as the small model: the
    engine's own continuation, teacher-forced through the full-recompute forward, must be that forward's
    argmax wherever the logits are not near-tied."""
    from nanoquantization_amd.engine import LLMEngine
    from nanoquantization_amd.models.random_init import QWEN3_32B, random_awq_qwen3
    print("engine at Qwen3-32B widths, 2 layers", flush=True)
    cfg = dict(QWEN3_32B, num_hidden_layers=2, max_position_embeddings=512)
    model = random_awq_qwen3(cfg, seed=5, std=0.02)
    torch.manual_seed(6)
    plen, new = 37, 6
    prompts = torch.randint(0, cfg["vocab_size"], (3, plen)).tolist()
    eng = LLMEngine(model, max_batch=64, max_seq_len=128, block_size=64, use_graph=True)
    got = eng.generate(prompts, new)
    seqs = torch.tensor([p + g for p, g in zip(prompts, got)], device="cuda")
    pos = torch.arange(seqs.shape[1], device="cuda").unsqueeze(0)
    logits = model.lm_head(model(seqs, pos)).float()[:, plen - 1:-1]
    chosen = torch.tensor(got, device="cuda")
    gap = logits.max(-1).values - logits.gather(-1, chosen.unsqueeze(-1)).squeeze(-1)
    scale = logits.abs().max().item()
    assert gap.max().item() <= 2e-2 * scale, (gap.max().item(), scale)
    top2 = logits.topk(2, dim=-1).values
    clear = (top2[..., 0] - top2[..., 1]) > 4e-2 * scale
    assert torch.equal(chosen[clear], logits.argmax(-1)[clear])
    assert eng.generate(prompts, new) == got


@pytest.mark.gpu
def test_engine_continuous_batching():
    """serve(): ragged prompts, more requests than batch rows, different token budgets.  Every request's
    continuation, teacher-forced through the full-recompute forward, must be that forward's argmax wherever the
    logits are not near-tied; rows and cache blocks are all given back; an end-of-sequence token cuts a request."""
    from nanoquantization_amd.engine import LLMEngine
    from nanoquantization_amd.models.random_init import random_awq_qwen3
    print("engine continuous batching", flush=True)
    model = random_awq_qwen3(TINY, seed=7, std=0.05)
    g = torch.Generator().manual_seed(8)
    lens = [5, 19, 33, 7, 12, 40, 3, 26, 9]
    budgets = [6, 3, 9, 1, 12, 4, 8, 5, 7]
    reqs = [(torch.randint(0, 512, (n,), generator=g).tolist(), m) for n, m in zip(lens, budgets)]
    eng = LLMEngine(model, max_batch=4, max_seq_len=64, block_size=16, use_graph=True)
    total_blocks = len(eng.cache.free)
    st = {}
    got = eng.serve(reqs, stats=st)
    assert [len(o) for o in got] == budgets
    assert len(eng.cache.free) == total_blocks and st["prefills"] == len(reqs)
    assert st["decode_steps"] < sum(b - 1 for b in budgets), "requests must share decode steps"
    def check_against_recompute(conts):
        for (prompt, _), cont in zip(reqs, conts):
            seq = torch.tensor([prompt + cont], device="cuda")
            pos = torch.arange(seq.shape[1], device="cuda").unsqueeze(0)
            logits = model.lm_head(model(seq, pos)).float()[0, len(prompt) - 1:-1]
            chosen = torch.tensor(cont, device="cuda")
            gap = logits.max(-1).values - logits.gather(-1, chosen.unsqueeze(-1)).squeeze(-1)
            scale = logits.abs().max().item()
            assert gap.max().item() <= 2e-2 * scale
            top2 = logits.topk(2, dim=-1).values
            clear = (top2[..., 0] - top2[..., 1]) > 4e-2 * scale
            assert torch.equal(chosen[clear], logits.argmax(-1)[clear])

    check_against_recompute(got)
    # the same requests again (the captured graph and the freed blocks are reused) give the same tokens
    assert eng.serve(reqs) == got
    # requests admitted together prefilled in one ragged pass: fewer prefill launches, same check
    stb = {}
    gotb = eng.serve(reqs, stats=stb, batch_prefill=True)
    assert [len(o) for o in gotb] == budgets and stb["prefills"] == len(reqs) and stb["prefill_calls"] < len(reqs)
    check_against_recompute(gotb)
    assert len(eng.cache.free) == total_blocks
    assert eng.serve(reqs, batch_prefill=True) == gotb
    # end-of-sequence: pick a token that some request emits mid-way and check the cut
    ri = max(range(len(got)), key=lambda i: len(got[i]))
    eos = got[ri][len(got[ri]) // 2]
    cut = eng.serve(reqs, eos_token_id=eos)
    for a, b in zip(cut, got):
        want = b[: b.index(eos) + 1] if eos in b else b
        assert a == want
    assert len(eng.cache.free) == total_blocks
    # a request that can never fit is refused, not queued forever
    small = LLMEngine(model, max_batch=2, max_seq_len=64, block_size=16, num_blocks=2, use_graph=False)
    with pytest.raises(RuntimeError, match="KV cache too small"):
        small.serve([(list(range(40)), 8)])


@pytest.mark.gpu
def test_engine_norm_fused_decode_equals_separate_kernels():
    """The decode step with the residual adds and RMSNorms folded into the GEMVs (five launches per block) produces
    the tokens of the step with stand-alone add + norm kernels (seven): every fused piece returns the same bits."""
    from nanoquantization_amd.engine import LLMEngine
    from nanoquantization_amd.models.random_init import random_awq_qwen3
    print("engine: norm-fused decode vs separate kernels", flush=True)
    cfg = dict(TINY, hidden_size=512, head_dim=128, intermediate_size=768)
    model = random_awq_qwen3(cfg, seed=11, std=0.05)
    torch.manual_seed(12)
    prompts = torch.randint(0, 512, (5, 23)).tolist()
    outs = []
    for fuse in (False, True):
        eng = LLMEngine(model, max_batch=8, max_seq_len=96, block_size=16, use_graph=True, fuse_norm=fuse)
        assert eng.norm_fused_ok == fuse
        # the static batch, then the same engine under continuous batching with ragged requests
        reqs = [(p[: 5 + 3 * i], 6 + i) for i, p in enumerate(prompts)]
        outs.append((eng.generate(prompts, 20), eng.serve(reqs)))
    assert outs[0] == outs[1]


def _teacher_forced_check(model, prompts, got, rows=None, gap_tol=2e-2):
    """The engine's own continuation pushed through the full-recompute forward (the reference semantics: no cache):
    every chosen token is that forward's argmax up to the 16-bit noise of a near-tie, and exactly it wherever the
    logits are not near-tied.  `rows` limits the recompute to some sequences.  `gap_tol` (a fraction of the largest
    logit) is the near-tie noise allowed; it grows with depth -- measured on these random-weight stacks at the
    Qwen3-32B widths over 256 decoded tokens: at most 0.010 with 2 blocks, 0.015 with 8, 0.026 with 32, 0.066 with
    64, while a token from a wrong cache row or position lands about 1.0 away."""
    rows = list(range(len(prompts))) if rows is None else rows
    plen = len(prompts[0])
    seqs = torch.tensor([prompts[r] + got[r] for r in rows], device="cuda")
    pos = torch.arange(seqs.shape[1], device="cuda").unsqueeze(0)
    hidden = model(seqs, pos)[:, plen - 1:-1]
    logits = model.lm_head(hidden).float()
    chosen = torch.tensor([got[r] for r in rows], device="cuda")
    gap = logits.max(-1).values - logits.gather(-1, chosen.unsqueeze(-1)).squeeze(-1)
    scale = logits.abs().max().item()
    assert gap.max().item() <= gap_tol * scale, (gap.max().item(), scale)
    top2 = logits.topk(2, dim=-1).values
    clear = (top2[..., 0] - top2[..., 1]) > 2 * gap_tol * scale
    assert torch.equal(chosen[clear], logits.argmax(-1)[clear])
    return clear.float().mean().item()


@pytest.mark.gpu
def test_engine_full_qwen3_0p6b_architecture_batch_32():
    """The whole Qwen3-0.6B architecture (28 blocks, hidden 1024, 16 q / 8 kv heads, intermediate 3072, vocabulary
    151,936, tied head) at batch 32 with 96-token prompts: the graph-captured decode step with every fused GEMV form,
    against the full-recompute forward."""
    from nanoquantization_amd.engine import LLMEngine
    from nanoquantization_amd.models.random_init import QWEN3_0P6B, random_awq_qwen3
    print("engine: Qwen3-0.6B architecture, 28 layers, batch 32", flush=True)
    cfg = dict(QWEN3_0P6B, max_position_embeddings=1024)
    model = random_awq_qwen3(cfg, seed=21, std=0.02)
    torch.manual_seed(22)
    plen, new = 96, 6
    prompts = torch.randint(0, cfg["vocab_size"], (32, plen)).tolist()
    eng = LLMEngine(model, max_batch=32, max_seq_len=128, block_size=64, use_graph=True)
    assert eng.norm_fused_ok and eng.qkv_fused_ok and eng.swiglu_ok
    got = eng.generate(prompts, new)
    assert len(got) == 32 and all(len(g) == new for g in got)
    _teacher_forced_check(model, prompts, got)
    assert eng.generate(prompts, new) == got


@pytest.mark.gpu
def test_engine_full_qwen3_0p6b_architecture_full_length():
    """The same architecture at the full length of the small end-to-end configuration: 32 sequences, 512-token
    prompts, 256 new tokens each (contexts of 512..767 tokens, 8..12 cache blocks per sequence, 256 replays of the
    captured decode step), against the full-recompute forward on a sample of the sequences."""
    from nanoquantization_amd.engine import LLMEngine
    from nanoquantization_amd.models.random_init import QWEN3_0P6B, random_awq_qwen3
    print("engine: Qwen3-0.6B architecture, 28 layers, batch 32, 512 + 256 tokens", flush=True)
    cfg = dict(QWEN3_0P6B, max_position_embeddings=1024)
    model = random_awq_qwen3(cfg, seed=25, std=0.02)
    torch.manual_seed(26)
    plen, new = 512, 256
    prompts = torch.randint(0, cfg["vocab_size"], (32, plen)).tolist()
    eng = LLMEngine(model, max_batch=32, max_seq_len=plen + new, block_size=64, use_graph=True)
    got = eng.generate(prompts, new)
    assert len(got) == 32 and all(len(g) == new for g in got)
    clear = _teacher_forced_check(model, prompts, got, rows=[0, 17, 31])
    assert clear > 0.2, clear   # a good share of the steps has a clear winner: the exact comparison is not vacuous


@pytest.mark.gpu
@pytest.mark.timeout(600)
def test_engine_full_qwen3_32b_architecture_batch_64_context_2048():
    """The largest configuration at full depth: all 64 blocks of the Qwen3-32B architecture (16 GB of packed weights),
    64 sequences of 2,048 prompt tokens (one 131,072-token prefill pass through the fused GEMM), then captured decode
    steps at 64 rows over 2,048..2,050 cached tokens per sequence, against the full-recompute forward on two of the
    sequences."""
    from nanoquantization_amd.engine import LLMEngine
    from nanoquantization_amd.models.random_init import QWEN3_32B, random_awq_qwen3
    print("engine: Qwen3-32B architecture, 64 layers, batch 64, context 2048", flush=True)
    cfg = dict(QWEN3_32B, max_position_embeddings=4096)
    model = random_awq_qwen3(cfg, seed=27, std=0.02)
    torch.manual_seed(28)
    plen, new = 2048, 3
    prompts = torch.randint(0, cfg["vocab_size"], (64, plen)).tolist()
    eng = LLMEngine(model, max_batch=64, max_seq_len=plen + 64, block_size=64, use_graph=True)
    assert eng.o_add_norm and eng.down_add_norm
    got = eng.generate(prompts, new)
    assert len(got) == 64 and all(len(g) == new for g in got)
    _teacher_forced_check(model, prompts, got, rows=[0, 21, 42, 63], gap_tol=0.12)   # 64 blocks deep
    del eng, model
    torch.cuda.empty_cache()


@pytest.mark.gpu
def test_engine_qwen3_32b_widths_batch_64_context_2048():
    """Two blocks at the Qwen3-32B widths with 64 sequences of 2,048 cached tokens each: the decode shapes of the
    largest configuration (64-row GEMVs on the shared-chunk kernel, paged attention over 32 blocks per sequence with 8
    query heads per kv head), a 131,072-token batched prefill through the fused GEMM, against the recompute forward
    on a sample of the sequences."""
    from nanoquantization_amd.engine import LLMEngine
    from nanoquantization_amd.models.random_init import QWEN3_32B, random_awq_qwen3
    print("engine: Qwen3-32B widths, 2 layers, batch 64, context 2048", flush=True)
    cfg = dict(QWEN3_32B, num_hidden_layers=2, max_position_embeddings=4096)
    model = random_awq_qwen3(cfg, seed=23, std=0.02)
    torch.manual_seed(24)
    plen, new = 2048, 4
    prompts = torch.randint(0, cfg["vocab_size"], (64, plen)).tolist()
    eng = LLMEngine(model, max_batch=64, max_seq_len=plen + 64, block_size=64, use_graph=True)
    got = eng.generate(prompts, new)
    assert len(got) == 64 and all(len(g) == new for g in got)
    _teacher_forced_check(model, prompts, got, rows=[0, 13, 31, 63])


@pytest.mark.gpu
def test_engine_qwen3_14b_widths_five_heads_per_kv_head():
    """Two blocks at the Qwen3-14B widths (hidden 5120, 40 query / 8 kv heads, intermediate 17408): five query heads
    per kv head, a ratio only the matrix-core attention kernel takes (the count at run time), at 16 and at 64 rows --
    the 16 rows on 16-token cache blocks, where every 32-token tile of the kernel spans two table entries."""
    from nanoquantization_amd.engine import LLMEngine
    from nanoquantization_amd.models.random_init import QWEN3_32B, random_awq_qwen3
    print("engine: Qwen3-14B widths, 2 layers", flush=True)
    cfg = dict(QWEN3_32B, total_num_heads=40, intermediate_size=17408, num_hidden_layers=2,
               max_position_embeddings=1024, vocab_size=32000)
    model = random_awq_qwen3(cfg, seed=51, std=0.02)
    torch.manual_seed(52)
    plen, new = 150, 4
    for B, bs in ((16, 16), (64, 64)):
        prompts = torch.randint(0, cfg["vocab_size"], (B, plen)).tolist()
        eng = LLMEngine(model, max_batch=B, max_seq_len=plen + 42, block_size=bs, use_graph=True)
        got = eng.generate(prompts, new)
        assert len(got) == B and all(len(g) == new for g in got)
        _teacher_forced_check(model, prompts, got, rows=[0, B // 3, B - 1])


@pytest.mark.gpu
def test_engine_qwen3_8b_widths_batch_64():
    """Two blocks at the Qwen3-8B widths (hidden 4096, 32 query / 8 kv heads, intermediate 12288) with 64 rows: here
    only down_proj (12288 x 4096) and gate|up have a K-split shared-chunk plan, so the decode step mixes the routes --
    q|k|v on the one-tile kernel with its own epilogue, o_proj followed by the stand-alone add + norm kernel,
    down_proj with the add + norm in its second pass, attention at 4 query heads per kv head."""
    from nanoquantization_amd.engine import LLMEngine
    from nanoquantization_amd.models.random_init import QWEN3_32B, random_awq_qwen3
    print("engine: Qwen3-8B widths, 2 layers, batch 64", flush=True)
    cfg = dict(QWEN3_32B, hidden_size=4096, intermediate_size=12288, total_num_heads=32, total_num_kv_heads=8,
               num_hidden_layers=2, max_position_embeddings=1024, vocab_size=32000)
    model = random_awq_qwen3(cfg, seed=41, std=0.02)
    torch.manual_seed(42)
    plen, new = 200, 4
    prompts = torch.randint(0, cfg["vocab_size"], (64, plen)).tolist()
    eng = LLMEngine(model, max_batch=64, max_seq_len=plen + 56, block_size=64, use_graph=True)
    assert eng.down_add_norm and not eng.o_add_norm and not eng.norm_fused_ok
    got = eng.generate(prompts, new)
    assert len(got) == 64 and all(len(g) == new for g in got)
    _teacher_forced_check(model, prompts, got, rows=[0, 21, 63])


@pytest.mark.gpu
def test_engine_mixed_decode_and_long_prefill_qwen3_32b_widths():
    """The mixed run of the largest configuration in miniature: two blocks at the Qwen3-32B widths, one serve() call in
    which eight rows decode at a context of 1,024 and more while a longer request (1,536 tokens) waits, is admitted
    when the first row frees and is prefilled between two decode steps of the other rows.  Every request's
    continuation is checked against the full-recompute forward."""
    from nanoquantization_amd.engine import LLMEngine
    from nanoquantization_amd.models.random_init import QWEN3_32B, random_awq_qwen3
    print("engine: mixed decode + long prefill at Qwen3-32B widths, 2 layers", flush=True)
    cfg = dict(QWEN3_32B, num_hidden_layers=2, max_position_embeddings=2048)
    model = random_awq_qwen3(cfg, seed=31, std=0.02)
    rg = torch.Generator().manual_seed(32)
    B, P, LONG = 8, 1024, 1536
    prompts = torch.randint(0, cfg["vocab_size"], (B, P), generator=rg).tolist()
    long_prompt = torch.randint(0, cfg["vocab_size"], (LONG,), generator=rg).tolist()
    reqs = [(p, 3 if i == 0 else 8) for i, p in enumerate(prompts)] + [(long_prompt, 4)]
    eng = LLMEngine(model, max_batch=B, max_seq_len=LONG + 64, block_size=64, use_graph=True)
    st = {}
    got = eng.serve(reqs, stats=st, batch_prefill=True, max_prefill_tokens=4 * P)
    assert [len(g) for g in got] == [m for _, m in reqs]
    long_pf = [p for p in st["prefill_log"] if p[0] == LONG]
    assert len(long_pf) == 1 and long_pf[0][1] == 1, st["prefill_log"]
    assert 1 <= long_pf[0][2] < st["decode_steps"], "the long prefill must sit between decode steps of the other rows"
    for (prompt, _), cont in zip(reqs, got):
        _teacher_forced_check(model, [prompt], [cont])
    assert eng.serve(reqs, batch_prefill=True, max_prefill_tokens=4 * P) == got


@pytest.mark.gpu
@pytest.mark.timeout(900)
def test_engine_mixed_run_full_qwen3_32b_architecture():
    """The mixed run of the largest configuration at full size: all 64 blocks of the Qwen3-32B architecture, one
    serve() call with 64 requests of 2,048 prompt tokens and a 4,096-token request that is admitted when the first
    row frees and prefilled between two decode steps of the other 63 rows.  Three of the continuations (a short
    request, a long-running one and the 4,096-token one) are checked against the full-recompute forward."""
    from nanoquantization_amd.engine import LLMEngine
    from nanoquantization_amd.models.random_init import QWEN3_32B, random_awq_qwen3
    print("engine: mixed decode + 4096-token prefill, Qwen3-32B architecture, 64 layers, batch 64", flush=True)
    cfg = dict(QWEN3_32B, max_position_embeddings=8192)
    model = random_awq_qwen3(cfg, seed=33, std=0.02)
    rg = torch.Generator().manual_seed(34)
    B, P, LONG = 64, 2048, 4096
    prompts = torch.randint(0, cfg["vocab_size"], (B, P), generator=rg).tolist()
    long_prompt = torch.randint(0, cfg["vocab_size"], (LONG,), generator=rg).tolist()
    reqs = [(p, 3 if i == 0 else 8) for i, p in enumerate(prompts)] + [(long_prompt, 4)]
    eng = LLMEngine(model, max_batch=B, max_seq_len=LONG + 64, block_size=64, use_graph=True)
    st = {}
    got = eng.serve(reqs, stats=st, batch_prefill=True, max_prefill_tokens=4 * P)
    assert [len(g) for g in got] == [m for _, m in reqs]
    long_pf = [p for p in st["prefill_log"] if p[0] == LONG]
    assert len(long_pf) == 1 and long_pf[0][1] == 1, st["prefill_log"]
    assert 1 <= long_pf[0][2] < st["decode_steps"], "the long prefill must sit between decode steps of the other rows"
    for i in (0, 37, B):
        _teacher_forced_check(model, [reqs[i][0]], [got[i]], gap_tol=0.12)   # 64 blocks deep
    del eng, model
    torch.cuda.empty_cache()


@pytest.mark.gpu
@pytest.mark.parametrize("group_size,max_batch", [(64, 4), (128, 65), (32, 3)])
def test_engine_shapes_outside_the_fused_decode_forms(group_size, max_batch):
    """Group sizes 32 / 64 and widths that are not multiples of 128 (the register-path GEMV, no q|k|v / gate|up / norm
    fusion), and more than 64 batch rows (the decode linears on the MFMA GEMM): the engine issues its prefetch hints
    before every linear whatever kernel takes it; nothing may be left pending or fail."""
    from nanoquantization_amd import _lib
    from nanoquantization_amd.engine import LLMEngine
    from nanoquantization_amd.models.random_init import random_awq_qwen3
    print(f"engine: group size {group_size}, max_batch {max_batch}", flush=True)
    cfg = TINY if group_size == 128 else dict(TINY, hidden_size=192, total_num_heads=4, total_num_kv_heads=2,
                                              head_dim=64, intermediate_size=320)
    model = random_awq_qwen3(cfg, seed=31, std=0.05, group_size=group_size)
    torch.manual_seed(32)
    n = min(max_batch, 5)
    prompts = torch.randint(0, 512, (n, 21)).tolist()
    for use_graph in (False, True):
        eng = LLMEngine(model, max_batch=max_batch, max_seq_len=64, block_size=16, use_graph=use_graph)
        assert not eng.norm_fused_ok and not eng.qkv_fused_ok
        got = eng.generate(prompts, 8)
        assert _lib.lib().awq_prefetch_pending() == 0
        assert _teacher_forced_check(model, prompts, got) > 0.5


def test_paged_kv_cache_block_bookkeeping():
    """Host logic of the cache: blocks are handed out once, come back on release, exhaustion raises (CPU)."""
    from nanoquantization_amd.engine.llm_engine import PagedKVCache
    c = PagedKVCache(num_layers=2, num_blocks=6, block_size=4, num_kv_heads=2, head_dim=8, dtype=torch.bfloat16,
                     device=torch.device("cpu"))
    assert c.k.shape == (2, 6, 2, 4, 8) and c.v.shape == c.k.shape
    a = c.allocate(4)
    b = c.allocate(2)
    assert sorted(a + b) == list(range(6)) and len(c.free) == 0
    with pytest.raises(RuntimeError, match="KV cache exhausted"):
        c.allocate(1)
    c.release(a)
    assert sorted(c.free) == sorted(a)
    assert sorted(c.allocate(3) + c.free) == sorted(a)
