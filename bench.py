#!/usr/bin/env python3
"""Benchmark of the AWQ W4A16 linear path on one MI355X.

Headline (`value`): packed-weight GB/s of the decode GEMV sweep -- M in {1,2,4,8,16} over every
Qwen3-0.6B linear shape, fp16, g=128 -- streaming from HBM: one step walks LAYERS distinct copies of
the 7 linears of a block (LAYERS * 8.17 MB of packed weights, more than twice the 256 MB Infinity
Cache) once per M.  The step is captured in a HIP graph (the form a decode loop runs in); the eager
number is reported next to it.

Also on the JSON line: `roofline` for the GEMV kernel of that sweep, `cpu_baseline` (the torch
restatement of the reference path on the host cores, bounded sample), and -- as extra objects, not the
headline -- the same GEMV on the Qwen3-32B MLP shapes where a launch is long enough to be HBM-bound,
the prefill GEMM TFLOP/s at the Qwen3-8B MLP shapes, the dequantise kernel, and config 1's latency.

python bench.py [--gpus 1] [--steps K] [--warmup W] [--quick] [--no-cfg5] [--only-cfg5] [--no-cpu]

For a profiler or a counter collection to look at one kernel (no timing, no JSON line):
python bench.py --one linear|dequant|copy K N M [--one-dtype bf16|f16] [--one-iters 6] [--one-copies 1]
launches that one problem a few times on seeded buffers, walking over `--one-copies` distinct packed weights (more
than the 256 MB Infinity Cache holds: the launches stream from HBM as the timed sections do).  `copy`: a device copy
of the packed weight, the known-size kernel the traffic counters are calibrated with.
"""
from __future__ import annotations

import argparse
import re
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# HBM bytes per GEMV launch of the headline sweep, from two `rocprofv3 --pmc` runs of this file
# (FETCH_SIZE, then WRITE_SIZE; profiles/gemv_cfg2_sweep_hbm_traffic.txt).  Each counter is scaled by
# what it reads for a device-to-device copy of 65,536,000 bytes: FETCH_SIZE 32,012.8 -> 2047.2 B per count,
# WRITE_SIZE 64,000 -> 1024 B per count.
MEASURED_FETCH_BYTES_PER_LAUNCH = 1129.27 * 2047.2
MEASURED_WRITE_BYTES_PER_LAUNCH = 100.68 * 1024.0

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_PEAK_TFLOPS = 2500.0      # dense fp16/bf16, published
QWEN3_0P6B = [("q", 1024, 2048), ("k", 1024, 1024), ("v", 1024, 1024), ("o", 2048, 1024),
              ("gate", 1024, 3072), ("up", 1024, 3072), ("down", 3072, 1024)]
DECODE_MS = (1, 2, 4, 8, 16)
G = 128


def packed_bytes(K, N, g=G):
    return K * N // 2 + (K // g) * N // 2 + 2 * (K // g) * N


def rand_packed(K, N, tdt, dev, g=G):
    """Random nibbles/zeros/scales straight on the device (bandwidth does not depend on the values)."""
    qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (K, N // 8), dtype=torch.int32, device=dev)
    qz = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // g, N // 8), dtype=torch.int32, device=dev)
    sc = (torch.rand(K // g, N, device=dev) * 0.02 + 0.001).to(tdt)
    return qw, sc, qz


def decode_step_bytes(model, ctx_tokens):
    """Algorithmic HBM bytes of one decode step: every packed AWQ buffer and the dense lm_head read once, plus the
    K and V rows of `ctx_tokens` cached tokens (summed over the batch) in every layer."""
    from nanoquantization_amd.layers.gemm import WQLinear_GEMM
    wbytes = 0
    for m in model.modules():
        if isinstance(m, WQLinear_GEMM):
            wbytes += m.qweight.numel() * 4 + m.qzeros.numel() * 4 + m.qscales.numel() * m.qscales.element_size()
    head = model.lm_head.weight
    a0 = model.model.layers[0].self_attn
    kv = ctx_tokens * len(model.model.layers) * 2 * a0.num_kv_heads * a0.head_dim * head.element_size()
    return {"awq_weights": wbytes, "lm_head": head.numel() * head.element_size(), "kv_cache": int(kv),
            "total": int(wbytes + head.numel() * head.element_size() + kv)}


def step_roofline(nbytes, ms_per_step, kernel):
    gbs = nbytes["total"] / (ms_per_step * 1e-3) / 1e9
    return {"kernel": kernel, "bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(gbs / HBM_PEAK_GBS, 4), "algorithmic_bytes_per_step": nbytes,
            "note": "whole decode step (all launches of the graph), not one kernel: packed weights + lm_head + cached "
                    "K/V of the batch, each read once, / wall time per step"}


def time_graph(fn, steps, warmup):
    """Capture fn() once on a side stream, replay `steps` times between two events on that stream."""
    s = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(s):
        fn()                              # allocations (outputs, workspace) happen before capture
        torch.cuda.synchronize()
        with torch.cuda.graph(g, stream=s):
            fn()
        torch.cuda.synchronize()
        for _ in range(warmup):
            g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(s)
        for _ in range(steps):
            g.replay()
        e1.record(s)
        torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps    # ms per step


def time_eager(fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def run_one(kind, K, N, M, dtype, iters, copies=1, g=G):
    """One problem, `iters` launches over `copies` distinct weights, nothing timed: the subject of a rocprofv3 run."""
    import nanoquantization_amd as nq
    dev = torch.device("cuda:0")
    tdt = torch.bfloat16 if dtype == "bf16" else torch.float16
    gen = torch.Generator(device=dev).manual_seed(K + N)
    ws = []
    for _ in range(max(1, copies)):
        qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (K, N // 8), dtype=torch.int32, device=dev, generator=gen)
        qz = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // g, N // 8), dtype=torch.int32, device=dev, generator=gen)
        qs = (torch.rand(K // g, N, device=dev, generator=gen) * 0.02 + 0.001).to(tdt)
        ws.append((qw, qs, qz))
    x = torch.randn(max(M, 1), K, device=dev, generator=gen).to(tdt)
    fn = {"linear": lambda w: nq.awq_gemm(x, w[0], w[1], w[2], 8),
          "dequant": lambda w: nq.awq_dequantize(*w), "copy": lambda w: w[0].clone()}[kind]
    for i in range(iters):
        fn(ws[i % len(ws)])
    torch.cuda.synchronize()
    print(f"{kind} K={K} N={N} M={M} {dtype}: {iters} launches over {len(ws)} weight copies")


def gemm_kernel_name(M, N, K, dtype_name, g=G):
    """The kernel awq_gemm runs for a prefill problem, from the library's own plan."""
    import ctypes
    from nanoquantization_amd import _lib
    L = _lib.lib()
    v, sp = ctypes.c_int(), ctypes.c_int()
    did = _lib.AWQ_F16 if dtype_name == "f16" else _lib.AWQ_BF16
    if L.awq_gemm_plan(M, N, K, g, did, ctypes.byref(v), ctypes.byref(sp)) != 0:
        return "?"
    name = L.awq_gemm_variant_name(v.value).decode()
    T = "F16" if dtype_name == "f16" else "BF16"
    kern = {"256x256p": f"awq::gemm_pipe_kernel<{T},2,4>", "256x256pt": f"awq::gemm_pipe_kernel<{T},2,4>",
            "256x256r": f"awq::gemm_regb_kernel<{T}>", "256x256rt": f"awq::gemm_regb_kernel<{T}>"}.get(
                name, f"awq::gemm_kernel<{T},{name}>")
    return f"{kern} (plan {name}, split {sp.value})"


def gemv_kernel_name(M, N, K, dtype_name, g=G):
    """The kernel awq_gemv runs for a decode problem, from the library's own plan."""
    import ctypes
    from nanoquantization_amd import _lib
    L = _lib.lib()
    v, sp = ctypes.c_int(), ctypes.c_int()
    if L.awq_gemv_plan(M, N, K, g, ctypes.byref(v), ctypes.byref(sp)) != 0:
        return "?"
    name = L.awq_gemv_variant_name(v.value).decode()
    T = "F16" if dtype_name == "f16" else "BF16"
    wide = re.fullmatch(r"wide(2?)d(\d)m(\d)(t?)", name)   # wide[2]d<DEPTH>m<MT>[t]: 256 columns per workgroup, in-kernel tail
    if wide:
        wn = 2 if wide.group(1) else 4
        kern = f"awq::gemv_wide_kernel<{T},{wide.group(2)},{wide.group(3)},{'true' if wide.group(4) else 'false'},{wn}>"
        if not wide.group(4):   # the K splits are added by a second kernel
            kern += f" + awq::gemv_wide_reduce_kernel<{T}>"
    elif name.startswith("dma"):
        kern = f"awq::gemv_dma_kernel<{T},{name[5]},plain>"
    else:
        kern = f"awq::gemv_kernel<{T}> ({name})"
    return f"{kern} (plan {name}, split {sp.value})"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--one", nargs=4, metavar=("KIND", "K", "N", "M"),
                    help="launch one problem a few times for a profiler: linear|dequant|copy K N M")
    ap.add_argument("--one-dtype", choices=["bf16", "f16"], default="bf16")
    ap.add_argument("--one-iters", type=int, default=6)
    ap.add_argument("--one-copies", type=int, default=1)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--layers", type=int, default=64, help="distinct weight copies of one block per step")
    ap.add_argument("--quick", action="store_true", help="skip the extra (non-headline) measurements")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--only-cfg5", action="store_true",
                    help="with the headline, run only the Qwen3-32B-architecture section of the extra measurements")
    ap.add_argument("--no-cfg5", action="store_true",
                    help="skip the Qwen3-32B-architecture section (about 90 GB of device memory, a minute)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the AWQ linear path has no multi-GPU part); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no HIP device visible", file=sys.stderr)
        sys.exit(1)

    from nanoquantization_amd import _lib
    import nanoquantization_amd as nq
    if not (os.path.exists(_lib.LIB_PATH) and os.path.exists(_lib.TORCH_LIB_PATH)):
        from nanoquantization_amd.build import build
        build(verbose=False)
    _lib.lib()

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.one:
        kind, K1, N1, M1 = args.one[0], int(args.one[1]), int(args.one[2]), int(args.one[3])
        if kind not in ("linear", "dequant", "copy"):
            ap.error("--one KIND must be linear, dequant or copy")
        run_one(kind, K1, N1, M1, args.one_dtype, args.one_iters, args.one_copies)
        return
    tdt = torch.float16
    torch.manual_seed(0)

    # ---------------- headline: decode GEMV sweep, streaming ----------------------------------------------
    layers = [[rand_packed(K, N, tdt, dev) for (_, K, N) in QWEN3_0P6B] for _ in range(args.layers)]
    xs = {(M, K): torch.randn(M, K, device=dev).to(tdt) for M in DECODE_MS for K in (1024, 2048, 3072)}
    bytes_per_pass = sum(packed_bytes(K, N) for (_, K, N) in QWEN3_0P6B) * args.layers
    launches_per_step = len(DECODE_MS) * len(QWEN3_0P6B) * args.layers
    bytes_per_step = bytes_per_pass * len(DECODE_MS)

    flat = [(w, K) for layer in layers for w, (_, K, N) in zip(layer, QWEN3_0P6B)]

    def sweep_step():
        # like a decode loop, every launch names the packed weight of the launch after it: spare workgroups
        # of the (small) GEMV grid pull it into the Infinity Cache (awq_prefetch_hint)
        for M in DECODE_MS:
            for i, ((qw, sc, qz), K) in enumerate(flat):
                nq.prefetch_hint(*flat[(i + 1) % len(flat)][0][:2])        # qweight, qscales
                nq.awq_gemm(xs[(M, K)], qw, sc, qz, 8)

    ms_graph = time_graph(sweep_step, args.steps, args.warmup)
    ms_eager = time_eager(sweep_step, max(2, args.steps // 4), 1)
    value = bytes_per_step / (ms_graph * 1e-3) / 1e9
    avg_launch_us = ms_graph * 1e3 / launches_per_step
    avg_bytes = bytes_per_step / launches_per_step
    roofline = {
        "kernel": "awq::gemv_dma_kernel<F16, WK=4|8, plain, one chunk per wave>", "bound": "hbm",
        "achieved": avg_bytes / (avg_launch_us * 1e-6) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": avg_bytes / (avg_launch_us * 1e-6) / 1e9 / HBM_PEAK_GBS,
        "traffic": MEASURED_FETCH_BYTES_PER_LAUNCH + MEASURED_WRITE_BYTES_PER_LAUNCH,
        "traffic_note": "bytes per launch crossing the L2/fabric boundary (fetch 2.32 MB + write 0.10 MB) from rocprofv3 "
                        "FETCH_SIZE / WRITE_SIZE, copy-calibrated.  The counters sit between the L2s and the fabric "
                        "and cannot tell Infinity Cache hits from HBM reads: about 0.87 MB of the fetch is the prefetch "
                        "(spare workgroups read the next launch's weights once to park them in the Infinity Cache, "
                        "the consumer reads them again from there); the remaining 1.45 MB is 1.24 x the packed "
                        "weights (x, scales, zeros per workgroup; lines shared across XCDs on the 16-tile shape); "
                        "the writes are split-K partials.  At the 68 MB shapes fetch = 1.05 x algorithmic",
        "avg_launch_us": avg_launch_us, "algorithmic_bytes_per_launch": avg_bytes,
        "note": "packed-weight bytes (0.5195 B/weight) / HIP-event time per launch over the timed graph replays; "
                "0.5-1.6 MB per launch: latency-bound, see roofline_large for the HBM-bound regime",
    }

    # per-shape hot-cache numbers (single buffer, stays in L2 / Infinity Cache), labelled as such
    per_shape = {}
    for (name, K, N), w in zip(QWEN3_0P6B, layers[0]):
        for M in (1, 16):
            fn = lambda: [nq.awq_gemm(xs[(M, K)], *w, 8) for _ in range(50)]
            us = time_graph(fn, 5, 1) * 1e3 / 50
            per_shape[f"{name}_{K}x{N}_M{M}"] = {"hot_us": round(us, 2),
                                                   "hot_GBs": round(packed_bytes(K, N) / us / 1e3, 1)}
    del layers
    torch.cuda.empty_cache()

    out = {
        "metric": "W4A16 GEMM TFLOP/s & weight GB/s vs roofline; Qwen3-0.6B decode tok/s",
        "value": value, "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_graph,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "cfg2: decode GEMV sweep, M in {1,2,4,8,16} x Qwen3-0.6B linear shapes "
                               "(q 1024x2048, k/v 1024x1024, o 2048x1024, gate/up 1024x3072, down 3072x1024), "
                               "fp16 x ~N(0,1), AWQ-packed g=128",
                   "distinct_weight_copies": args.layers, "launches_per_step": launches_per_step,
                   "packed_bytes_per_step": bytes_per_step,
                   "launch": "HIP graph replay; each launch prefetches the next launch's packed weights into the "
                             "Infinity Cache with workgroups its own grid leaves idle (awq_prefetch_hint)",
                   "eager_GBs": bytes_per_step / (ms_eager * 1e-3) / 1e9, "eager_ms_per_step": ms_eager},
        "roofline": roofline,
        "per_shape_hot_cache": per_shape,
    }

    if not args.quick and not args.only_cfg5:
        # ---------------- extra: HBM-bound GEMV at the Qwen3-32B MLP shapes -----------------------------
        large, batched = {}, {}
        for (K, N) in ((5120, 25600), (25600, 5120)):
            copies = [rand_packed(K, N, tdt, dev) for _ in range(6)]   # 6 x 68 MB > Infinity Cache
            for M in (1, 16, 32, 64):
                x = torch.randn(M, K, device=dev).to(tdt)
                fn = lambda: [nq.awq_gemm(x, *w, 8) for w in copies]
                us = time_graph(fn, 10, 2) * 1e3 / len(copies)
                gbs = packed_bytes(K, N) / us / 1e3
                (large if M <= 16 else batched)[f"{K}x{N}_M{M}"] = {
                    "us": round(us, 2), "GBs": round(gbs, 1), "frac_of_8TBs": round(gbs / HBM_PEAK_GBS, 4),
                    "kernel": gemv_kernel_name(M, N, K, "f16")}
            del copies
            torch.cuda.empty_cache()
        out["batched_decode_gemv"] = {
            "kernel": "awq::gemv_wide_kernel + awq::gemv_wide_reduce_kernel (each case names its own form)",
            "unit": "GB/s of packed weights",
            "note": "17..64 rows (cfg5 decodes at 64): bound by the SIMDs' issue ports (MFMA + unpack + fold + load-to-LDS "
                    "instructions; at 33..64 rows the 244 registers a wave holds leave two waves per SIMD) plus the K "
                    "splits' fp32 partial round trip, not by HBM",
            "cases": batched}
        best = max(v["GBs"] for v in large.values())
        best_large = max(large, key=lambda k: large[k]["GBs"])
        out["roofline_large"] = {"kernel": large[best_large]["kernel"] + f" at {best_large} (each case names its own)",
                                 "bound": "hbm", "achieved": best,
                                 "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": best / HBM_PEAK_GBS,
                                 "workload": "Qwen3-32B MLP shapes (68.1 MB packed), HBM-streaming over 6 copies",
                                 "cases": large}

        # ---------------- extra: prefill GEMM, cfg3 -----------------------------------------------------
        # the fused dequant + MFMA kernel: what awq_linear / WQLinear_GEMM.forward run at these row counts
        bdt = torch.bfloat16
        fused = {}
        for (K, N) in ((4096, 12288), (12288, 4096)):
            w = rand_packed(K, N, bdt, dev)
            for M in (512, 2048, 8192):
                x = torch.randn(M, K, device=dev).to(bdt)
                fn = lambda: [nq.awq_gemm(x, *w, 8) for _ in range(4)]
                us = time_graph(fn, 5, 1) * 1e3 / 4
                tf = 2.0 * M * N * K / us / 1e6
                fused[f"M{M}_{K}x{N}"] = {"us": round(us, 1), "TFLOPs": round(tf, 1),
                                          "frac_of_2.5PF": round(tf / MFMA_PEAK_TFLOPS, 4),
                                          "kernel": gemm_kernel_name(M, N, K, "bf16")}
            del w
        bestf = max(v["TFLOPs"] for v in fused.values())
        best_case = max(fused, key=lambda k: fused[k]["TFLOPs"])
        out["roofline_prefill"] = {
            "kernel": fused[best_case]["kernel"] + f" at {best_case} (each case names its own)", "bound": "mfma",
            "achieved": bestf,
            "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": bestf / MFMA_PEAK_TFLOPS,
            "workload": "cfg3: Qwen3-8B MLP shapes, bf16, M in {512,2048,8192}; the fused dequant + MFMA kernel "
                        "(default dispatch at every M)",
            "cases": fused}
        # the same shapes in fp16 at the row counts whose work items fill the CUs: the default dispatch runs the
        # kernel with resident workgroups that builds its B operands in registers there (awq::gemm_regb_kernel)
        hdt = torch.float16
        fused16 = {}
        for (K, N) in ((4096, 12288), (12288, 4096)):
            w = rand_packed(K, N, hdt, dev)
            for M in (2048, 8192):
                x = torch.randn(M, K, device=dev).to(hdt)
                fn = lambda: [nq.awq_gemm(x, *w, 8) for _ in range(4)]
                us = time_graph(fn, 5, 1) * 1e3 / 4
                tf = 2.0 * M * N * K / us / 1e6
                fused16[f"M{M}_{K}x{N}"] = {"us": round(us, 1), "TFLOPs": round(tf, 1),
                                            "frac_of_2.5PF": round(tf / MFMA_PEAK_TFLOPS, 4),
                                            "kernel": gemm_kernel_name(M, N, K, "f16")}
            del w
        best16 = max(v["TFLOPs"] for v in fused16.values())
        best_case16 = max(fused16, key=lambda k: fused16[k]["TFLOPs"])
        out["roofline_prefill_f16"] = {
            "kernel": fused16[best_case16]["kernel"] + f" at {best_case16} (each case names its own)",
            "bound": "mfma", "achieved": best16, "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": best16 / MFMA_PEAK_TFLOPS,
            "workload": "cfg3's shapes with fp16 activations and scales, M in {2048, 8192}, default dispatch",
            "cases": fused16}

        # ---------------- extra: dequantise kernel ------------------------------------------------------
        K, N = 4096, 12288
        copies = [rand_packed(K, N, bdt, dev) for _ in range(4)]
        fn = lambda: [nq.awq_dequantize(*w) for w in copies]
        us = time_graph(fn, 10, 2) * 1e3 / len(copies)
        db = packed_bytes(K, N) + 2 * K * N
        out["dequant"] = {"shape": f"{K}x{N} bf16", "us": round(us, 1), "GBs": round(db / us / 1e3, 1),
                          "frac_of_8TBs": round(db / us / 1e3 / HBM_PEAK_GBS, 4), "bytes": db}
        del copies
        torch.cuda.empty_cache()

        # ---------------- extra: cfg1 latency -----------------------------------------------------------
        w = rand_packed(1024, 3072, tdt, dev)
        x = torch.randn(16, 1024, device=dev).to(tdt)
        fn = lambda: [nq.awq_gemm(x, *w, 8) for _ in range(50)]
        out["cfg1_single_linear"] = {"shape": "x[16,1024] @ W[1024,3072]", "graph_us": round(time_graph(fn, 5, 1) * 1e3 / 50, 2),
                                     "eager_us": round(time_eager(lambda: nq.awq_gemm(x, *w, 8), 200, 20) * 1e3, 2)}

    if not args.quick and not args.only_cfg5:
        # ---------------- extra: cfg4, end-to-end Qwen3-0.6B-architecture decode ------------------------
        try:
            from nanoquantization_amd.engine import LLMEngine
            from nanoquantization_amd.models.random_init import QWEN3_0P6B as Q06B_CFG, random_awq_qwen3
            model = random_awq_qwen3(Q06B_CFG, seed=0, device=dev, dtype=torch.bfloat16)
            B, P, NEW = 32, 512, 256
            eng = LLMEngine(model, max_batch=B, max_seq_len=P + NEW, block_size=64, use_graph=True)
            prompts = torch.randint(0, Q06B_CFG["vocab_size"], (B, P), generator=torch.Generator().manual_seed(1)).tolist()
            eng.generate(prompts, 8)                      # warm-up: graph capture, workspaces
            st = {}
            eng.generate(prompts, NEW, stats=st)
            out["e2e_qwen3_0p6b"] = {
                "workload": "cfg4: Qwen3-0.6B architecture, random AWQ g=128 weights, bf16, paged KV (block 64), "
                            "batch 32 x 512-token random prompts, 256 greedy tokens, decode step in a HIP graph",
                "decode_tok_per_s": round(B * st["decode_steps"] / st["decode_s"], 1),
                "decode_ms_per_step": round(st["decode_s"] / st["decode_steps"] * 1e3, 3),
                "prefill_s": round(st["prefill_s"], 4),
                "prefill_tok_per_s": round(B * P / st["prefill_s"], 1),
                "launches_per_block": 5 if eng.norm_fused_ok else 7,
                "roofline": step_roofline(decode_step_bytes(model, B * (P + NEW // 2)),
                                          st["decode_s"] / st["decode_steps"] * 1e3,
                                          "decode step: awq::gemv_dma_kernel forms + awq::paged_attn_decode"),
            }
            # the same engine under continuous batching: ragged requests, rows and cache blocks recycled
            rg = torch.Generator().manual_seed(2)
            lens = torch.randint(32, 513, (96,), generator=rg).tolist()
            news = torch.randint(16, 129, (96,), generator=rg).tolist()
            reqs = [(torch.randint(0, Q06B_CFG["vocab_size"], (n,), generator=rg).tolist(), m) for n, m in zip(lens, news)]
            sv, svb = {}, {}
            eng.serve(reqs[:8])                            # warm-up of the prefill shapes
            eng.serve(reqs[:40], batch_prefill=True)
            eng.serve(reqs, stats=sv)
            eng.serve(reqs, stats=svb, batch_prefill=True)
            out["serve_qwen3_0p6b"] = {
                "workload": "96 requests, prompts of 32..512 tokens, 16..128 new tokens each, 32 batch rows, greedy",
                "one_prefill_per_request": {
                    "generated_tok_per_s": round(sv["tokens"] / sv["wall_s"], 1), "wall_s": round(sv["wall_s"], 3),
                    "decode_steps": sv["decode_steps"], "prefill_calls": sv["prefill_calls"], "tokens": sv["tokens"]},
                "batched_ragged_prefill": {
                    "generated_tok_per_s": round(svb["tokens"] / svb["wall_s"], 1), "wall_s": round(svb["wall_s"], 3),
                    "decode_steps": svb["decode_steps"], "prefill_calls": svb["prefill_calls"], "tokens": svb["tokens"]},
            }
            del eng, model
            torch.cuda.empty_cache()
        except Exception as e:  # the headline must still be printed
            out["e2e_qwen3_0p6b"] = {"error": repr(e)}

    if not args.quick and not args.no_cfg5:
        # ---------------- extra: cfg5, Qwen3-32B architecture: batch-64 decode at 2048 context with a 4096-token
        # prefill admitted in between (one serve() call), then the steady decode step on its own
        try:
            from nanoquantization_amd.engine import LLMEngine
            from nanoquantization_amd.models.random_init import QWEN3_32B, random_awq_qwen3
            cfg = dict(QWEN3_32B, max_position_embeddings=8192)
            model = random_awq_qwen3(cfg, seed=0, device=dev, dtype=torch.bfloat16)
            B, P, NEW, LONG = 64, 2048, 24, 4096
            eng = LLMEngine(model, max_batch=B, max_seq_len=LONG + 64, block_size=64, use_graph=True)
            rg = torch.Generator().manual_seed(1)
            prompts = torch.randint(0, cfg["vocab_size"], (B, P), generator=rg).tolist()
            long_prompt = torch.randint(0, cfg["vocab_size"], (LONG,), generator=rg).tolist()
            eng.generate(prompts[:4], 3)                  # warm-up: graph capture, workspaces
            eng.serve([(long_prompt, 2)])                 # warm-up of the long prefill's shapes
            # mixed run: 64 requests at 2048 tokens fill the batch (prefilled four at a time); request 0 ends after
            # 4 tokens, which frees a row for the 4096-token request: it is prefilled while 63 rows wait at a
            # context of ~2052, then all 64 rows decode together
            reqs = [(p, 4 if i == 0 else NEW) for i, p in enumerate(prompts)] + [(long_prompt, 12)]
            sv = {}
            eng.serve(reqs, stats=sv, batch_prefill=True, max_prefill_tokens=4 * P)
            long_pf = [p for p in sv["prefill_log"] if p[0] == LONG]
            st = {}
            eng.generate(prompts, 17, stats=st)           # the steady decode step alone, batch 64 at 2048..2064
            ms_step = st["decode_s"] / st["decode_steps"] * 1e3
            out["cfg5_qwen3_32b"] = {
                "workload": "Qwen3-32B architecture (64 layers, hidden 5120, 64 q / 8 kv heads, intermediate 25600), random "
                            "AWQ g=128 weights, bf16, paged KV (block 64).  mixed: one serve() of 64 requests x 2048-token "
                            "prompts (24 new tokens; one of them 4) plus a 4096-token request admitted when the first row "
                            "frees, i.e. prefilled between decode steps of the other 63 rows.  steady: generate() of 64 x "
                            "2048 prompts, 16 timed decode steps",
                "mixed": {
                    "wall_s": round(sv["wall_s"], 3), "generated_tokens": sv["tokens"],
                    "generated_tok_per_s": round(sv["tokens"] / sv["wall_s"], 1),
                    "decode_steps": sv["decode_steps"], "decode_s": round(sv["decode_s"], 4),
                    "decode_ms_per_step": round(sv["decode_s"] / max(1, sv["decode_steps"]) * 1e3, 2),
                    "prefill_calls": sv["prefill_calls"], "prefill_s": round(sv["prefill_s"], 4),
                    "batch_prefill_tok_per_s": round(sum(p[0] for p in sv["prefill_log"] if p[0] != LONG)
                                                     / max(1e-9, sum(p[3] for p in sv["prefill_log"] if p[0] != LONG)), 1),
                    "prefill_4096_s": round(long_pf[0][3], 4) if long_pf else None,
                    "prefill_4096_tok_per_s": round(LONG / long_pf[0][3], 1) if long_pf else None,
                    "prefill_4096_after_decode_steps": long_pf[0][2] if long_pf else None,
                },
                "decode_tok_per_s": round(B * st["decode_steps"] / st["decode_s"], 1),
                "decode_ms_per_step": round(ms_step, 2),
                "roofline": step_roofline(decode_step_bytes(model, B * (P + 8)), ms_step,
                                          "decode step: awq::gemv_wide_kernel / gemv_dma_kernel forms + "
                                          "awq::paged_attn_decode_mfma_kernel"),
            }
            del eng, model
            torch.cuda.empty_cache()
        except Exception as e:
            out["cfg5_qwen3_32b"] = {"error": repr(e)}

    # ---------------- CPU baseline: the reference's path restated on host tensors (bounded sample) ----------
    if not args.no_cpu:
        from oracle import torch_cpu_path as cpu
        torch.set_num_threads(os.cpu_count() or 1)
        K, N, M = 1024, 3072, 16
        qw, sc, qz = [t.cpu() for t in rand_packed(K, N, tdt, dev)]
        xc = torch.randn(M, K).to(tdt)
        t_end = time.time() + 12.0
        times_native, times_up, times_dq = [], [], []
        for _ in range(3):
            cpu.linear(xc, qw, sc, qz, upcast=True)
        while time.time() < t_end and len(times_up) < 200:
            t0 = time.perf_counter(); wd = cpu.dequant(qw, sc, qz); t1 = time.perf_counter()
            torch.matmul(xc.float(), wd.float()).to(tdt); t2 = time.perf_counter()
            times_dq.append(t1 - t0); times_up.append(t2 - t0)
        t_end = time.time() + 6.0
        while time.time() < t_end and len(times_native) < 50:
            t0 = time.perf_counter(); cpu.linear(xc, qw, sc, qz, upcast=False); times_native.append(time.perf_counter() - t0)
        med = lambda v: sorted(v)[len(v) // 2]
        t_up = med(times_up)
        out["cpu_baseline"] = {
            "value": packed_bytes(K, N) / t_up / 1e9, "unit": "GB/s",
            "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"cfg1 single linear x[16,1024] @ W[1024,3072] fp16 g=128, torch unpack + (q-z)*s + matmul on CPU "
                      f"tensors, fp32-upcast matmul, median of {len(times_up)} iterations",
            "ms_total_fp32_upcast": t_up * 1e3, "ms_dequant": med(times_dq) * 1e3,
            "ms_total_native_fp16": med(times_native) * 1e3 if times_native else None,
            "TFLOPs": 2.0 * M * N * K / t_up / 1e12, "os_cpu_count": os.cpu_count(),
        }

    print(json.dumps(out))


if __name__ == "__main__":
    main()
