"""Launch one AWQ linear of a given shape a few times, for a profiler or counter collection to look at:

    python3 -m nanoquantization_amd.profile_one linear K N M [--dtype bf16|f16] [--iters 6] [--group-size 128]
    python3 -m nanoquantization_amd.profile_one dequant K N 0 ...
    python3 -m nanoquantization_amd.profile_one copy K N 0 ...       # device copy of the packed weight (counter calibration)

Random packed weights and activations (seeded); every iteration uses the same buffers."""
from __future__ import annotations

import argparse

import torch


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("kind", choices=["linear", "dequant", "copy"])
    ap.add_argument("K", type=int)
    ap.add_argument("N", type=int)
    ap.add_argument("M", type=int)
    ap.add_argument("--dtype", choices=["bf16", "f16"], default="bf16")
    ap.add_argument("--iters", type=int, default=6)
    ap.add_argument("--group-size", type=int, default=128)
    a = ap.parse_args()
    import nanoquantization_amd as nq
    dev, g = torch.device("cuda:0"), a.group_size
    tdt = torch.bfloat16 if a.dtype == "bf16" else torch.float16
    gen = torch.Generator(device=dev).manual_seed(a.K + a.N)
    qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (a.K, a.N // 8), dtype=torch.int32, device=dev, generator=gen)
    qz = torch.randint(-2 ** 31, 2 ** 31 - 1, (a.K // g, a.N // 8), dtype=torch.int32, device=dev, generator=gen)
    qs = (torch.rand(a.K // g, a.N, device=dev, generator=gen) * 0.02 + 0.001).to(tdt)
    x = torch.randn(max(a.M, 1), a.K, device=dev, generator=gen).to(tdt)
    fn = {"linear": lambda: nq.awq_gemm(x, qw, qs, qz, 8),
          "dequant": lambda: nq.awq_dequantize(qw, qs, qz), "copy": lambda: qw.clone()}[a.kind]
    for _ in range(a.iters):
        fn()
    torch.cuda.synchronize()
    print(f"{a.kind} K={a.K} N={a.N} M={a.M} {a.dtype}: {a.iters} launches")


if __name__ == "__main__":
    main()
