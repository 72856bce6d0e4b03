"""Builds csrc/*.hip into nanoquantization_amd/libawq_hip.so for gfx950, and csrc/torch_binding.cpp (host code
only: the PyTorch operator registration over the C ABI) into nanoquantization_amd/libawq_torch.so.

Usage: python -m nanoquantization_amd.build
"""
from __future__ import annotations

import glob
import os
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libawq_hip.so")

TORCH_LIB_PATH = os.path.join(PKG_DIR, "libawq_torch.so")

ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
HIPCC = os.environ.get("HIPCC", os.path.join(ROCM, "bin", "hipcc"))
CXX = os.environ.get("CXX", "g++")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # packed-fp32 arithmetic is switched off for every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


# per-source extra flags
EXTRA = {
    # keep MFMA results in VGPRs: the GEMV folds every accumulator into fp32 state right away,
    # AGPR destinations would cost a v_accvgpr_read per value and 4 more registers per wave
    "awq_gemv.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    # the SLP vectoriser pairs the two k rows of the unpack into <2 x i32> and/or, which then no
    # longer select as one v_and_or_b32 each
    "awq_gemm_pipe.hip": ["-fno-slp-vectorize"],
    "awq_gemm_regb.hip": ["-fno-slp-vectorize"],
}


def sources() -> list[str]:
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the device-only target feature and says so once per file
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{out}")
    if verbose and out.strip():
        print(out)


def build(verbose: bool = True) -> str:
    """Compile every HIP source (in parallel) and link one shared library; returns its path."""
    from concurrent.futures import ThreadPoolExecutor

    objdir = os.path.join(PKG_DIR, "build")
    os.makedirs(objdir, exist_ok=True)
    compile_flags = [f for f in FLAGS if f != "-shared"]
    jobs = []
    for src in sources():
        obj = os.path.join(objdir, os.path.basename(src) + ".o")
        jobs.append(([HIPCC, *compile_flags, *EXTRA.get(os.path.basename(src), []), "-c", src, "-o", obj], obj))
    with ThreadPoolExecutor(max_workers=min(4, len(jobs))) as pool:
        list(pool.map(lambda j: _run(j[0], verbose), jobs))
    with ThreadPoolExecutor(max_workers=2) as pool:
        # the operator binding has no device code: host compiler, torch headers; it only needs the C header
        binding = pool.submit(_run, torch_binding_compile_cmd(os.path.join(objdir, "torch_binding.o")), verbose)
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *[o for _, o in jobs], "-o", LIB_PATH], verbose)
        binding.result()
    _run(torch_binding_link_cmd(os.path.join(objdir, "torch_binding.o")), verbose)
    return LIB_PATH


def _torch_dirs():
    import torch
    root = os.path.dirname(torch.__file__)
    return ([os.path.join(root, "include"), os.path.join(root, "include", "torch", "csrc", "api", "include")],
            os.path.join(root, "lib"), int(torch._C._GLIBCXX_USE_CXX11_ABI))


def torch_binding_compile_cmd(obj: str) -> list[str]:
    incs, _, abi = _torch_dirs()
    return [CXX, "-O2", "-fPIC", "-std=c++17", "-w", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
            f"-D_GLIBCXX_USE_CXX11_ABI={abi}", *[f"-I{i}" for i in incs], f"-I{ROCM}/include",
            "-c", os.path.join(CSRC, "torch_binding.cpp"), "-o", obj]


def torch_binding_link_cmd(obj: str) -> list[str]:
    _, libdir, _ = _torch_dirs()
    return [CXX, "-shared", "-fPIC", obj, "-o", TORCH_LIB_PATH, f"-L{libdir}", "-ltorch", "-ltorch_cpu", "-lc10",
            "-lc10_hip", "-ltorch_hip", f"-L{PKG_DIR}", "-lawq_hip", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{libdir}"]


if __name__ == "__main__":
    build()
    sys.exit(0)
