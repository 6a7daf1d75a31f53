"""Builds ``libpmetal_hip.so`` for gfx950 with hipcc, in-tree (next to this file).

The library is a plain C-ABI shared object (see ``include/pmetal_hip.h``); nothing here depends
on PyTorch.  ``codec.hip`` holds the bit-exact quantize/dequantize kernels and is compiled without
floating-point contraction; the matmul kernels may fuse.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libpmetal_hip.so")
ARCH = "gfx950"

COMMON = [
    "--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC", "-fno-fast-math",
    # packed-fp32 VALU ops are unreliable on this hardware pool: never let the compiler emit them
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes", "-Wno-unused-command-line-argument",
]
# per-file extra flags
EXTRA = {
    "codec.hip": ["-ffp-contract=off", "-fhip-fp32-correctly-rounded-divide-sqrt", "-fno-gpu-flush-denormals-to-zero"],
    # the first 16 dwords of kernel arguments arrive in scalar registers with the wave (no argument fetch
    # in front of the first load of these latency-bound kernels)
    "gemv.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=16"],
    "gemv_q4k.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=16"],
    "gemv_q23k.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=16"],
    "gemv_q5k.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=16"],
    "gemv_q6k.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=16"],
    "gemv_q8_0.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=16"],
    "gemm.hip": [],
    "q8k.hip": ["-ffp-contract=off", "-fno-gpu-flush-denormals-to-zero"],
    "util.hip": [],
    "api.hip": [],
}


def _compile(name: str, verbose: bool) -> str:
    src = os.path.join(CSRC, name)
    obj = os.path.join(CSRC, name.replace(".hip", ".o"))
    cmd = ["hipcc", *COMMON, *EXTRA[name], "-c", src, "-o", obj]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        sys.stderr.write(r.stdout + r.stderr)
        raise RuntimeError(f"hipcc failed on {name}")
    return obj


def build(verbose: bool = False, jobs: int = 4) -> str:
    """Compile every translation unit and link the shared library. Always recompiles."""
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda n: _compile(n, verbose), EXTRA))
    cmd = ["hipcc", "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        sys.stderr.write(r.stdout + r.stderr)
        raise RuntimeError("link failed")
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
