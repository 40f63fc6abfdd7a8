"""Build libmoe_gfx950.so (hand-written HIP kernels + C ABI) for gfx950 with hipcc.

Usage: ``python nki-library_amd/build.py``.  The library is written in-tree to
``nki-library_amd/nkilib/_lib/libmoe_gfx950.so`` where ``nkilib._native`` loads it.
hipcc cross-compiles, so no GPU is needed to build.
"""

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OUT_DIR = os.path.join(HERE, "nkilib", "_lib")
OUT = os.path.join(OUT_DIR, "libmoe_gfx950.so")
SOURCES = ["rmsnorm_quant.hip", "build_blocks.hip", "combine.hip", "bwmm.hip", "bwmm_mx.hip", "router_topk.hip", "capi.hip"]
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # packed fp32 ALU ops are kept off for every HIP translation unit
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def build(verbose=True):
    os.makedirs(OUT_DIR, exist_ok=True)
    srcs = [os.path.join(CSRC, s) for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    cmd = ["hipcc", *FLAGS, "-I", os.path.join(ROOT, "include"), "-I", CSRC, *srcs, "-o", OUT]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{err}")
    if verbose and err.strip():
        print(err)
    return OUT


if __name__ == "__main__":
    build()
    print("built", OUT)
    sys.exit(0)
