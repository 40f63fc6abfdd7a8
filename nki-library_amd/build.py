"""Build libmoe_gfx950.so (hand-written HIP kernels + C ABI) for gfx950 with hipcc.

Usage: ``python nki-library_amd/build.py``.  The library is written in-tree to
``nki-library_amd/nkilib/_lib/libmoe_gfx950.so`` where ``nkilib._native`` loads it.
hipcc cross-compiles, so no GPU is needed to build.  Translation units are compiled in
parallel into ``nki-library_amd/build/`` and linked; the MXFP8 large-tile GEMM
(``csrc/bwmm_mx.hip``) is compiled once per (stage, weight format) plus once as the dispatcher.
"""

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
OUT_DIR = os.path.join(HERE, "nkilib", "_lib")
OUT = os.path.join(OUT_DIR, "libmoe_gfx950.so")
SOURCES = ["rmsnorm_quant.hip", "build_blocks.hip", "combine.hip", "bwmm.hip", "bwmm_mx.hip", "router_topk.hip", "index_ops.hip", "capi.hip"]
# (stage, weight format) instances of the large-tile MX GEMM; formats as MX_WFMT_* in csrc/bwmm.hpp
MX_INSTANCES = [(1, 0), (2, 0), (1, 1), (2, 1), (1, 2), (2, 2), (1, 3), (2, 3), (1, 4), (2, 4)]
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # packed fp32 ALU ops are kept off for every HIP translation unit
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
# The two sources whose loads into LDS list M0 as clobbered (ld_lds_b128 in csrc/bwmm_mx.hip, the same in
# csrc/router_topk.hip) draw one inline-asm diagnostic per such load, thousands of times; every other translation
# unit keeps the diagnostic on
MX_FLAGS = ["-Wno-inline-asm"]
M0_CLOBBER_SOURCES = ("bwmm_mx.hip", "router_topk.hip")
NOISE = "is not a recognized feature for this target"


def _run(cmd):
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if NOISE not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}): {' '.join(cmd)}\n{err}")
    return err


def build(verbose=True, jobs=None):
    os.makedirs(OUT_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    inc = ["-I", os.path.join(ROOT, "include"), "-I", CSRC]
    units = []  # (object path, extra defines, source); the long-running instances of the large-tile GEMM go first
    for stage, fmt in MX_INSTANCES:
        units.append((os.path.join(OBJ_DIR, f"bwmm_mx_s{stage}_f{fmt}.o"),
                      [*MX_FLAGS, f"-DMX_INST_STAGE={stage}", f"-DMX_INST_WFMT={fmt}"], os.path.join(CSRC, "bwmm_mx.hip")))
    for s in SOURCES:
        units.append((os.path.join(OBJ_DIR, s.replace(".hip", ".o")), MX_FLAGS if s in M0_CLOBBER_SOURCES else [],
                      os.path.join(CSRC, s)))
    cmds = [["hipcc", *FLAGS, *defs, *inc, "-c", src, "-o", obj] for obj, defs, src in units]
    if verbose:
        for c in cmds:
            print(" ".join(c), flush=True)
    jobs = jobs or min(len(cmds), os.cpu_count() or 4, 16)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        errs = list(ex.map(_run, cmds))
    link = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", *[u[0] for u in units], "-o", OUT]
    if verbose:
        print(" ".join(link), flush=True)
    errs.append(_run(link))
    if verbose:
        for e in errs:
            if e.strip():
                print(e)
    return OUT


if __name__ == "__main__":
    build()
    print("built", OUT)
    sys.exit(0)
