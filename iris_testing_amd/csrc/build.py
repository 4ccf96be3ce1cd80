"""Builds libmoe_gfx950.so in-tree with hipcc (gfx950 only; cross-compiles without a GPU).

    python -m iris_testing_amd.csrc.build
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libmoe_gfx950.so")
SOURCES = ["capi.hip", "route.hip", "dispatch.hip", "grouped_gemm.hip", "diag.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
    # a*b+c stays two roundings unless fmaf() is written out (the combine is specified as multiply-then-add)
    "-ffp-contract=off",
    # keep the compiler from forming packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _compile(src: str, verbose: bool) -> str:
    obj = os.path.join(HERE, src.replace(".hip", ".o"))
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(HERE, src), "-o", obj]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip() and verbose:
        print(err, file=sys.stderr)
    return obj


def build(verbose: bool = True) -> str:
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(HERE, s))]
    with ThreadPoolExecutor(max_workers=5) as ex:
        objs = list(ex.map(lambda s: _compile(s, verbose), srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    print(build())
