"""Builds libmj_grpo.so (the C-ABI library of HIP kernels) and libmj_grpo_bench.so (bench.py's
measurement support: event timing behind the launch-trace hook, the MFMA-only probe) for gfx950
with hipcc.

`python -m mllm_jax_amd.build` compiles in-tree; tests, the smoke entry and the bench
load the built libraries and never compile on a GPU box.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "csrc", "mj_grpo.hip")
LIB = os.path.join(HERE, "libmj_grpo.so")
BENCH_SRC = os.path.join(HERE, "csrc", "mj_bench.hip")
BENCH_LIB = os.path.join(HERE, "libmj_grpo_bench.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # keep hipcc from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH, /opt/rocm/bin/hipcc)")


def build(verbose: bool = True) -> str:
    _compile(BENCH_SRC, BENCH_LIB, verbose)
    return _compile(SRC, LIB, verbose)


def _compile(src: str, lib: str, verbose: bool) -> str:
    cmd = [hipcc_path(), *HIPCC_FLAGS, src, "-o", lib + ".tmp"]
    if verbose:
        print("+", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    import ctypes
    ctypes.CDLL(lib + ".tmp")          # an unresolved symbol must fail the build, not the first call
    os.replace(lib + ".tmp", lib)
    return lib


if __name__ == "__main__":
    print(build())
