"""Ahead-of-time build of the gfx950 kernel library (``libsvdq_mi355x.so``) with hipcc.

Run as ``python -m nunchaku_rocm_amd.build``.  The library is built in-tree next to this file so that it travels
with the source tree; nothing is compiled at import time or at run time.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libsvdq_mi355x.so")
SOURCES = ["common.hip", "quantize.hip", "gemm_w4a4.hip", "awq_gemv.hip", "attention.hip", "layout.hip"]
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # packed fp32 VALU ops stay off: plain v_fma_f32 / v_mul_f32 only
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]  # fmt: skip


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or add /opt/rocm/bin to PATH)")


def build(verbose: bool = False) -> str:
    cmd = [hipcc(), *FLAGS, *[os.path.join(CSRC, s) for s in SOURCES], "-o", LIB + ".tmp"]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(ln for ln in proc.stderr.splitlines() if "not a recognized feature" not in ln)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    os.replace(LIB + ".tmp", LIB)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
