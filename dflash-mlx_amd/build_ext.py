"""Compile the HIP sources under csrc/ into libdflash_mi355.so (gfx950 only).

Usage: ``python build_ext.py`` (or ``build()`` from Python).  hipcc cross-compiles,
so no GPU is needed to build.
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libdflash_mi355.so")

SOURCES = ["api.hip", "qmm_m16.hip", "qmm_m16_stream.hip", "qmm_m16_chain.hip", "tape_replay.hip", "gdn_forward.hip", "gdn_glue.hip", "sdpa_q16.hip",
           "conv_state.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-fno-gpu-rdc",
    # scalar fp32 code only: keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-command-line-argument",
]


def build(verbose: bool = False) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *HIPCC_FLAGS, "-I", os.path.join(ROOT, "include"), "-I", CSRC,
           *[os.path.join(CSRC, s) for s in SOURCES], "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
