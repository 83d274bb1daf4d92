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
    """Every source to an object file of its own, side by side (the sources do not depend on each
    other's objects; one compiler run over all of them takes twice as long), then one link."""
    import tempfile
    from concurrent.futures import ThreadPoolExecutor

    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    flags = [f for f in HIPCC_FLAGS if f != "-shared"]
    jobs = max(1, min(len(SOURCES), int(os.environ.get("MAX_JOBS", "8"))))
    with tempfile.TemporaryDirectory() as tmp:
        def compile_one(src: str) -> str:
            obj = os.path.join(tmp, src.replace(".hip", ".o"))
            cmd = [hipcc, *flags, "-I", os.path.join(ROOT, "include"), "-I", CSRC, "-c", os.path.join(CSRC, src), "-o", obj]
            if verbose:
                print(" ".join(cmd), flush=True)
            subprocess.run(cmd, check=True)
            return obj

        with ThreadPoolExecutor(max_workers=jobs) as pool:
            objects = list(pool.map(compile_one, SOURCES))
        link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *objects, "-o", LIB_PATH + ".tmp"]
        if verbose:
            print(" ".join(link), flush=True)
        subprocess.run(link, check=True)
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
