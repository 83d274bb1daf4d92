"""Static checks of the machine code of the kernels that read LDS by hand (build-time; needs hipcc, no GPU).

The kernels start LDS reads whose destination registers are written after the issuing
instruction block has ended, and wait for them in a later block; the compiler does not know
that.  ``scan`` reads gfx950 assembly: between an LDS read and the wait that covers it, no
instruction may name a register the read is still writing (a register copy or spill placed
there by the compiler would read garbage).  ``check_kernels`` compiles a source, scans every
instantiation of its kernel and also refuses spills to scratch memory (a loader wave's own
memory operations would break its count of loads in flight).  ``check_arrivals``: between the
last store before a bump of an arrival counter and the bump itself the code must wait for all
of the wave's memory operations - nothing else keeps the counter from overtaking the stores.
``check_wide_stores``: a global store of more than 64 bits reads the upper half of its data a
cycle after it has been issued; where the compiler places such a store it also places the wait
states, but it cannot see one inside a hand-written block, so every such store in a block must
be followed by wait states of its own (seen on the device as partial tiles whose upper two
words were those of whatever the next instruction wrote).
"""
from __future__ import annotations

import os
import re
import subprocess
import tempfile
from typing import List, Tuple

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")

# source, mangled-name prefix of its kernel, instantiations, LDS reads each must at least hold
KERNELS = (
    ("qmm_m16_stream.hip", "_ZN6dflash6stream17qmm_stream_kernel", 16, 40),  # activation x scale dtype x chunk x dense|gathered
    ("qmm_m16_chain.hip", "_ZN6dflash6stream16qmm_chain_kernel", 8, 40),     # activation x scale dtype x weight layout
)
# source, number of counter bumps (arrival counters; the chained kernel's per-problem and exit counters too)
ARRIVALS = (("qmm_m16.hip", 24), ("qmm_m16_stream.hip", 0), ("qmm_m16_chain.hip", 64))


def _regs(text: str) -> set:
    out = set()
    for m in re.finditer(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b", text):
        if m.group(1):
            out.update(range(int(m.group(1)), int(m.group(2)) + 1))
        else:
            out.add(int(m.group(3)))
    return out


def scan(asm_text: str) -> Tuple[int, List[Tuple[int, str]]]:
    """Returns (number of LDS reads seen, list of offending lines).

    LDS operations complete in issue order, so after `s_waitcnt lgkmcnt(n)` only the n most
    recent ones can still be outstanding; scalar memory operations share the counter and are
    counted as if they were LDS operations, which errs on the side of flagging."""
    pending, bad, reads = [], [], 0   # pending: destination registers per outstanding operation
    for no, line in enumerate(asm_text.split("\n"), 1):
        t = line.split(";")[0].strip()
        if not t or t.startswith(".") or t.endswith(":"):
            continue
        busy = set().union(*pending) if pending else set()
        op = t.split(None, 1)[0]
        if op.startswith("ds_"):
            ops = t.split(None, 1)[1].split(",") if " " in t else []
            returns = op.startswith("ds_read") or op.startswith("ds_bpermute") or "_rtn" in op
            srcs = ops[1:] if returns else ops
            if _regs(",".join(srcs)) & busy:
                bad.append((no, t))
            pending.append(_regs(ops[0]) if returns else set())
            reads += 1 if op.startswith("ds_read") else 0
            continue
        if op.startswith(("s_load", "s_buffer_load", "s_memtime", "s_memrealtime")):
            pending.append(set())
            continue
        if op == "s_waitcnt":
            m = re.search(r"lgkmcnt\((\d+)\)", t)
            if m:
                n = int(m.group(1))
                pending = pending[-n:] if n > 0 else []
            continue
        if op == "s_endpgm":
            pending = []
            continue
        if _regs(t) & busy:
            bad.append((no, t))
    return reads, bad


def compile_to_isa(source: str) -> str:
    """gfx950 assembly of csrc/<source>, with the flags the library is built with."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "k.s")
        cmd = [hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature",
               "-Xclang", "-packed-fp32-ops", "-I", os.path.join(ROOT, "include"), "-I", CSRC,
               "--cuda-device-only", "-S", "-o", out, os.path.join(CSRC, source)]
        subprocess.run(cmd, check=True, capture_output=True, timeout=900)
        return open(out).read()


def check_kernels(text: str, prefix: str, count: int, min_reads: int) -> None:
    kernels = re.findall(rf"^({prefix}\w+):", text, flags=re.M)
    if len(kernels) != count:
        raise AssertionError(f"{prefix}: {len(kernels)} instantiations, expected {count}")
    for name in kernels:
        body = text[text.index(name + ":"):]
        body = body[:body.index(".Lfunc_end")]
        reads, bad = scan(body)
        if reads < min_reads:
            raise AssertionError(f"{name}: only {reads} LDS reads found")
        if bad:
            raise AssertionError(f"{name}: registers of LDS reads in flight are touched: {bad[:5]}")
        if "scratch_" in body:
            raise AssertionError(f"{name}: spills to scratch memory")


def check_arrivals(text: str, source: str, arrivals: int) -> None:
    lines = text.split("\n")
    found = 0
    for i, line in enumerate(lines):
        if "global_atomic_inc" not in line and "global_atomic_add" not in line:
            continue
        found += 1
        j, waited = i - 1, False
        while j >= 0 and "global_store" not in lines[j] and ".Lfunc_begin" not in lines[j]:
            waited = waited or bool(re.search(r"s_waitcnt\b.*vmcnt\(0\)", lines[j]))
            j -= 1
        if not (j >= 0 and "global_store" in lines[j]):
            raise AssertionError(f"{source}: no store before the counter bump at line {i + 1}")
        if not waited:
            raise AssertionError(f"{source}: counter bump at line {i + 1} follows the store at line {j + 1} without a wait")
    if found != arrivals:
        raise AssertionError(f"{source}: {found} counter bumps, expected {arrivals}")


def check_wide_stores(text: str, source: str) -> int:
    """Every 96/128-bit global store inside a hand-written block is followed by s_nop; returns how many."""
    lines = text.split("\n")
    in_block, found = False, 0
    for i, line in enumerate(lines):
        t = line.strip()
        if t.startswith(";;#ASMSTART"):
            in_block = True
        elif t.startswith(";;#ASMEND"):
            in_block = False
        elif in_block and re.match(r"(global|flat|buffer)_store_dwordx[34]\b", t):
            found += 1
            nxt = next((l.strip() for l in lines[i + 1:] if l.strip()), "")
            if not nxt.startswith("s_nop"):
                raise AssertionError(f"{source}: wide store at line {i + 1} of the assembly is not followed by wait states")
    return found


def check_all() -> None:
    """Every check on every source; raises AssertionError on the first finding."""
    from concurrent.futures import ThreadPoolExecutor

    sources = sorted({s for s, *_ in KERNELS} | {s for s, _ in ARRIVALS})
    with ThreadPoolExecutor(max_workers=3) as pool:
        isa = dict(zip(sources, pool.map(compile_to_isa, sources)))
    for source, prefix, count, min_reads in KERNELS:
        check_kernels(isa[source], prefix, count, min_reads)
    for source, arrivals in ARRIVALS:
        check_arrivals(isa[source], source, arrivals)
    for source in ("qmm_m16_stream.hip", "qmm_m16_chain.hip"):
        if check_wide_stores(isa[source], source) == 0:
            raise AssertionError(f"{source}: no partial-tile store found")
