"""Static check of the streaming qmm kernel's machine code.

The kernel starts LDS reads whose destination registers are written after the issuing
instruction block has ended, and waits for them in a later block; the compiler does not
know that.  This test compiles the kernel to gfx950 assembly and scans it: between an LDS
read and the next wait for lgkmcnt(0), no instruction may name a register the read is still
writing (a register copy or spill placed there by the compiler would read garbage).
"""
import os
import re
import shutil
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "dflash-mlx_amd", "csrc", "qmm_m16_stream.hip")


def _regs(text):
    out = set()
    for m in re.finditer(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b", text):
        if m.group(1):
            out.update(range(int(m.group(1)), int(m.group(2)) + 1))
        else:
            out.add(int(m.group(3)))
    return out


def scan(asm_text):
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


def test_scanner_flags_a_premature_use():
    ok = "ds_read_b128 v[4:7], v1\nv_add_f32 v9, v8, v8\ns_waitcnt lgkmcnt(0)\nv_add_f32 v9, v4, v8\n"
    assert scan(ok) == (1, [])
    early = "ds_read_b128 v[4:7], v1\nv_mov_b32 v9, v5\ns_waitcnt lgkmcnt(0)\n"
    reads, bad = scan(early)
    assert reads == 1 and len(bad) == 1 and "v_mov_b32" in bad[0][1]
    partial = "ds_read_b64 v[4:5], v1\ns_waitcnt lgkmcnt(1)\nv_mov_b32 v9, v4\n"
    assert len(scan(partial)[1]) == 1
    in_order = "ds_read_b32 v4, v1\nds_read_b32 v5, v1\ns_waitcnt lgkmcnt(1)\nv_mov_b32 v9, v4\n"
    assert scan(in_order) == (2, [])
    too_early = "ds_read_b32 v4, v1\nds_read_b32 v5, v1\ns_waitcnt lgkmcnt(1)\nv_mov_b32 v9, v5\n"
    assert len(scan(too_early)[1]) == 1


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="hipcc not available")
def test_no_instruction_touches_registers_of_reads_in_flight():
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "stream.s")
        cmd = ["hipcc", "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature",
               "-Xclang", "-packed-fp32-ops", "-I", os.path.join(ROOT, "include"),
               "-I", os.path.dirname(SRC), "--cuda-device-only", "-S", "-o", out, SRC]
        subprocess.run(cmd, check=True, capture_output=True, timeout=600)
        text = open(out).read()
    kernels = re.findall(r"^(_ZN6dflash6stream17qmm_stream_kernel\w+):", text, flags=re.M)
    assert len(kernels) == 16, kernels  # activation x scale dtype x chunk size x dense|gathered
    for name in kernels:
        body = text[text.index(name + ":"):]
        body = body[:body.index(".Lfunc_end")]
        reads, bad = scan(body)
        assert reads >= 40, (name, reads)   # the operand reads are there at all
        assert not bad, (name, bad[:5])
        assert "scratch_" not in body, name  # nothing spilled


def _compile_to_isa(src, out):
    cmd = ["hipcc", "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature",
           "-Xclang", "-packed-fp32-ops", "-I", os.path.join(ROOT, "include"),
           "-I", os.path.dirname(src), "--cuda-device-only", "-S", "-o", out, src]
    subprocess.run(cmd, check=True, capture_output=True, timeout=600)
    return open(out).read().split("\n")


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="hipcc not available")
@pytest.mark.parametrize("source,arrivals", [("qmm_m16.hip", 24), ("qmm_m16_stream.hip", 32)])
def test_partial_tiles_are_acknowledged_before_the_arrival_counter(source, arrivals):
    """Split K: a workgroup stores its partial tile and then bumps the row block's arrival
    counter; the last to arrive adds the tiles.  Nothing but a wait for the stores'
    acknowledgement keeps the counter from overtaking them (a workgroup barrier does not wait
    for global stores on this target), so between the last store before an arrival and the
    arrival itself the code must wait for all of the wave's memory operations."""
    with tempfile.TemporaryDirectory() as tmp:
        lines = _compile_to_isa(os.path.join(os.path.dirname(SRC), source), os.path.join(tmp, "k.s"))
    found = 0
    for i, line in enumerate(lines):
        if "global_atomic_inc" not in line:
            continue
        found += 1
        j, waited = i - 1, False
        while j >= 0 and "global_store" not in lines[j] and ".Lfunc_begin" not in lines[j]:
            waited = waited or bool(re.search(r"s_waitcnt\b.*vmcnt\(0\)", lines[j]))
            j -= 1
        assert j >= 0 and "global_store" in lines[j], (source, i)
        assert waited, f"{source}: arrival at line {i + 1} follows the store at line {j + 1} without a wait"
    assert found == arrivals, (source, found)
