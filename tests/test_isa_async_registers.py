"""Static checks of the streaming qmm kernels' machine code (dflash_mlx_amd/isa_check.py): the
scanner on hand-made snippets, then every kernel as hipcc compiles it for gfx950."""
import shutil

import pytest

from dflash_mlx_amd import isa_check
from dflash_mlx_amd.isa_check import scan

needs_hipcc = pytest.mark.skipif(shutil.which("hipcc") is None, reason="hipcc not available")
_isa = {}


def _text(source):
    if source not in _isa:
        _isa[source] = isa_check.compile_to_isa(source)
    return _isa[source]


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


def test_checks_flag_what_they_are_for():
    spilled = "_ZN1kEv:\n" + "ds_read_b32 v4, v1\n" * 3 + "s_waitcnt lgkmcnt(0)\nscratch_store_dword off, v4, s0\n.Lfunc_end0:\n"
    with pytest.raises(AssertionError, match="scratch"):
        isa_check.check_kernels(spilled, "_ZN1k", 1, 3)
    with pytest.raises(AssertionError, match="instantiations"):
        isa_check.check_kernels(spilled, "_ZN1k", 2, 3)
    hasty = ".Lfunc_begin0:\nglobal_store_dword v1, v2, off\ns_barrier\nglobal_atomic_inc v3, v4, s[0:1]\n"
    with pytest.raises(AssertionError, match="without a wait"):
        isa_check.check_arrivals(hasty, "x.hip", 1)
    patient = hasty.replace("s_barrier", "s_waitcnt vmcnt(0)\ns_barrier")
    isa_check.check_arrivals(patient, "x.hip", 1)
    with pytest.raises(AssertionError, match="expected 2"):
        isa_check.check_arrivals(patient, "x.hip", 2)
    bare = ";;#ASMSTART\nglobal_store_dwordx4 v[2:3], v[4:7], off sc1\n;;#ASMEND\nv_mov_b32 v6, v9\n"
    with pytest.raises(AssertionError, match="wait states"):
        isa_check.check_wide_stores(bare, "x.hip")
    padded = bare.replace("off sc1\n", "off sc1\ns_nop 1\n")
    assert isa_check.check_wide_stores(padded, "x.hip") == 1
    assert isa_check.check_wide_stores("global_store_dwordx4 v[2:3], v[4:7], off\nv_mov_b32 v6, v9\n", "x.hip") == 0


@needs_hipcc
@pytest.mark.parametrize("source,prefix,count,min_reads", isa_check.KERNELS)
def test_no_instruction_touches_registers_of_reads_in_flight(source, prefix, count, min_reads):
    isa_check.check_kernels(_text(source), prefix, count, min_reads)


@needs_hipcc
@pytest.mark.parametrize("source,arrivals", isa_check.ARRIVALS)
def test_partial_tiles_are_acknowledged_before_the_arrival_counter(source, arrivals):
    """Split K: a workgroup stores its partial tile and then bumps the row block's arrival
    counter; the last to arrive adds the tiles.  Nothing but a wait for the stores'
    acknowledgement keeps the counter from overtaking them (a workgroup barrier does not wait
    for global stores on this target)."""
    isa_check.check_arrivals(_text(source), source, arrivals)


@needs_hipcc
@pytest.mark.parametrize("source", ["qmm_m16_stream.hip", "qmm_m16_chain.hip"])
def test_hand_written_wide_stores_carry_their_wait_states(source):
    """A 128-bit global store reads the upper half of its data a cycle after issue; inside a
    hand-written block the compiler does not add the wait states that protect those registers."""
    assert isa_check.check_wide_stores(_text(source), source) > 0
