"""The C-ABI library loads without a GPU, exports every symbol the header declares,
and rejects bad arguments before touching the device."""
import ctypes
import os
import re

import pytest

import dflash_mlx_amd._native as nat

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "dflash_mi355.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dflash_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported(native_lib):
    declared = _declared_symbols()
    assert declared, "no declarations parsed from the header"
    raw = ctypes.CDLL(nat.LIB_PATH)
    for name in declared:
        assert hasattr(raw, name), f"{name} declared in the header but not exported"
    assert sorted(nat.EXPORTED_SYMBOLS) == declared


def test_abi_version_matches_header(native_lib):
    m = re.search(r"#define\s+DFLASH_ABI_VERSION\s+(\d+)", open(HEADER).read())
    assert native_lib.dflash_abi_version() == int(m.group(1)) == nat.ABI_VERSION


def test_argument_errors_do_not_reach_the_device(native_lib):
    L = native_lib
    one = ctypes.c_void_p(256)  # never dereferenced: validation fails first
    # null operand
    assert L.dflash_qmm_m16(None, None, None, None, None, None, 0, 64, 32, 64, 0, 0, 0, 1, 0, None) == -1
    assert b"null operand" in L.dflash_last_error()
    # unsupported group size
    assert L.dflash_qmm_m16(one, one, one, one, one, None, 0, 64, 32, 48, 0, 0, 0, 1, 0, None) == -2
    assert b"group_size" in L.dflash_last_error()
    # N not a multiple of 16
    assert L.dflash_qmm_m16(one, one, one, one, one, None, 0, 64, 24, 64, 0, 0, 0, 1, 0, None) == -2
    # pipe variant without workspace
    assert L.dflash_qmm_m16(one, one, one, one, one, None, 0, 512, 32, 64, 0, 0, 1, 8, 0, None) == -3
    assert b"workspace" in L.dflash_last_error()
    # streaming kernel forced on a shape it does not cover
    assert L.dflash_qmm_m16(one, one, one, one, one, one, 1 << 20, 320, 32, 64, 0, 0, 0, 1, 2, None) == -2
    assert b"streaming kernel" in L.dflash_last_error()
    # unknown kernel selector
    assert L.dflash_qmm_m16(one, one, one, one, one, one, 1 << 20, 320, 32, 64, 0, 0, 0, 1, 9, None) == -1
    # K not a multiple of 32*k_parts
    assert L.dflash_qmm_m16(one, one, one, one, one, one, 1 << 20, 320, 32, 64, 0, 0, 1, 8, 0, None) == -2
    # replay: aliasing, head mismatch, Dk not multiple of 4
    assert L.dflash_tape_replay(one, one, one, one, one, None, 1, None, 1, 4, 2, 4, 128, 128,
                                2, 0, 0, 2, 0, 0, None) == -1
    two = ctypes.c_void_p(512)
    assert L.dflash_tape_replay(one, one, one, one, two, None, 1, None, 1, 4, 3, 4, 128, 128,
                                2, 0, 0, 2, 0, 0, None) == -2
    assert b"align K heads" in L.dflash_last_error()
    assert L.dflash_tape_replay(one, one, one, one, two, None, 1, None, 1, 4, 2, 4, 30, 128,
                                2, 0, 0, 2, 0, 0, None) == -2
    # conv rebuild: aliasing
    assert L.dflash_conv_state_rebuild(one, one, one, None, 1, 1, 16, 3, 64, 2, None) == -1


def test_workspace_size_formula(native_lib):
    L = native_lib
    assert L.dflash_qmm_m16_workspace_bytes(4096, 4096, 64, nat.QMM_MMA2BIG, 1, nat.QMM_KERNEL_TILE) == 0
    need = L.dflash_qmm_m16_workspace_bytes(4096, 4096, 64, nat.QMM_MMA2BIG_PIPE, 8, nat.QMM_KERNEL_TILE)
    assert need >= 8 * 16 * 4096 * 4
    # shapes only the tile kernel covers need no more than the tile kernel's workspace
    assert L.dflash_qmm_m16_workspace_bytes(320, 64, 32, nat.QMM_MMA2BIG, 1, nat.QMM_KERNEL_AUTO) == 0


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(nat, "_lib", None)
    monkeypatch.setattr(nat, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(nat.NativeLibraryError):
        nat.lib()
