"""ctypes binding of libdflash_mi355.so (the C ABI declared in include/dflash_mi355.h).

There is no software fallback: if the library has not been built, or an entry
point reports an error, the caller gets an exception.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdflash_mi355.so")

ABI_VERSION = 18

BF16, FP16, FP32 = 0, 1, 2
QMM_MMA2BIG, QMM_MMA2BIG_PIPE = 0, 1
QMM_KERNEL_AUTO, QMM_KERNEL_TILE, QMM_KERNEL_STREAM = 0, 1, 2
QMM_STATIC_SCRATCH_BYTES = 8 << 20  # DFLASH_QMM_STATIC_SCRATCH_BYTES
QMM_CHAIN_MAX = 16                       # DFLASH_QMM_CHAIN_MAX
QMM_ERROR_OFFSET = (16384 - 64 + 1) * 4        # DFLASH_QMM_ERROR_OFFSET
QMM_CHAIN_ERROR_OFFSET = QMM_ERROR_OFFSET      # DFLASH_QMM_CHAIN_ERROR_OFFSET
QMM_EPILOGUE_NONE, QMM_EPILOGUE_SILU_MUL = 0, 1
QMM_CHAIN_JOINT_SPLIT = 1                # DFLASH_QMM_CHAIN_JOINT_SPLIT
QMM_LAYOUT_ROWS, QMM_LAYOUT_PACKED = 0, 1  # DFLASH_QMM_LAYOUT_*
OPT_GDN_STEP_BY_STEP, OPT_SDPA_SPLITS, OPT_QMM_SPIN_LIMIT = 0, 1, 2  # DFLASH_OPT_*


class QmmProblem(ctypes.Structure):
    """dflash_qmm_problem of include/dflash_mi355.h."""
    _fields_ = [("x", ctypes.c_void_p), ("w_q", ctypes.c_void_p), ("scales", ctypes.c_void_p),
                ("biases", ctypes.c_void_p), ("y", ctypes.c_void_p), ("K", ctypes.c_int), ("N", ctypes.c_int),
                ("wait_for", ctypes.c_int), ("epilogue", ctypes.c_int), ("layout", ctypes.c_int)]

# every symbol include/dflash_mi355.h declares
EXPORTED_SYMBOLS = (
    "dflash_abi_version",
    "dflash_last_error",
    "dflash_set_option",
    "dflash_get_option",
    "dflash_qmm_m16_workspace_bytes",
    "dflash_qmm_m16",
    "dflash_qmm_error",
    "dflash_qmm_m16_static",
    "dflash_qmm_m16_pack_gate_up",
    "dflash_qmm_m16_chain_workspace_bytes",
    "dflash_qmm_m16_chain",
    "dflash_qmm_m16_packed_bytes",
    "dflash_qmm_m16_pack",
    "dflash_qmm_m16_packed",
    "dflash_qmm_m16_gather_workspace_bytes",
    "dflash_qmm_m16_gather",
    "dflash_tape_replay",
    "dflash_gdn_forward_tape",
    "dflash_gdn_forward_tape_norm",
    "dflash_gdn_prepare",
    "dflash_gdn_gated_norm",
    "dflash_sdpa_q16_workspace_bytes",
    "dflash_sdpa_q16",
    "dflash_conv_state_rebuild",
    "dflash_rollback_layer",
)


class NativeLibraryError(RuntimeError):
    """The HIP library is missing, mismatched, or one of its calls failed."""


_lib: Optional[ctypes.CDLL] = None


def _declare(lib: ctypes.CDLL) -> None:
    c = ctypes
    lib.dflash_abi_version.restype = c.c_int
    lib.dflash_abi_version.argtypes = []
    lib.dflash_last_error.restype = c.c_char_p
    lib.dflash_last_error.argtypes = []
    lib.dflash_set_option.restype = c.c_int
    lib.dflash_set_option.argtypes = [c.c_int, c.c_int]
    lib.dflash_get_option.restype = c.c_int
    lib.dflash_get_option.argtypes = [c.c_int]
    lib.dflash_qmm_m16_workspace_bytes.restype = c.c_size_t
    lib.dflash_qmm_m16_workspace_bytes.argtypes = [c.c_int] * 6
    lib.dflash_qmm_m16.restype = c.c_int
    lib.dflash_qmm_m16.argtypes = (
        [c.c_void_p] * 6 + [c.c_size_t] + [c.c_int] * 8 + [c.c_void_p]
    )
    lib.dflash_qmm_error.restype = c.c_int
    lib.dflash_qmm_error.argtypes = [c.c_void_p, c.POINTER(c.c_uint32), c.c_void_p]
    lib.dflash_qmm_m16_static.restype = c.c_int
    lib.dflash_qmm_m16_static.argtypes = [c.c_void_p] * 5 + [c.c_int] * 8 + [c.c_void_p]
    lib.dflash_qmm_m16_chain_workspace_bytes.restype = c.c_size_t
    lib.dflash_qmm_m16_chain_workspace_bytes.argtypes = [c.POINTER(QmmProblem), c.c_int, c.c_int, c.c_int]
    lib.dflash_qmm_m16_chain.restype = c.c_int
    lib.dflash_qmm_m16_chain.argtypes = [c.POINTER(QmmProblem), c.c_int, c.c_void_p, c.c_size_t] + [c.c_int] * 5 + [c.c_void_p]
    lib.dflash_qmm_m16_packed_bytes.restype = c.c_int
    lib.dflash_qmm_m16_packed_bytes.argtypes = [c.c_int] * 3 + [c.POINTER(c.c_size_t)] * 2
    lib.dflash_qmm_m16_pack.restype = c.c_int
    lib.dflash_qmm_m16_pack.argtypes = [c.c_void_p] * 6 + [c.c_int] * 3 + [c.c_void_p]
    lib.dflash_qmm_m16_pack_gate_up.restype = c.c_int
    lib.dflash_qmm_m16_pack_gate_up.argtypes = [c.c_void_p] * 6 + [c.c_int] * 3 + [c.c_void_p]
    lib.dflash_qmm_m16_packed.restype = c.c_int
    lib.dflash_qmm_m16_packed.argtypes = [c.c_void_p] * 6 + [c.c_size_t] + [c.c_int] * 5 + [c.c_void_p]
    lib.dflash_qmm_m16_gather_workspace_bytes.restype = c.c_size_t
    lib.dflash_qmm_m16_gather_workspace_bytes.argtypes = [c.c_int] * 5
    lib.dflash_qmm_m16_gather.restype = c.c_int
    lib.dflash_qmm_m16_gather.argtypes = (
        [c.c_void_p] * 7 + [c.c_size_t] + [c.c_int] * 7 + [c.c_void_p]
    )
    lib.dflash_gdn_forward_tape.restype = c.c_int
    lib.dflash_gdn_forward_tape.argtypes = [c.c_void_p] * 10 + [c.c_int] * 11 + [c.c_void_p]
    lib.dflash_gdn_forward_tape_norm.restype = c.c_int
    lib.dflash_gdn_forward_tape_norm.argtypes = [c.c_void_p] * 12 + [c.c_int] * 12 + [c.c_float, c.c_void_p]
    lib.dflash_gdn_prepare.restype = c.c_int
    lib.dflash_gdn_prepare.argtypes = [c.c_void_p] * 14 + [c.c_int] * 9 + [c.c_float, c.c_void_p]
    lib.dflash_gdn_gated_norm.restype = c.c_int
    lib.dflash_gdn_gated_norm.argtypes = [c.c_void_p] * 4 + [c.c_longlong] + [c.c_int] * 3 + [c.c_float, c.c_void_p]
    lib.dflash_sdpa_q16_workspace_bytes.restype = c.c_size_t
    lib.dflash_sdpa_q16_workspace_bytes.argtypes = [c.c_int] * 5
    lib.dflash_sdpa_q16.restype = c.c_int
    lib.dflash_sdpa_q16.argtypes = ([c.c_void_p] * 6 + [c.c_size_t] + [c.c_int] * 5 + [c.c_longlong] * 6 +
                                    [c.c_float, c.c_int, c.c_void_p])
    lib.dflash_tape_replay.restype = c.c_int
    lib.dflash_tape_replay.argtypes = (
        [c.c_void_p] * 6 + [c.c_int] + [c.c_void_p] + [c.c_int] * 12 + [c.c_void_p]
    )


    lib.dflash_conv_state_rebuild.restype = c.c_int
    lib.dflash_conv_state_rebuild.argtypes = [c.c_void_p] * 4 + [c.c_int] * 6 + [c.c_void_p]
    lib.dflash_rollback_layer.restype = c.c_int
    lib.dflash_rollback_layer.argtypes = [c.c_void_p] * 9 + [c.c_int] * 16 + [c.c_void_p]


def lib() -> ctypes.CDLL:
    """Load (once) and return the native library; raise if it is not there."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise NativeLibraryError(
            f"{LIB_PATH} not found: build it with `python dflash-mlx_amd/build_ext.py` "
            "(hipcc --offload-arch=gfx950); there is no fallback for the HIP path"
        )
    loaded = ctypes.CDLL(LIB_PATH)
    for name in EXPORTED_SYMBOLS:
        if not hasattr(loaded, name):
            raise NativeLibraryError(f"{LIB_PATH} does not export {name}")
    _declare(loaded)
    got = loaded.dflash_abi_version()
    if got != ABI_VERSION:
        raise NativeLibraryError(f"ABI version {got} != expected {ABI_VERSION}; rebuild the library")
    _lib = loaded
    return loaded


def is_built() -> bool:
    return os.path.exists(LIB_PATH)


def raw_stream(device) -> int:
    """Handle of the current stream of ``device`` (torch's Stream object costs microseconds per
    call to build; the handle is all the C ABI takes)."""
    import torch

    index = device.index if device.index is not None else torch.cuda.current_device()
    try:
        return torch._C._cuda_getCurrentRawStream(index)
    except AttributeError:  # a torch without the raw accessor
        return torch.cuda.current_stream(device).cuda_stream


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = lib().dflash_last_error().decode("utf-8", "replace")
        raise NativeLibraryError(f"{what} failed (code {rc}): {msg}")
