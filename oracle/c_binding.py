"""ctypes binding of liboracle_c.so (the C restatement in dflash_oracle_c.c).

Test infrastructure only.  ``build_c_oracle`` compiles it with gcc when asked;
``load_c_oracle`` loads the built library.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle_c.so")


def build_c_oracle(force: bool = True) -> str:
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "-B", "liboracle_c.so"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


class COracle:
    def __init__(self, lib: ctypes.CDLL):
        self._lib = lib
        c = ctypes
        lib.oracle_qmm_m16.restype = c.c_int
        lib.oracle_qmm_m16.argtypes = [c.c_void_p] * 6 + [c.c_int] * 6
        lib.oracle_tape_replay.restype = c.c_int
        lib.oracle_tape_replay.argtypes = [c.c_void_p] * 7 + [c.c_int] * 8
        lib.oracle_num_threads.restype = c.c_int

    def num_threads(self) -> int:
        return int(self._lib.oracle_num_threads())

    def qmm_m16(self, x_bf16, w_u32, scales_bf16, biases_bf16, group_size, *, flavour=0, k_parts=1):
        """x_bf16 [M,K] uint16 bits; returns (y_f32 [M,N], y_bf16 bits [M,N])."""
        x = np.ascontiguousarray(x_bf16, dtype=np.uint16)
        w = np.ascontiguousarray(w_u32).view(np.uint32)
        s = np.ascontiguousarray(scales_bf16, dtype=np.uint16)
        b = np.ascontiguousarray(biases_bf16, dtype=np.uint16)
        m, k = x.shape
        n = w.shape[0]
        y32 = np.empty((m, n), dtype=np.float32)
        y16 = np.empty((m, n), dtype=np.uint16)
        rc = self._lib.oracle_qmm_m16(x.ctypes.data, w.ctypes.data, s.ctypes.data, b.ctypes.data,
                                      y32.ctypes.data, y16.ctypes.data, m, k, n, group_size,
                                      flavour, k_parts)
        if rc != 0:
            raise ValueError(f"oracle_qmm_m16 rc={rc}")
        return y32, y16

    def tape_replay(self, tape, k_bf16, g_f32, state_f32, steps=None, mask=None):
        """tape [S,T,Hv,Dv] (uint16 bf16 bits or float32); k [S,T,Hk,Dk] uint16;
        g [S,T,Hv] or [S,T,Hv,Dk] float32; state [S,Hv,Dv,Dk] float32."""
        tape = np.ascontiguousarray(tape)
        tape_f32 = 1 if tape.dtype == np.float32 else 0
        if not tape_f32:
            tape = tape.astype(np.uint16, copy=False)
        k = np.ascontiguousarray(k_bf16, dtype=np.uint16)
        g = np.ascontiguousarray(g_f32, dtype=np.float32)
        st = np.ascontiguousarray(state_f32, dtype=np.float32)
        S, T, Hv, Dv = tape.shape
        Hk, Dk = k.shape[2], k.shape[3]
        out = np.empty_like(st)
        steps_p = None
        if steps is not None:
            steps = np.ascontiguousarray(steps, dtype=np.int32)
            steps_p = steps.ctypes.data
        mask_p = None
        if mask is not None:
            mask = np.ascontiguousarray(mask, dtype=np.uint8)
            mask_p = mask.ctypes.data
        rc = self._lib.oracle_tape_replay(tape.ctypes.data, k.ctypes.data, g.ctypes.data,
                                          st.ctypes.data, out.ctypes.data, steps_p, mask_p,
                                          S, T, Hk, Hv, Dk, Dv, tape_f32, 1 if g.ndim == 4 else 0)
        if rc != 0:
            raise ValueError(f"oracle_tape_replay rc={rc}")
        return out


def load_c_oracle(build_if_missing: bool = True) -> COracle:
    if not os.path.exists(_LIB_PATH):
        if not build_if_missing:
            raise FileNotFoundError(_LIB_PATH)
        build_c_oracle()
    return COracle(ctypes.CDLL(_LIB_PATH))
