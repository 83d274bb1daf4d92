"""M=16 int4 affine quantized matmul for the target-verify step (host side).

Mirror of dflash_mlx/verify_qmm.py: the same call surface, env switches, gate
and shape dispatch, with the device work done by the gfx950 kernel behind
``dflash_qmm_m16`` (include/dflash_mi355.h) instead of a Metal kernel.

    verify_matmul(x, w, scales, biases, *, transpose=True, group_size=64, bits=4)

* ``DFLASH_VERIFY_QMM=1`` enables the kernel (verify_qmm.py:11-12); otherwise, and
  for every call the gate rejects (verify_qmm.py:246-263) or whose shape fails a
  divisibility guard (:300, :317), the stock ``quantized_matmul`` runs instead -
  silently, as in the reference.
* ``DFLASH_VERIFY_VARIANT`` in {auto, mma2big, mma2big_pipe} and
  ``DFLASH_VERIFY_QMM_KPARTS`` select the variant (:15-22, 292-297).
* ``DFLASH_QMM_KERNEL`` in {auto, tile, stream} picks the device kernel (no counterpart
  in the reference; auto uses the streaming kernel for group 64 and K % 512 == 0).
* An eligible call needs device tensors and the built HIP library; there is no
  software fallback for it.
"""
from __future__ import annotations

import ctypes
import os
from typing import Dict, Optional, Tuple

import torch

from . import _native
from .quantized import quantized_matmul

_DTYPE_CODE = {torch.bfloat16: _native.BF16, torch.float16: _native.FP16}
_VARIANT_CODE = {"mma2big": _native.QMM_MMA2BIG, "mma2big_pipe": _native.QMM_MMA2BIG_PIPE}
_KERNEL_CODE = {"auto": _native.QMM_KERNEL_AUTO, "tile": _native.QMM_KERNEL_TILE,
                "stream": _native.QMM_KERNEL_STREAM}


def _kernel_select() -> int:
    """``DFLASH_QMM_KERNEL`` in {auto, tile, stream}: which device kernel serves eligible
    calls (auto: the streaming kernel wherever it applies, the tile kernel elsewhere)."""
    return _KERNEL_CODE.get(os.environ.get("DFLASH_QMM_KERNEL", "auto").strip().lower(),
                            _native.QMM_KERNEL_AUTO)


def is_enabled() -> bool:
    return os.environ.get("DFLASH_VERIFY_QMM", "") == "1"


def _variant() -> str:
    return os.environ.get("DFLASH_VERIFY_VARIANT", "auto")


def _auto_variant(K: int, N: int) -> Tuple[str, int]:
    if K >= 8192 or N <= 8192:
        return ("mma2big_pipe", 8)
    return ("mma2big", 1)


def _should_use_verify(x: torch.Tensor, group_size: int, bits: int, transpose: bool) -> bool:
    if not is_enabled():
        return False
    if bits != 4 or group_size not in (32, 64, 128):
        return False
    if x.dtype not in (torch.bfloat16, torch.float16):
        return False
    if not transpose:
        return False
    m = 1
    for d in x.shape[:-1]:
        m *= d
    return m == 16


# One zero-initialised scratch buffer per (device, stream): calls on a stream are
# ordered, so they can share it; the kernel hands it back zeroed where it has to be.
_WORKSPACES: Dict[Tuple[int, int], torch.Tensor] = {}


# what dflash_qmm_m16_workspace_bytes answered per (K, N, group size, variant, k_parts, kernel)
_WORKSPACE_BYTES: Dict[Tuple[int, int, int, int, int, int], int] = {}


def _workspace(device: torch.device, stream: int, nbytes: int) -> torch.Tensor:
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream)
    ws = _WORKSPACES.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.zeros(max(nbytes, 1 << 23), dtype=torch.uint8, device=device)
        _WORKSPACES[key] = ws
    return ws


def raise_on_device_errors(device: Optional[torch.device] = None) -> None:
    """Call where the host synchronises with the device anyway (the read-back of the acceptance
    length in a speculative cycle): a bounded wait inside a qmm kernel that gave up - a chained
    projection waiting for its input, the streaming kernel's adding workgroup waiting for partial
    tiles - leaves a word in the workspace and wrong outputs behind, and nothing else tells the
    caller.  Reads that word of every workspace of ``device`` (all devices if None; each read waits
    for the device); on a non-zero word the workspace is zero-filled again, as its contract asks,
    and ``NativeLibraryError`` raised."""
    for (index, stream), ws in list(_WORKSPACES.items()):
        if device is not None and device.index is not None and device.index != index:
            continue
        word = int(ws[_native.QMM_ERROR_OFFSET:_native.QMM_ERROR_OFFSET + 4].view(torch.int32).item()) & 0xFFFFFFFF
        if word == 0:
            continue
        ws.zero_()
        if word & 0x80000000:
            what = f"the streaming kernel gave up waiting for the partial tiles of row block {word & 0x3FFFFFFF}"
        else:
            what = f"projection {word - 1} of a chained launch gave up waiting for its input"
        raise _native.NativeLibraryError(
            f"qmm workspace of device {index}, stream {stream:#x}: {what}; the outputs of that launch and of "
            "everything computed from them are undefined (is the device shared with a long-running kernel?)")


def _require_operands(who: str, K: int, N: int, group_size: int, w: torch.Tensor, scales: torch.Tensor,
                      biases: torch.Tensor, device: torch.device, lead: Tuple[int, ...] = ()) -> None:
    """The kernels read what K, N and the group size say: weights of any other extent, word size
    or device must not reach them (``lead``: leading extents, the experts of the gathered form)."""
    groups = lead + (N, K // group_size)
    if (tuple(w.shape) != lead + (N, K // 8) or w.element_size() != 4 or tuple(scales.shape) != groups
            or tuple(biases.shape) != groups or scales.dtype not in _DTYPE_CODE or biases.dtype != scales.dtype
            or not (w.device == scales.device == biases.device == device)):
        raise ValueError(f"{who}: K={K}, N={N} need w {list(lead + (N, K // 8))} of 32-bit words and bf16/fp16 scales, "
                         f"biases {list(groups)} on {device}; got {tuple(w.shape)} {w.dtype}, {tuple(scales.shape)} "
                         f"{scales.dtype}, {tuple(biases.shape)} {biases.dtype} on {w.device}, {scales.device}, "
                         f"{biases.device}")


def _launch(x2: torch.Tensor, w: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor,
            K: int, N: int, group_size: int, variant: str, k_parts: int) -> torch.Tensor:
    if not x2.is_cuda:
        raise _native.NativeLibraryError(
            "verify_matmul: the M=16 kernel runs on the GPU only; got tensors on "
            f"{x2.device} (unset DFLASH_VERIFY_QMM to use the stock operator)")
    lib = _native.lib()
    if scales.dtype not in _DTYPE_CODE or biases.dtype != scales.dtype:
        raise TypeError(f"scales/biases must both be bf16 or fp16, got {scales.dtype}/{biases.dtype}")
    _require_operands("verify_matmul", K, N, group_size, w, scales, biases, x2.device)
    y = torch.empty((16, N), dtype=x2.dtype, device=x2.device)
    stream = _native.raw_stream(x2.device)
    vcode = _VARIANT_CODE[variant]
    kernel = _kernel_select()
    key = (K, N, group_size, vcode, k_parts, kernel)
    need = _WORKSPACE_BYTES.get(key)
    if need is None:
        need = _WORKSPACE_BYTES[key] = int(lib.dflash_qmm_m16_workspace_bytes(*key))
    ws_ptr, ws_bytes = None, 0
    if need:
        ws = _workspace(x2.device, stream, need)
        ws_ptr, ws_bytes = ws.data_ptr(), ws.numel()
    rc = lib.dflash_qmm_m16(x2.data_ptr(), w.data_ptr(), scales.data_ptr(), biases.data_ptr(),
                            y.data_ptr(), ws_ptr, ws_bytes, K, N, group_size,
                            _DTYPE_CODE[x2.dtype], _DTYPE_CODE[scales.dtype], vcode, k_parts, kernel,
                            stream)
    _native.check(rc, "dflash_qmm_m16")
    return y


def verify_matmul(x: torch.Tensor, w: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor,
                  *, transpose: bool = True, group_size: int = 64, bits: int = 4) -> torch.Tensor:
    if not _should_use_verify(x, group_size, bits, transpose):
        return quantized_matmul(x, w, scales, biases, transpose=transpose,
                                group_size=group_size, bits=bits)

    orig_shape = x.shape
    x2 = x.reshape(16, orig_shape[-1]).contiguous()
    w_q = w.contiguous()
    scales = scales.contiguous()
    biases = biases.contiguous()

    K = int(x2.shape[-1])
    N = int(w_q.shape[0])

    variant = _variant()
    auto_kp = None
    if variant == "auto":
        variant, auto_kp = _auto_variant(K, N)

    K_PARTS = auto_kp if auto_kp is not None else int(os.environ.get("DFLASH_VERIFY_QMM_KPARTS", "4"))

    if variant == "mma2big_pipe":
        if N % 32 != 0 or K % (32 * K_PARTS) != 0:
            return quantized_matmul(x, w, scales, biases, transpose=transpose,
                                    group_size=group_size, bits=bits)
        y = _launch(x2, w_q, scales, biases, K, N, group_size, "mma2big_pipe", K_PARTS)
        return y.reshape(*orig_shape[:-1], N)

    if N % 32 != 0 or K % 32 != 0:
        return quantized_matmul(x, w, scales, biases, transpose=transpose,
                                group_size=group_size, bits=bits)
    y = _launch(x2, w_q, scales, biases, K, N, group_size, "mma2big", 1)
    return y.reshape(*orig_shape[:-1], N)


def verify_qmm(x: torch.Tensor, w_packed: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor,
               group_size: int = 64, bits: int = 4, *, transpose: bool = True) -> torch.Tensor:
    """The name the hot path is known by: ``verify_matmul`` with ``group_size`` and ``bits``
    accepted positionally as well."""
    return verify_matmul(x, w_packed, scales, biases, transpose=transpose, group_size=group_size, bits=bits)


class ChainProblem:
    """One projection of a ``QmmChain``: ``y = x @ dequant(w, scales, biases).T`` for 16 rows.

    ``x`` is a device tensor of 16 rows of K values, or the ``ChainProblem`` whose output this
    projection reads (its weights then stream while that output is still being computed).
    ``epilogue="silu_mul"``: ``w``/``scales``/``biases`` hold the gate rows followed by the up rows
    of an MLP and the output is ``silu(gate) * up`` of ``[16, N/2]``.
    ``w`` may be a ``PackedWeights`` (``pack_weights``; ``scales`` and ``biases`` are then left out):
    same bits out, the loads read consecutive memory; with ``epilogue="silu_mul"`` the images
    must come from ``pack_weights(..., gate_up=True)``."""

    def __init__(self, x, w, scales: Optional[torch.Tensor] = None, biases: Optional[torch.Tensor] = None, *,
                 epilogue: Optional[str] = None, out: Optional[torch.Tensor] = None):
        if epilogue not in (None, "silu_mul"):
            raise ValueError(f"unknown epilogue {epilogue!r}")
        self.packed = None
        if isinstance(w, PackedWeights):
            if scales is not None or biases is not None:
                raise ValueError("ChainProblem: packed weights come alone")
            if (epilogue == "silu_mul") != bool(w.gate_up):
                raise ValueError("ChainProblem: the silu-mul epilogue reads images of pack_weights(..., gate_up=True), "
                                 "every other problem those of pack_weights(...)")
            self.packed, w, scales, biases = w, w.codes, w.scales, w.biases
        elif scales is None or biases is None:
            raise ValueError("ChainProblem: scales and biases are missing")
        self.x, self.w, self.scales, self.biases = x, w, scales, biases
        self.epilogue, self.out = epilogue, out


class QmmChain:
    """Several 16-row quantized matmuls in ONE launch (``dflash_qmm_m16_chain``): the projections
    of a layer handed over as a list and run back to back by one persistent grid.  No counterpart
    in the reference, which launches its kernel once per projection
    (``dflash_mlx/verify_linear.py:103-143``); every output is bit for bit what ``verify_matmul``
    gives for the same operands through the streaming kernel.

    The chain is planned once (argument block, outputs, workspace) and can be launched any number
    of times: ``chain()`` enqueues the launch on the current stream and returns the outputs, which
    are the same tensors every time.  Inputs are read from where they were when the chain was
    built (``x`` tensors are not copied).  Needs 4-bit codes, group 64, K a multiple of 1024,
    N of 32, bf16/fp16 activations on the GPU; at most 16 projections.

    ``joint_split=True`` (independent projections only): the units of all projections are divided
    among the workgroups as ONE range, so that nearly every row block is computed by a single
    workgroup over all of K and hardly any partial sums cross workgroups.  Outputs then equal
    ``verify_matmul``'s to within one rounding of the output type (a row block's sum is cut in
    other places), and are the same from run to run."""

    def __init__(self, problems, *, group_size: int = 64, bits: int = 4, spin_limit: int = 0,
                 joint_split: bool = False):
        problems = list(problems)
        if bits != 4 or group_size != 64:
            raise ValueError("QmmChain: 4-bit codes in groups of 64 only")
        if not 1 <= len(problems) <= _native.QMM_CHAIN_MAX:
            raise ValueError(f"QmmChain: 1 to {_native.QMM_CHAIN_MAX} projections, got {len(problems)}")
        lib = _native.lib()
        self._keep, self.outputs = [], []
        self._table = (_native.QmmProblem * len(problems))()
        index = {}
        act = sb = device = None
        for i, pr in enumerate(problems):
            wait_for = -1
            if isinstance(pr.x, ChainProblem):
                if id(pr.x) not in index:
                    raise ValueError(f"QmmChain: projection {i} reads a projection that does not come before it")
                wait_for = index[id(pr.x)]
                x2 = self.outputs[wait_for]
            else:
                m = 1
                for d in pr.x.shape[:-1]:
                    m *= int(d)
                if m != 16 or not pr.x.is_cuda or pr.x.dtype not in _DTYPE_CODE:
                    raise ValueError(f"QmmChain: x of projection {i} must hold 16 rows of bf16/fp16 values on the GPU")
                x2 = pr.x.reshape(16, pr.x.shape[-1])
                if not x2.is_contiguous():
                    raise ValueError(f"QmmChain: x of projection {i} must be contiguous (it is read in place)")
            w, s, b = pr.w.contiguous(), pr.scales.contiguous(), pr.biases.contiguous()
            if pr.packed is not None:
                K, N = pr.packed.K, pr.packed.N
                if pr.packed.group_size != group_size or w.device != x2.device:
                    raise ValueError(f"QmmChain: packed weights of projection {i} do not fit this chain")
            else:
                K, N = int(w.shape[1]) * 8, int(w.shape[0])
            if int(x2.shape[1]) != K or s.dtype not in _DTYPE_CODE or b.dtype != s.dtype or N % 32 != 0:
                raise ValueError(f"QmmChain: operands of projection {i} do not fit together (K={K}, N={N})")
            if pr.packed is None:
                _require_operands(f"QmmChain, projection {i}", K, N, group_size, w, s, b, x2.device)
            act = x2.dtype if act is None else act
            sb = s.dtype if sb is None else sb
            device = x2.device if device is None else device
            if x2.dtype != act or s.dtype != sb or x2.device != device or w.device != device:
                raise ValueError("QmmChain: all projections share one activation dtype, one scale dtype and one device")
            cols = N // 2 if pr.epilogue == "silu_mul" else N
            y = pr.out if pr.out is not None else torch.empty((16, cols), dtype=act, device=device)
            if tuple(y.shape) != (16, cols) or y.dtype != act or not y.is_contiguous() or y.device != device:
                raise ValueError(f"QmmChain: out of projection {i} must be a contiguous [16, {cols}] tensor of {act}")
            t = self._table[i]
            t.x, t.w_q, t.scales, t.biases, t.y = x2.data_ptr(), w.data_ptr(), s.data_ptr(), b.data_ptr(), y.data_ptr()
            t.K, t.N, t.wait_for = K, N, wait_for
            t.epilogue = _native.QMM_EPILOGUE_SILU_MUL if pr.epilogue == "silu_mul" else _native.QMM_EPILOGUE_NONE
            t.layout = _native.QMM_LAYOUT_PACKED if pr.packed is not None else _native.QMM_LAYOUT_ROWS
            self._keep.append((x2, w, s, b))
            self.outputs.append(y)
            index[id(pr)] = i
        if len({pr.packed is not None for pr in problems}) > 1:
            raise ValueError("QmmChain: packed weights for all projections of a chain or for none")
        self._count, self._group = len(problems), group_size
        self._act, self._sb, self._device = _DTYPE_CODE[act], _DTYPE_CODE[sb], device
        self._spin = int(spin_limit)
        self._flags = _native.QMM_CHAIN_JOINT_SPLIT if joint_split else 0
        if joint_split and any(self._table[i].wait_for >= 0 for i in range(len(problems))):
            raise ValueError("QmmChain: joint_split is for projections that do not read each other")
        self._need = int(lib.dflash_qmm_m16_chain_workspace_bytes(self._table, self._count, group_size, self._flags))
        if self._need == 0:
            raise ValueError("QmmChain: a projection has a shape the chained kernel does not cover "
                             "(group 64, K % 1024 == 0, N % 32 == 0; N % 128 == 0 with an epilogue)")

    def __call__(self):
        stream = _native.raw_stream(self._device)
        ws = _workspace(self._device, stream, self._need)
        self._ws = ws
        rc = _native.lib().dflash_qmm_m16_chain(self._table, self._count, ws.data_ptr(), ws.numel(), self._group,
                                                self._act, self._sb, self._spin, self._flags, stream)
        _native.check(rc, "dflash_qmm_m16_chain")
        return self.outputs

    def rebind(self, index: int, *, x: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> None:
        """Points projection ``index`` at another input and/or output of the same shape and dtype
        for the launches that follow (a projection that reads another one keeps doing so; outputs
        that a later projection reads cannot be moved)."""
        t = self._table[index]
        x_old, w, s, b = self._keep[index]
        if x is not None:
            if t.wait_for >= 0:
                raise ValueError("QmmChain.rebind: this projection reads another projection's output")
            x2 = x.reshape(16, x.shape[-1]) if x.numel() == x_old.numel() else x
            if tuple(x2.shape) != tuple(x_old.shape) or x2.dtype != x_old.dtype or x2.device != x_old.device \
                    or not x2.is_contiguous():
                raise ValueError(f"QmmChain.rebind: x must be a contiguous {tuple(x_old.shape)} tensor of {x_old.dtype}")
            t.x = x2.data_ptr()
            self._keep[index] = (x2, w, s, b)
        if out is not None:
            y_old = self.outputs[index]
            if any(self._table[j].wait_for == index for j in range(self._count)):
                raise ValueError("QmmChain.rebind: another projection of the chain reads this output")
            if tuple(out.shape) != tuple(y_old.shape) or out.dtype != y_old.dtype or out.device != y_old.device \
                    or not out.is_contiguous():
                raise ValueError(f"QmmChain.rebind: out must be a contiguous {tuple(y_old.shape)} tensor of {y_old.dtype}")
            t.y = out.data_ptr()
            self.outputs[index] = out

    def error_word(self) -> int:
        """0, or 1 + the index of a projection whose wait for its input was given up (read back
        from the workspace of the last launch; synchronises with the device)."""
        word = self._ws[_native.QMM_CHAIN_ERROR_OFFSET:_native.QMM_CHAIN_ERROR_OFFSET + 4]
        return int(word.view(torch.int32).item())

    def clear_error(self) -> None:
        self._ws[_native.QMM_CHAIN_ERROR_OFFSET:_native.QMM_CHAIN_ERROR_OFFSET + 4].zero_()

    def check(self) -> None:
        """Waits for the device and raises ``NativeLibraryError`` if a wait of the last launches
        was given up (``raise_on_device_errors`` for this chain's device).  A chain with
        projections that read one another should be checked before its outputs are trusted."""
        raise_on_device_errors(self._device)


class PackedWeights:
    """One linear's codes, scales and biases in the order the streaming kernel consumes them
    (``pack_weights``).  A second copy of the weights, made once when the model is loaded; the
    row-major MLX triple it was made from is not referenced."""

    __slots__ = ("codes", "scales", "biases", "K", "N", "group_size", "gate_up")

    def __init__(self, codes, scales, biases, K, N, group_size, gate_up=False):
        self.codes, self.scales, self.biases = codes, scales, biases
        self.K, self.N, self.group_size = K, N, group_size
        self.gate_up = gate_up  # rows ordered for the chained kernel's silu-mul epilogue: that use only


def packable(w: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor, group_size: int = 64,
             bits: int = 4) -> bool:
    """Shapes the packed form covers: 4 bits, group 64, K a multiple of 1024, N of 32 (the
    Python gate's rule for N), bf16/fp16 scales, device tensors."""
    if bits != 4 or group_size != 64 or w.ndim != 2 or not w.is_cuda:
        return False
    K, N = int(w.shape[1]) * 8, int(w.shape[0])
    return (K % 1024 == 0 and N % 32 == 0 and scales.dtype in _DTYPE_CODE and biases.dtype == scales.dtype
            and tuple(scales.shape) == (N, K // 64) and tuple(biases.shape) == (N, K // 64))


def pack_weights(w: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor, *, group_size: int = 64,
                 bits: int = 4, gate_up: bool = False) -> PackedWeights:
    """Rewrites an MLX affine triple (``w [N, K/8]`` words, ``scales``/``biases [N, K/64]``) into the
    packed images ``verify_matmul_packed`` reads: per 128 rows and 256 k the 16 KiB of codes in
    the order of the kernel's LDS slot, per 128 rows and 1024 k the 4 KiB of scales and of
    biases.  No counterpart in the reference, whose kernel gathers 4-byte words from the
    row-major arrays (``verify_qmm.py:68-72``).  ``gate_up=True``: ``w`` holds the gate rows of an
    MLP followed by its up rows, and the images are those a ``ChainProblem`` with the silu-mul
    epilogue reads (64 gate rows and the 64 up rows of the same columns per row block; N a
    multiple of 128) - not ``verify_matmul_packed``."""
    if gate_up and int(w.shape[0]) % 128 != 0:
        raise ValueError("pack_weights: gate_up needs a number of rows that is a multiple of 128")
    if not packable(w, scales, biases, group_size, bits):
        raise ValueError("pack_weights: needs 4-bit codes, group 64, K % 1024 == 0, N % 32 == 0, "
                         "bf16/fp16 scales and biases of shape [N, K/64], on the GPU")
    lib = _native.lib()
    K, N = int(w.shape[1]) * 8, int(w.shape[0])
    cb, sb = ctypes.c_size_t(), ctypes.c_size_t()
    _native.check(lib.dflash_qmm_m16_packed_bytes(K, N, group_size, ctypes.byref(cb), ctypes.byref(sb)),
                  "dflash_qmm_m16_packed_bytes")
    w, scales, biases = w.contiguous(), scales.contiguous(), biases.contiguous()
    codes = torch.empty(cb.value, dtype=torch.uint8, device=w.device)
    s_img = torch.empty(sb.value // 2, dtype=scales.dtype, device=w.device)
    b_img = torch.empty(sb.value // 2, dtype=scales.dtype, device=w.device)
    pack = lib.dflash_qmm_m16_pack_gate_up if gate_up else lib.dflash_qmm_m16_pack
    rc = pack(w.data_ptr(), scales.data_ptr(), biases.data_ptr(), codes.data_ptr(),
              s_img.data_ptr(), b_img.data_ptr(), K, N, group_size, _native.raw_stream(w.device))
    _native.check(rc, "dflash_qmm_m16_pack_gate_up" if gate_up else "dflash_qmm_m16_pack")
    return PackedWeights(codes, s_img, b_img, K, N, group_size, gate_up)


def verify_matmul_packed(x: torch.Tensor, packed: PackedWeights) -> torch.Tensor:
    """``verify_matmul`` on packed weights: 16 rows of bf16/fp16 device activations; the result is
    bit for bit that of the streaming kernel on the triple the weights were packed from."""
    K, N = packed.K, packed.N
    if packed.gate_up:
        raise ValueError("verify_matmul_packed: these images are ordered for the silu-mul epilogue of a chain")
    m = 1
    for d in x.shape[:-1]:
        m *= int(d)
    if m != 16 or int(x.shape[-1]) != K or x.dtype not in _DTYPE_CODE or not x.is_cuda:
        raise ValueError("verify_matmul_packed: x must hold 16 rows of K bf16/fp16 values on the GPU")
    lib = _native.lib()
    x2 = x.reshape(16, K).contiguous()
    y = torch.empty((16, N), dtype=x2.dtype, device=x2.device)
    stream = _native.raw_stream(x2.device)
    key = (K, N, packed.group_size, _VARIANT_CODE["mma2big"], 1, _native.QMM_KERNEL_STREAM)
    need = _WORKSPACE_BYTES.get(key)
    if need is None:
        need = _WORKSPACE_BYTES[key] = int(lib.dflash_qmm_m16_workspace_bytes(*key))
    ws = _workspace(x2.device, stream, need)
    rc = lib.dflash_qmm_m16_packed(x2.data_ptr(), packed.codes.data_ptr(), packed.scales.data_ptr(),
                                   packed.biases.data_ptr(), y.data_ptr(), ws.data_ptr(), ws.numel(),
                                   K, N, packed.group_size, _DTYPE_CODE[x2.dtype],
                                   _DTYPE_CODE[packed.scales.dtype], stream)
    _native.check(rc, "dflash_qmm_m16_packed")
    return y.reshape(*x.shape[:-1], N)


def small_m_matmul(x: torch.Tensor, w: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor,
                   *, group_size: int = 64, bits: int = 4) -> "torch.Tensor | None":
    """``x @ dequant(w).T`` for at most 16 rows of device activations through the M=16 kernel:
    the rows are padded with zeros to 16 (a row of the product depends on its own row of x only,
    so a row comes out the same whatever shares the block with it).  Covers what the C ABI covers
    (N a multiple of 16, K a multiple of the group size, bf16/fp16), which is more than the
    Python gate of ``verify_matmul`` lets through; returns None for anything else.  No
    counterpart in the reference, whose stock operator is a fused kernel of its own: here the
    stock operator dequantises the whole matrix with array ops, which for a one-token step or a
    48-row projection costs far more than the product itself."""
    if (not x.is_cuda or bits != 4 or group_size not in (32, 64, 128) or x.dtype not in _DTYPE_CODE or
            scales.dtype not in _DTYPE_CODE or biases.dtype != scales.dtype or w.ndim != 2 or not _native.is_built()):
        return None
    K, N = int(x.shape[-1]), int(w.shape[0])
    m = 1
    for d in x.shape[:-1]:
        m *= int(d)
    if m < 1 or m > 16 or N % 16 != 0 or K % group_size != 0 or K % 32 != 0 or int(w.shape[1]) * 8 != K:
        return None
    x2 = x.reshape(m, K)
    if m < 16:
        x16 = torch.zeros((16, K), dtype=x.dtype, device=x.device)
        x16[:m] = x2
    else:
        x16 = x2.contiguous()
    y = _launch(x16, w.contiguous(), scales.contiguous(), biases.contiguous(), K, N, group_size, "mma2big", 1)
    return y[:m].reshape(*x.shape[:-1], N)


def gather_qmm(x: torch.Tensor, w: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor,
               expert_ids: torch.Tensor, *, group_size: int = 64, bits: int = 4) -> torch.Tensor:
    """Per-row expert selection for MoE layers: ``y[p] = x[p] @ dequant(w[expert_ids[p]]).T``.

    ``x [P, K]`` bf16/fp16, ``w [E, N, K/8]`` packed, ``scales``/``biases [E, N, K/group]``,
    ``expert_ids [P]`` integer.  Not part of the reference (its experts use mlx_lm's switch
    layers); provided for the MoE-shaped verify step.  Device tensors only."""
    if bits != 4:
        raise NotImplementedError("only 4-bit codes are implemented")
    if not x.is_cuda:
        raise _native.NativeLibraryError("gather_qmm runs on the GPU only")
    lib = _native.lib()
    x2 = x.reshape(-1, x.shape[-1]).contiguous()
    ids = expert_ids.reshape(-1).to(torch.int32).contiguous()
    w_q, scales, biases = w.contiguous(), scales.contiguous(), biases.contiguous()
    P, K = int(x2.shape[0]), int(x2.shape[1])
    E, N = int(w_q.shape[0]), int(w_q.shape[1])
    if ids.numel() != P:
        raise ValueError("one expert id per row of x is required")
    if w_q.ndim != 3 or x2.dtype not in _DTYPE_CODE or ids.device != x2.device:
        raise ValueError("gather_qmm: w [E, N, K/8], bf16/fp16 x and the expert ids on x's device are required")
    _require_operands("gather_qmm", K, N, group_size, w_q, scales, biases, x2.device, lead=(E,))
    y = torch.empty((P, N), dtype=x2.dtype, device=x2.device)
    stream = _native.raw_stream(x2.device)
    # DFLASH_QMM_KERNEL=tile keeps the streaming kernel out of the gathered form as well
    need = 0 if _kernel_select() == _native.QMM_KERNEL_TILE else \
        lib.dflash_qmm_m16_gather_workspace_bytes(P, K, N, E, group_size)
    ws_ptr, ws_bytes = None, 0
    if need:
        ws = _workspace(x2.device, stream, need)
        ws_ptr, ws_bytes = ws.data_ptr(), ws.numel() * ws.element_size()
    rc = lib.dflash_qmm_m16_gather(x2.data_ptr(), ids.data_ptr(), w_q.data_ptr(), scales.data_ptr(),
                                   biases.data_ptr(), y.data_ptr(), ws_ptr, ws_bytes, P, K, N, E,
                                   group_size, _DTYPE_CODE[x2.dtype], _DTYPE_CODE[scales.dtype], stream)
    _native.check(rc, "dflash_qmm_m16_gather")
    return y.reshape(*x.shape[:-1], N)


def join_expert_projections(*projections):
    """Lays the rows of several per-expert projections that read the same rows of x (gate and up
    of a switch MLP) end to end per expert: from ``(w [E, N_i, K/8], scales, biases)`` triples to
    one ``(w [E, sum N_i, K/8], scales, biases)`` and the column bounds of each in the joint output,
    so that one ``gather_qmm`` launch serves them all (a launch costs the same ~8 us around its
    weight stream whether it covers one projection or two)."""
    if len(projections) < 2:
        raise ValueError("at least two (w, scales, biases) triples are needed")
    w = torch.cat([p[0] for p in projections], dim=1).contiguous()
    scales = torch.cat([p[1] for p in projections], dim=1).contiguous()
    biases = torch.cat([p[2] for p in projections], dim=1).contiguous()
    bounds, row = [], 0
    for p in projections:
        bounds.append((row, row + int(p[0].shape[1])))
        row += int(p[0].shape[1])
    return (w, scales, biases), bounds


def append_shared_expert(experts, shared):
    """Stores an always-active shared expert behind the routed experts of the same shape: from
    ``(w [E, N, K/8], scales, biases)`` and the shared expert's ``(w [N, K/8], scales, biases)`` to
    one ``(w [E+1, N, K/8], scales, biases)`` and the shared expert's id ``E``.  With
    ``shared_expert_rows`` one ``gather_qmm`` launch then serves the routed pairs and the shared
    expert, instead of a gathered launch plus a ``verify_matmul`` launch per projection.  Done
    once when the weights are loaded; no counterpart in the reference (its shared expert is a
    plain linear next to mlx_lm's switch layers)."""
    (w, scales, biases), (sw, ss, sb) = experts, shared
    if tuple(sw.shape) != tuple(w.shape[1:]) or tuple(ss.shape) != tuple(scales.shape[1:]) \
            or tuple(sb.shape) != tuple(biases.shape[1:]):
        raise ValueError("the shared expert must have the shape of one routed expert")
    if sw.dtype != w.dtype or ss.dtype != scales.dtype or sb.dtype != biases.dtype:
        raise ValueError("the shared expert must have the dtypes of the routed experts")
    joined = tuple(torch.cat([a, b.unsqueeze(0)], dim=0).contiguous()
                   for a, b in ((w, sw), (scales, ss), (biases, sb)))
    return joined, int(w.shape[0])


def shared_expert_rows(x_pairs: torch.Tensor, expert_ids: torch.Tensor, x_tokens: torch.Tensor,
                       shared_id: int):
    """Rows and expert ids of a gathered launch that also runs the shared expert: the
    ``[P, K]`` rows of the routed (token, expert) pairs followed by the ``[T, K]`` rows the
    shared expert reads, all of the latter with id ``shared_id``.  Rows ``[:P]`` of the
    launch's output belong to the routed pairs, rows ``[P:]`` to the shared expert."""
    xt = x_tokens.reshape(-1, x_tokens.shape[-1])
    x = torch.cat([x_pairs.reshape(-1, x_pairs.shape[-1]), xt], dim=0)
    ids = torch.cat([expert_ids.reshape(-1).to(torch.int32),
                     torch.full((xt.shape[0],), shared_id, dtype=torch.int32, device=expert_ids.device)])
    return x, ids
