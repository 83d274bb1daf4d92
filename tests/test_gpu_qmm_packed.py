"""The packed weight layout of the M=16 qmm: the pack kernel against an index-by-index
restatement of the layout, the packed product against the exact closed form and, bit for
bit, against the streaming kernel on the row-major triple, and the module-level switch.
The reference has no packed form; what is pinned is the product (same bar as the row-major
call) and the equality of the two routes."""
import ctypes

import numpy as np
import pytest
import torch

import dflash_mlx_amd._native as nat
from dflash_mlx_amd import verify_qmm as VQ
from dflash_mlx_amd.quantized import QuantizedLinear
from dflash_mlx_amd.verify_linear import (VerifyQuantizedLinear, fuse_shared_input_linears,
                                          install_verify_linears, pack_verify_linears)
from dflash_mlx_amd.workloads import make_qmm_case, seed_for

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _layout(case):
    """The images written index by index from the layout's definition: codes of unit (rb, st),
    instruction q, lane l = 16 bytes number (l & 7) ^ (((l >> 3) >> 1 & 3) << 1) of row
    128 rb + 8 q + (l >> 3) within bytes 128 st ..; scales of chunk (rb, c), part p, lane l =
    16 bytes number l & 1 of row 128 rb + 32 p + (l >> 1), groups 16 c ..; rows past N repeat
    the last row."""
    w = case.w.numpy().view(np.uint8)               # [N, K/2]
    s, b = _bits(case.scales).view(np.uint8), _bits(case.biases).view(np.uint8)  # [N, K/64 * 2]
    N, K = w.shape[0], w.shape[1] * 2
    RB, stages = (N + 127) // 128, K // 256
    codes = np.zeros((RB, stages, 16, 64, 16), np.uint8)
    for rb in range(RB):
        for q in range(16):
            for lane in range(64):
                r8 = lane >> 3
                row = min(rb * 128 + 8 * q + r8, N - 1)
                g = (lane & 7) ^ (((r8 >> 1) & 3) << 1)
                codes[rb, :, q, lane] = w[row].reshape(stages, 8, 16)[:, g]
    imgs = []
    for m in (s, b):
        img = np.zeros((RB, stages // 4, 4, 64, 16), np.uint8)
        for rb in range(RB):
            for part in range(4):
                for lane in range(64):
                    row = min(rb * 128 + 32 * part + (lane >> 1), N - 1)
                    img[rb, :, part, lane] = m[row].reshape(stages // 4, 2, 16)[:, lane & 1]
        imgs.append(img)
    return codes.reshape(-1), imgs[0].reshape(-1), imgs[1].reshape(-1)


@pytest.mark.parametrize("K,N", [(1024, 128), (2048, 352), (1024, 32)])
def test_pack_kernel_writes_the_stated_layout(native_lib, K, N):
    case = make_qmm_case(K, N, seed_for(0, 500 + N))
    d = case.to(DEV)
    pk = VQ.pack_weights(d.w, d.scales, d.biases)
    torch.cuda.synchronize()
    codes, s_img, b_img = _layout(case)
    RB = (N + 127) // 128
    assert pk.codes.numel() == RB * (K // 256) * 16384 and pk.scales.numel() * 2 == RB * (K // 1024) * 4096
    assert np.array_equal(pk.codes.cpu().numpy(), codes)
    assert np.array_equal(_bits(pk.scales).view(np.uint8), s_img)
    assert np.array_equal(_bits(pk.biases).view(np.uint8), b_img)


@pytest.mark.parametrize("K,N,dtype", [(4096, 4096, torch.bfloat16), (1024, 96, torch.bfloat16),
                                       (5120, 1184, torch.bfloat16), (2048, 512, torch.float16),
                                       (17408, 640, torch.bfloat16)])
def test_packed_product_equals_the_row_major_route(verify_env, native_lib, c_oracle, K, N, dtype):
    """Same bits as the streaming kernel on the row-major triple (one kernel, two address
    schemes), and the bar of the closed form."""
    verify_env.setenv("DFLASH_QMM_KERNEL", "stream")
    case = make_qmm_case(K, N, seed_for(0, 600 + N), dtype=dtype)
    d = case.to(DEV)
    pk = VQ.pack_weights(d.w, d.scales, d.biases)
    y = VQ.verify_matmul_packed(d.x, pk)
    ref = VQ.verify_matmul(d.x, d.w, d.scales, d.biases, group_size=64, bits=4)
    torch.cuda.synchronize()
    assert y.shape == (16, N) and y.dtype == dtype
    assert torch.equal(y, ref)
    assert torch.equal(y, VQ.verify_matmul_packed(d.x.reshape(2, 8, K), pk).reshape(16, N))
    if dtype == torch.bfloat16:
        exact, _ = c_oracle.qmm_m16(_bits(case.x), case.w.numpy().view(np.uint32), _bits(case.scales),
                                    _bits(case.biases), 64, flavour=0)
        exact = exact.astype(np.float64)
        yv = y.float().cpu().numpy().astype(np.float64)
        assert np.all(np.abs(yv - exact) <= 2e-2 * np.max(np.abs(exact), axis=1, keepdims=True))
        assert np.linalg.norm(yv - exact) / np.linalg.norm(exact) <= 5e-3


def test_packed_form_rejects_what_it_does_not_cover(native_lib):
    lib = nat.lib()
    cb, sb = ctypes.c_size_t(), ctypes.c_size_t()
    assert lib.dflash_qmm_m16_packed_bytes(1536, 128, 64, ctypes.byref(cb), ctypes.byref(sb)) != 0
    assert b"1024" in lib.dflash_last_error()
    assert lib.dflash_qmm_m16_packed_bytes(1024, 128, 32, ctypes.byref(cb), ctypes.byref(sb)) != 0
    assert lib.dflash_qmm_m16_packed_bytes(1024, 144, 64, ctypes.byref(cb), ctypes.byref(sb)) == 0
    assert (cb.value, sb.value) == (2 * 4 * 16384, 2 * 4096)
    case = make_qmm_case(1536, 64, 1).to(DEV)
    assert not VQ.packable(case.w, case.scales, case.biases)
    with pytest.raises(ValueError):
        VQ.pack_weights(case.w, case.scales, case.biases)
    ok = make_qmm_case(1024, 64, 2).to(DEV)
    pk = VQ.pack_weights(ok.w, ok.scales, ok.biases)
    with pytest.raises(ValueError):
        VQ.verify_matmul_packed(ok.x[:8], pk)
    small = torch.zeros(16, dtype=torch.uint8, device=DEV)
    rc = lib.dflash_qmm_m16_packed(ok.x.data_ptr(), pk.codes.data_ptr(), pk.scales.data_ptr(), pk.biases.data_ptr(),
                                   ok.x.data_ptr(), small.data_ptr(), 16, 1024, 64, 64, nat.BF16, nat.BF16, None)
    assert rc != 0 and b"workspace" in lib.dflash_last_error()


def test_modules_switch_to_their_packed_copy(verify_env, native_lib):
    """pack_verify_linears: stand-alone swapped linears of a covered shape get a packed copy and
    return the same bits; uncovered shapes are left alone;
    a shared-input group gets one for its joint matrix; other call shapes still use the row-major
    buffers; moving a module drops the copy."""
    verify_env.setenv("DFLASH_QMM_KERNEL", "auto")
    shapes = {"gate_proj": (1024, 512), "up_proj": (1024, 512), "down_proj": (2048, 1024), "odd": (1536, 256)}
    cases = {n: make_qmm_case(K, N, seed_for(0, 700 + i)) for i, (n, (K, N)) in enumerate(shapes.items())}
    mlp = torch.nn.Module()
    for n, c in cases.items():
        setattr(mlp, n, QuantizedLinear(c.w.clone(), c.scales.clone(), c.biases.clone(), group_size=64, bits=4))
    model = torch.nn.Module()
    model.mlp = mlp.to(DEV)
    assert install_verify_linears(model) == 4
    before = {n: getattr(model.mlp, n)(cases[n].x.to(DEV)) for n in cases}
    assert fuse_shared_input_linears(model) == 1
    group = model.mlp.gate_proj._shared_input[0]
    xg = cases["gate_proj"].x.to(DEV)
    joint = VQ.verify_matmul(xg, group.weight, group.scales, group.biases, group_size=64, bits=4)
    assert pack_verify_linears(model) == 2 and pack_verify_linears(model) == 0  # down_proj and the gate/up group
    assert model.mlp.down_proj._packed is not None and model.mlp.odd._packed is None
    assert model.mlp.gate_proj._packed is None and group._packed is not None and group._packed.N == 1024
    import dflash_mlx_amd.verify_linear as VL
    called = []
    real = VL.verify_matmul_packed
    try:
        VL.verify_matmul_packed = lambda x, p: (called.append(p.N), real(x, p))[1]
        object.__setattr__(model.mlp.down_proj, "_call_fn", VL._build_dispatch(model.mlp.down_proj))
        both = VL.shared_input_outputs(model.mlp, ("gate_proj", "up_proj"), xg)
        after = {n: getattr(model.mlp, n)(cases[n].x.to(DEV)) for n in ("down_proj", "odd")}
    finally:
        VL.verify_matmul_packed = real
    torch.cuda.synchronize()
    assert called == [1024, 1024]  # the gate/up group's joint matrix, then down_proj
    assert torch.equal(torch.cat(both, dim=-1), joint)
    # members asked one by one: their rows of the row-major joint matrix, the same values
    assert torch.equal(model.mlp.gate_proj(xg), before["gate_proj"])
    for n in ("down_proj", "odd"):
        assert torch.equal(before[n], after[n])
    x3 = torch.randn(3, 2048, device=DEV).to(torch.bfloat16)
    c = cases["down_proj"].to(DEV)
    assert torch.equal(model.mlp.down_proj(x3), QuantizedLinear(c.w, c.scales, c.biases, group_size=64, bits=4)(x3))
    assert isinstance(model.mlp.down_proj, VerifyQuantizedLinear)
    model.mlp.down_proj.to(DEV)  # _apply runs: the copy is dropped
    assert model.mlp.down_proj._packed is None
