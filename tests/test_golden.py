"""Committed fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py from the
oracle; self-generated, the reference tree holds none): the oracle must keep reproducing
them on the CPU, and the device kernels must meet the parity bars on them."""
import glob
import os

import numpy as np
import pytest
import torch

from oracle import dflash_oracle as O

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
QMM = sorted(glob.glob(os.path.join(HERE, "qmm_*.npz")))


def test_fixtures_present():
    assert len(QMM) == 2 and os.path.exists(os.path.join(HERE, "replay_s3_t16.npz"))


@pytest.mark.parametrize("path", QMM, ids=os.path.basename)
def test_oracle_reproduces_qmm_fixture(path, c_oracle):
    f = np.load(path)
    gs = int(f["group_size"])
    xf, sf, bf = O.bf16_to_f32(f["x"]), O.bf16_to_f32(f["scales"]), O.bf16_to_f32(f["biases"])
    np.testing.assert_allclose(O.qmm_exact(xf, f["w"], sf, bf, gs), f["y_exact"], rtol=1e-13, atol=1e-13)
    assert np.array_equal(O.f32_to_bf16(O.qmm_kernel_semantics(xf, f["w"], sf, bf, gs)), f["y_kernel_bf16"])
    y32, _ = c_oracle.qmm_m16(f["x"], f["w"], f["scales"], f["biases"], gs, flavour=0)
    np.testing.assert_allclose(y32, f["y_exact"], rtol=2e-7, atol=1e-6)


def test_oracle_reproduces_replay_fixture(c_oracle):
    f = np.load(os.path.join(HERE, "replay_s3_t16.npz"))
    got = c_oracle.tape_replay(f["tape"], f["k"], f["g"], f["state"], steps=f["steps"])
    np.testing.assert_allclose(got, f["state_out"], rtol=2e-6, atol=1e-7)
    for s in range(3):
        want = O.rebuild_conv_state(f["conv"][s:s + 1], f["qkv"][s:s + 1], int(f["steps"][s]), 4)[0]
        assert np.array_equal(want, f["conv_out"][s])


def _bf16_tensor(bits):
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)


@pytest.mark.gpu
@pytest.mark.parametrize("kernel", ["auto", "tile"])
@pytest.mark.parametrize("path", QMM, ids=os.path.basename)
def test_device_qmm_on_fixture(path, kernel, verify_env, native_lib):
    from dflash_mlx_amd import verify_qmm as VQ

    verify_env.setenv("DFLASH_QMM_KERNEL", kernel)
    f = np.load(path)
    dev = "cuda:0"
    y = VQ.verify_matmul(_bf16_tensor(f["x"]).to(dev), torch.from_numpy(f["w"].view(np.int32)).to(dev),
                         _bf16_tensor(f["scales"]).to(dev), _bf16_tensor(f["biases"]).to(dev),
                         group_size=int(f["group_size"]), bits=4)
    yv = y.float().cpu().numpy().astype(np.float64)
    exact = f["y_exact"]
    assert np.all(np.abs(yv - exact) <= 2e-2 * np.max(np.abs(exact), axis=1, keepdims=True))
    assert np.linalg.norm(yv - exact) / np.linalg.norm(exact) <= 5e-3


@pytest.mark.gpu
def test_device_replay_on_fixture(native_lib):
    from dflash_mlx_amd.kernels import replay_launch
    from dflash_mlx_amd.recurrent_rollback_cache import conv_state_rebuild

    f = np.load(os.path.join(HERE, "replay_s3_t16.npz"))
    dev = "cuda:0"
    state = torch.from_numpy(f["state"]).to(dev)
    out = torch.empty_like(state)
    steps = torch.from_numpy(f["steps"]).to(dev)
    replay_launch(_bf16_tensor(f["tape"]).to(dev), _bf16_tensor(f["k"]).to(dev), torch.from_numpy(f["g"]).to(dev),
                  state, out, steps=steps, T_alloc=16, slots=3)
    got = out.cpu().numpy().astype(np.float64)
    want = f["state_out"].astype(np.float64)
    assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 1e-5
    conv = conv_state_rebuild(_bf16_tensor(f["conv"]).to(dev), _bf16_tensor(f["qkv"]).to(dev), steps, 3)
    assert np.array_equal(conv.cpu().view(torch.int16).numpy().view(np.uint16), f["conv_out"])
