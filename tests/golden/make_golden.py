"""Writes the small regression fixtures under tests/golden/ from the CPU oracle.

The reference tree holds no golden vectors for this path (its two test files draw
their data at run time), and its implementation cannot be imported here (it needs the
third-party mlx package).  These fixtures are therefore SELF-GENERATED: inputs drawn
from fixed seeds and expected outputs computed by oracle/dflash_oracle.py, whose
functions are pinned by tests/test_oracle_*.py.  They guard against regressions of the
oracle and give the device tests fixed inputs; they do not claim mlx provenance.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import dflash_oracle as O  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def qmm_fixture(seed, K, N, gs):
    rng = np.random.default_rng(seed)
    x = O.f32_to_bf16(rng.standard_normal((16, K)).astype(np.float32))
    w = rng.integers(0, 2 ** 32, size=(N, K // 8), dtype=np.uint64).astype(np.uint32)
    s = O.f32_to_bf16((np.abs(rng.standard_normal((N, K // gs))) * 0.02 + 1e-4).astype(np.float32))
    b = O.f32_to_bf16((-8.0 * O.bf16_to_f32(s) + rng.standard_normal((N, K // gs)).astype(np.float32) * 1e-3))
    xf, sf, bf = O.bf16_to_f32(x), O.bf16_to_f32(s), O.bf16_to_f32(b)
    return dict(x=x, w=w, scales=s, biases=b, group_size=np.int32(gs),
                y_exact=O.qmm_exact(xf, w, sf, bf, gs),
                y_kernel_bf16=O.f32_to_bf16(O.qmm_kernel_semantics(xf, w, sf, bf, gs)))


def replay_fixture(seed, S=3, T=16, Hk=1, Hv=1, Dk=128, Dv=128):
    rng = np.random.default_rng(seed)
    tape = O.f32_to_bf16((rng.standard_normal((S, T, Hv, Dv)) * 0.05).astype(np.float32))
    k = rng.standard_normal((S, T, Hk, Dk)).astype(np.float32)
    k = O.f32_to_bf16(k / np.linalg.norm(k, axis=-1, keepdims=True))
    g = np.exp(-np.log1p(np.exp(rng.standard_normal((S, T, Hv))))).astype(np.float32)
    state = (rng.standard_normal((S, Hv, Dv, Dk)) * 0.1).astype(np.float32)
    steps = np.array([0, 7, 16], dtype=np.int32)[:S]
    out = np.empty_like(state, dtype=np.float64)
    for s in range(S):
        a = int(steps[s])
        out[s] = O.tape_replay_ops(O.bf16_to_f32(tape[s:s + 1, :a]), O.bf16_to_f32(k[s:s + 1, :a]),
                                   g[s:s + 1, :a], state[s:s + 1])[0]
    qkv = O.f32_to_bf16(rng.standard_normal((S, T, 24)).astype(np.float32))
    conv = O.f32_to_bf16(rng.standard_normal((S, 3, 24)).astype(np.float32))
    conv_out = np.stack([O.rebuild_conv_state(conv[s:s + 1], qkv[s:s + 1], int(steps[s]), 4)[0] for s in range(S)])
    return dict(tape=tape, k=k, g=g, state=state, steps=steps, state_out=out.astype(np.float32),
                qkv=qkv, conv=conv, conv_out=conv_out)


def main():
    np.savez_compressed(os.path.join(HERE, "qmm_k1024_n64_gs64.npz"), **qmm_fixture(0xDF1A, 1024, 64, 64))
    np.savez_compressed(os.path.join(HERE, "qmm_k256_n32_gs32.npz"), **qmm_fixture(0xDF1B, 256, 32, 32))
    np.savez_compressed(os.path.join(HERE, "replay_s3_t16.npz"), **replay_fixture(0xDF1C))
    print("wrote fixtures to", HERE)


if __name__ == "__main__":
    main()
