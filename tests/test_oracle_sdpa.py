"""Pins of the oracle's 16-query attention (dflash_mlx/kernels.py:442-761): torch's own
scaled_dot_product_attention under the block's causal rule, the reference's two kernels
restated loop by loop, and closed forms."""
import numpy as np
import pytest
import torch

from dflash_mlx_amd.kernels import batched_sdpa_2pass_exact
from oracle import dflash_oracle as O


def _qkv(B, Hq, Hk, N, D, seed):
    rng = np.random.default_rng(0xDF1A + seed)
    return (rng.standard_normal((B, Hq, 16, D)), rng.standard_normal((B, Hk, N, D)),
            rng.standard_normal((B, Hk, N, D)))


@pytest.mark.parametrize("B,Hq,Hk,N,D", [(1, 2, 1, 40, 16), (2, 4, 2, 16, 8), (1, 6, 1, 75, 32)])
@pytest.mark.parametrize("masked", ["none", "bool", "additive"])
def test_exact_is_torch_sdpa_under_the_block_causal_rule(B, Hq, Hk, N, D, masked):
    q, k, v = _qkv(B, Hq, Hk, N, D, N)
    G = Hq // Hk
    allow = np.arange(N)[None, :] <= (N - 16 + np.arange(16))[:, None]
    allow = np.broadcast_to(allow, (B, Hq, 16, N)).copy()
    mask, add = None, np.zeros((B, Hq, 16, N))
    rng = np.random.default_rng(N)
    if masked == "bool":
        keep = rng.random((B, Hq, 16, N)) > 0.2
        keep[..., 0] = True                         # never a row without keys in this test
        mask = np.where(keep, 0.0, O._lowest("bf16"))
        allow &= keep
    if masked == "additive":
        mask = O.round_bf16(rng.standard_normal((B, Hq, 16, N)).astype(np.float32)).astype(np.float64)
        add = mask
    got = O.sdpa_q16_exact(q, k, v, D ** -0.5, mask)
    bias = torch.from_numpy(np.where(allow, add, -np.inf))
    want = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q), torch.from_numpy(np.repeat(k, G, 1)), torch.from_numpy(np.repeat(v, G, 1)),
        attn_mask=bias, scale=D ** -0.5).numpy()
    np.testing.assert_allclose(got, want, rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("blocks", [1, 4, 32])
def test_two_pass_restatement_is_the_same_attention(blocks):
    q, k, v = _qkv(1, 2, 1, 45, 16, blocks)
    q, k, v = (O.round_bf16(t.astype(np.float32)) for t in (q, k, v))
    mask = np.zeros((1, 2, 16, 45), np.float32)
    mask[0, 1, :, 5:9] = O._lowest("bf16")
    for m in (None, mask):
        exact = O.sdpa_q16_exact(q, k, v, 0.25, m)
        two = O.sdpa_q16_two_pass(q, k, v, 0.25, blocks, m)
        # partial outputs are rounded to bf16 before the merge: a few 2^-9 of the largest value
        assert np.abs(two - exact).max() <= 3 * 2.0 ** -9 * np.abs(v).max()


def test_closed_forms():
    q, k, v = _qkv(1, 1, 1, 16, 8, 3)
    out = O.sdpa_q16_exact(q, k, v, 1.0)
    np.testing.assert_allclose(out[0, 0, 0], v[0, 0, 0], rtol=1e-12)          # query 0 sees key 0 only
    out = O.sdpa_q16_exact(np.zeros_like(q), k, v, 1.0)                           # equal scores: a mean
    for i in range(16):
        np.testing.assert_allclose(out[0, 0, i], v[0, 0, :i + 1].mean(axis=0), rtol=1e-12)
    mask = np.zeros((1, 1, 16, 16))
    mask[0, 0, 3, :] = O._lowest("bf16") * 2                                      # below the lowest finite value
    out = O.sdpa_q16_exact(q, k, v, 1.0, mask)
    assert np.all(out[0, 0, 3] == 0) and np.all(np.isfinite(out))
    # softmax shift invariance: a constant added to one query's mask row changes nothing
    shift = np.zeros((1, 1, 16, 16))
    shift[0, 0, 5, :] = 7.0
    np.testing.assert_allclose(O.sdpa_q16_exact(q, k, v, 1.0, shift), O.sdpa_q16_exact(q, k, v, 1.0), rtol=1e-10)


def test_host_tensors_and_uncovered_shapes_return_none():
    q = torch.zeros(1, 4, 16, 128, dtype=torch.bfloat16)
    kv = torch.zeros(1, 2, 64, 128, dtype=torch.bfloat16)
    assert batched_sdpa_2pass_exact(q, kv, kv, 1.0) is None                       # host tensors
    assert batched_sdpa_2pass_exact(q[0], kv, kv, 1.0) is None
