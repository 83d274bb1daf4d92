"""The GatedDeltaNet layer glue (dflash_mlx/runtime.py:243-285, 344-455) on the host: the
oracle's restatement pinned by independent routes, the array-op mirror against the oracle,
and the layer hooks (pad to 16, speculative call with an armed rollback cache).

The operators belong to mlx / mlx-lm, which are not available: what is pinned here is their
mathematics (torch's conv1d, fp64 closed forms, the conv-state rule of the rollback cache, a
token-by-token evaluation of the same layer); where single bf16 roundings are placed inside
the sequence is the restatement's choice and is only checked for self-consistency."""
import numpy as np
import pytest
import torch

from dflash_mlx_amd import gdn_layer as G
from dflash_mlx_amd.quantized import QuantizedLinear
from dflash_mlx_amd.recurrent_rollback_cache import RecurrentRollbackCache
from oracle import dflash_oracle as O


def _inputs(B=2, S=5, Hk=2, Hv=4, Dk=64, Dv=64, K=4, seed=0, with_state=True, dtype="bf16"):
    rng = np.random.default_rng(0xDF1A + seed)
    C = 2 * Hk * Dk + Hv * Dv
    r = lambda x: O.round_to(np.asarray(x, np.float32), dtype)
    return dict(
        qkv=r(rng.standard_normal((B, S, C))), conv_state=r(rng.standard_normal((B, K - 1, C))) if with_state else None,
        conv_w=r(rng.standard_normal((C, K)) * 0.4), a=r(rng.standard_normal((B, S, Hv))),
        b=r(rng.standard_normal((B, S, Hv))), A_log=r(np.log(rng.uniform(0.5, 8.0, Hv))),
        dt_bias=r(rng.standard_normal(Hv) * 0.5 + 1.0)), dict(Hk=Hk, Hv=Hv, Dk=Dk, Dv=Dv)


def _silu64(x):
    x = np.asarray(x, np.float64)
    return x / (1.0 + np.exp(-x))


def test_oracle_conv_is_torch_conv1d_and_the_rest_is_closed_form():
    t, dims = _inputs(seed=1, dtype="fp32")
    conv_next, q, k, v, g, beta = O.gdn_prepare(**t, **dims, dtype="fp32")
    B, S, C = t["qkv"].shape
    x = torch.from_numpy(np.concatenate([t["conv_state"], t["qkv"]], axis=1)).double()
    w = torch.from_numpy(t["conv_w"]).double()
    conv = torch.nn.functional.conv1d(x.transpose(1, 2), w.unsqueeze(1), groups=C).transpose(1, 2).numpy()
    assert conv.shape == (B, S, C)
    act = _silu64(conv)
    kd = dims["Hk"] * dims["Dk"]
    q64 = act[..., :kd].reshape(B, S, dims["Hk"], dims["Dk"])
    k64 = act[..., kd:2 * kd].reshape(B, S, dims["Hk"], dims["Dk"])
    norm = lambda x: x / np.sqrt((x * x).mean(-1, keepdims=True) + 1e-6)
    np.testing.assert_allclose(q, norm(q64) / dims["Dk"], rtol=2e-5, atol=1e-7)
    np.testing.assert_allclose(k, norm(k64) / np.sqrt(dims["Dk"]), rtol=2e-5, atol=1e-7)
    np.testing.assert_allclose(v.reshape(B, S, -1), act[..., 2 * kd:], rtol=2e-5, atol=1e-7)
    sp = np.log1p(np.exp(t["a"].astype(np.float64) + t["dt_bias"].astype(np.float64)))
    np.testing.assert_allclose(g, np.exp(-np.exp(t["A_log"].astype(np.float64)) * sp), rtol=2e-5)
    np.testing.assert_allclose(beta, 1.0 / (1.0 + np.exp(-t["b"].astype(np.float64))), rtol=2e-6)
    assert np.all((g > 0) & (g < 1))
    # unit rms before the scale
    np.testing.assert_allclose(((q * dims["Dk"]) ** 2).mean(-1), 1.0, rtol=1e-3)


@pytest.mark.parametrize("S", [1, 2, 3, 7])
@pytest.mark.parametrize("with_state", [True, False])
def test_oracle_conv_state_hand_over_is_the_rollback_rule(S, with_state):
    """The conv state a call leaves behind is what the rollback cache rebuilds when every step
    of the block is accepted (recurrent_rollback_cache.py:129-146 with steps = S)."""
    t, dims = _inputs(S=S, seed=2 + S, with_state=with_state)
    mask = np.ones((2, S), bool)
    mask[1, S // 2] = False
    conv_next = O.gdn_prepare(**t, **dims, mask=mask)[0]
    masked = np.where(mask[..., None], t["qkv"], np.float32(0))
    np.testing.assert_array_equal(conv_next, O.rebuild_conv_state(t["conv_state"], masked, S))


def test_oracle_bf16_results_sit_within_two_roundings_of_the_exact_values():
    t, dims = _inputs(seed=3)
    lo = O.gdn_prepare(**t, **dims, dtype="bf16")
    hi = O.gdn_prepare(**t, **dims, dtype="fp32")
    for name, a, b in zip(("q", "k", "v", "beta"), lo[1:4] + lo[5:], hi[1:4] + hi[5:]):
        assert np.all(np.abs(a - b) <= 3 * 2.0 ** -8 * np.abs(b) + 1e-6), name
    # a + dt_bias and the softplus are rounded to bf16: two roundings of the exponent of g
    np.testing.assert_allclose(np.log(lo[4]), np.log(hi[4]), rtol=3 * 2.0 ** -8)


def test_oracle_gated_norm_closed_form():
    rng = np.random.default_rng(5)
    x, z = rng.standard_normal((2, 6, 128)).astype(np.float32), rng.standard_normal((2, 6, 128)).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(128)).astype(np.float32)
    want = _silu64(z) * x / np.sqrt((x.astype(np.float64) ** 2).mean(-1, keepdims=True) + 1e-6) * w
    np.testing.assert_allclose(O.gdn_gated_norm(x, z, w, "fp32"), want, rtol=2e-5, atol=1e-6)
    got = O.gdn_gated_norm(O.round_bf16(x), O.round_bf16(z), O.round_bf16(w), "bf16")
    assert np.all(O.round_bf16(got) == got)


def _as_torch(t, dtype):
    return {k: None if v is None else torch.from_numpy(v).to(dtype) for k, v in t.items()}


@pytest.mark.parametrize("dtype,name", [(torch.bfloat16, "bf16"), (torch.float32, "fp32")])
def test_array_op_mirror_matches_the_oracle(dtype, name):
    t, dims = _inputs(B=2, S=6, seed=7, dtype=name)
    mask = np.ones((2, 6), bool)
    mask[0, 2] = False
    want = O.gdn_prepare(**t, **dims, mask=mask, dtype=name)
    tt = _as_torch(t, dtype)
    got = G.gdn_prepare_ops(tt["qkv"], tt["conv_state"], tt["conv_w"], tt["a"], tt["b"], tt["A_log"], tt["dt_bias"],
                            torch.from_numpy(mask), **dims)
    ulp = {"bf16": 2.0 ** -8, "fp32": 2.0 ** -22}[name]
    np.testing.assert_array_equal(got[0].float().numpy(), want[0])
    for what, a, b in zip(("q", "k", "v", "g", "beta"), got[1:], want[1:]):
        a = a.float().numpy()
        if what == "g":                             # fp32 whatever the array dtype
            np.testing.assert_allclose(a, b, rtol=1e-5)
            continue
        assert np.all(np.abs(a - b) <= 2 * ulp * np.abs(b) + 1e-7), what
        assert np.mean(a == b) > 0.98 or name == "fp32", what


class _Spy(torch.nn.Module):
    def __init__(self, inner):
        super().__init__()
        self.inner, self.seen = inner, []

    def forward(self, x):
        self.seen.append(tuple(x.shape))
        return self.inner(x)


def test_exact_small_proj_pad_pads_short_blocks_to_sixteen():
    lin = _Spy(torch.nn.Linear(32, 8, bias=True))
    pad = G._ExactSmallProjPad(lin)
    x = torch.randn(2, 3, 32)
    y = pad(x)
    assert lin.seen == [(2, 16, 32)] and y.shape == (2, 3, 8)
    torch.testing.assert_close(y, lin.inner(x))
    pad(torch.randn(2, 16, 32)), pad(torch.randn(2, 20, 32)), pad(torch.randn(5, 32))
    assert lin.seen[1:] == [(2, 16, 32), (2, 20, 32), (5, 32)]
    assert pad.weight is lin.inner.weight if hasattr(lin, "weight") else True


def _layer(seed=0, hidden=128, Hk=2, Hv=4, D=64, dtype=torch.float32, quantized=False):
    g = torch.Generator().manual_seed(0xDF1A + seed)
    C = 2 * Hk * D + Hv * D

    def lin(n_in, n_out):
        m = torch.nn.Linear(n_in, n_out, bias=False, dtype=torch.float32)
        m.weight.data = torch.randn((n_out, n_in), generator=g) * n_in ** -0.5
        if quantized:
            return QuantizedLinear.from_linear(m.to(dtype))
        return m.to(dtype)

    layer = G.GatedDeltaNet(hidden, num_k_heads=Hk, num_v_heads=Hv, head_k_dim=D, head_v_dim=D,
                            in_proj_qkv=lin(hidden, C), in_proj_z=lin(hidden, Hv * D), in_proj_b=lin(hidden, Hv),
                            in_proj_a=lin(hidden, Hv), out_proj=lin(Hv * D, hidden), dtype=dtype)
    layer.conv1d.weight.data = (torch.randn((C, 4, 1), generator=g) * 0.4).to(dtype)
    layer.A_log.data = torch.log(torch.rand(Hv, generator=g) * 4 + 0.5).to(dtype)
    layer.dt_bias.data = (torch.randn(Hv, generator=g) * 0.3 + 0.5).to(dtype)
    layer.norm.weight.data = (1 + 0.1 * torch.randn(D, generator=g)).to(dtype)
    return layer


def test_hooks_are_installed_once_and_leave_unarmed_calls_alone():
    layer = _layer(seed=1)
    original = type(layer).forward if not getattr(type(layer), "_dflash_speculative_call_installed", False) \
        else type(layer)._dflash_original_call
    G._install_exact_small_proj_hooks(layer)
    G._install_exact_small_proj_hooks(layer)
    assert isinstance(layer.in_proj_b, G._ExactSmallProjPad) and not isinstance(layer.in_proj_b.linear, G._ExactSmallProjPad)
    G._install_speculative_linear_cache_hook(layer)
    patched = type(layer).forward
    G._install_speculative_linear_cache_hook(layer)
    assert type(layer).forward is patched and type(layer)._dflash_original_call is original
    x = torch.randn(1, 4, 128)
    cache = RecurrentRollbackCache()
    y = layer(x, cache=cache)                      # not armed: the original call, no tape
    assert cache._tape is None and cache[1] is not None and y.shape == x.shape


def test_speculative_block_equals_token_by_token_and_rolls_back_to_the_prefix():
    """One 16-token call with an armed cache gives what 16 single-token plain calls give; after
    rollback(n) the cache equals the one that saw only the first n + 1 tokens."""
    torch.manual_seed(3)
    layer = _layer(seed=2)
    G._install_exact_small_proj_hooks(layer)
    G._install_speculative_linear_cache_hook(layer)
    prompt, block = torch.randn(1, 5, 128), torch.randn(1, 16, 128)

    spec = RecurrentRollbackCache()
    layer(prompt, cache=spec)
    spec.arm_rollback(prefix_len=5)
    y_block = layer(block, cache=spec)
    assert spec._tape is not None and tuple(spec._tape.shape) == (1, 16, 4, 64)

    plain = RecurrentRollbackCache()
    layer(prompt, cache=plain)
    ys, states = [], []
    for t in range(16):
        ys.append(layer(block[:, t:t + 1], cache=plain))
        states.append((plain[0].clone(), plain[1].clone()))
    torch.testing.assert_close(y_block, torch.cat(ys, dim=1), rtol=2e-4, atol=2e-5)
    torch.testing.assert_close(spec[1], states[-1][1], rtol=2e-4, atol=2e-5)
    torch.testing.assert_close(spec[0], states[-1][0], rtol=2e-4, atol=2e-5)   # 16-row vs 1-row matmuls

    spec.rollback(6)                               # 6 drafts accepted: 7 tokens of the block stay
    torch.testing.assert_close(spec[1], states[6][1], rtol=2e-4, atol=2e-5)
    torch.testing.assert_close(spec[0], states[6][0], rtol=2e-4, atol=2e-5)
    assert not spec._armed and spec._tape is None


def test_speculative_call_with_quantized_projections_and_mask():
    layer = _layer(seed=4, dtype=torch.bfloat16, quantized=True)
    G._install_exact_small_proj_hooks(layer)
    G._install_speculative_linear_cache_hook(layer)
    x = torch.randn(2, 16, 128).to(torch.bfloat16)
    mask = torch.ones(2, 16, dtype=torch.bool)
    mask[1, :3] = False
    cache = RecurrentRollbackCache()
    cache.arm_rollback()
    y = layer(x, mask=mask, cache=cache)
    # on the host the array-op recurrence promotes through the fp32 gate, as the reference's does
    assert y.shape == x.shape and torch.isfinite(y.float()).all()
    assert torch.all(cache._tape[1, :3] == 0) and torch.all(cache._tape_qkv[1, :3] == 0)
