"""Parity of the gfx950 GatedDeltaNet glue kernels (dflash_gdn_prepare, dflash_gdn_gated_norm)
against the CPU oracle, and of the layer's speculative call on the device against the same
layer evaluated with array operators on the host.

Bars: the next conv state is a copy - bit-exact; q, k, v, beta and the normed output agree
with the oracle to two steps of the array dtype's grid everywhere and exactly on
at least 97 % of the elements (device exp / log differ from the host's in the last fp32 bit,
which now and then moves a rounding); g (fp32) to 2e-5 relative in its exponent."""
import numpy as np
import pytest
import torch

from dflash_mlx_amd import gdn_layer as G
from dflash_mlx_amd.recurrent_rollback_cache import RecurrentRollbackCache
from oracle import dflash_oracle as O
from test_gdn_layer_glue import _inputs, _layer

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TORCH = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}
ULP = {"bf16": 2.0 ** -7, "fp16": 2.0 ** -10, "fp32": 2.0 ** -22}     # grid spacing relative to |x|, upper bound
TINY = {"bf16": 1e-7, "fp16": 2.0 ** -22, "fp32": 1e-7}     # two steps of the fp16 subnormal grid


def _dev(t, dtype, param_dtype=None):
    out = {}
    for key, val in t.items():
        dt = param_dtype if (param_dtype is not None and key in ("A_log", "dt_bias")) else dtype
        out[key] = None if val is None else torch.from_numpy(val).to(dt).to(DEV)
    return out


def _check(got, want, name):
    np.testing.assert_array_equal(got[0].float().cpu().numpy(), want[0])
    for what, a, b in zip(("q", "k", "v", "g", "beta"), got[1:], want[1:]):
        a = a.float().cpu().numpy()
        assert a.shape == b.shape, what
        if what == "g":
            np.testing.assert_allclose(np.log(a), np.log(b), rtol=2e-5, atol=1e-6)
            continue
        assert np.all(np.abs(a - b) <= 2 * ULP[name] * np.abs(b) + TINY[name]), what
        assert np.mean(a == b) > 0.97 or name == "fp32", what


@pytest.mark.parametrize("name", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("S,with_state,masked", [(16, True, False), (16, False, True), (1, True, False),
                                                 (2, True, True), (3, False, False), (5, True, True)])
def test_prepare_against_the_oracle(native_lib, name, S, with_state, masked):
    t, dims = _inputs(B=2, S=S, Hk=2, Hv=4, Dk=128, Dv=128, seed=40 + S, with_state=with_state, dtype=name)
    mask = None
    if masked:
        mask = np.ones((2, S), bool)
        mask[1, S // 2] = False
    want = O.gdn_prepare(**t, **dims, mask=mask, dtype=name)
    d = _dev(t, TORCH[name])
    got = G.gdn_prepare(d["qkv"], d["conv_state"], d["conv_w"], d["a"], d["b"], d["A_log"], d["dt_bias"],
                        None if mask is None else torch.from_numpy(mask).to(DEV), **dims)
    torch.cuda.synchronize()
    assert got[1].dtype == TORCH[name] and got[4].dtype == torch.float32
    _check(got, want, name)


@pytest.mark.parametrize("dims", [dict(Hk=1, Hv=2, Dk=64, Dv=64), dict(Hk=2, Hv=2, Dk=256, Dv=128),
                                  dict(Hk=16, Hv=32, Dk=128, Dv=128), dict(Hk=2, Hv=4, Dk=128, Dv=192)])
def test_prepare_head_shapes_and_fp32_parameters(native_lib, dims):
    t, dims = _inputs(B=1, S=16, seed=50 + dims["Dk"], **dims)
    want = O.gdn_prepare(**t, **dims, dtype="bf16", bias_dtype="fp32")
    d = _dev(t, torch.bfloat16, param_dtype=torch.float32)
    got = G.gdn_prepare(d["qkv"], d["conv_state"], d["conv_w"].unsqueeze(-1), d["a"], d["b"], d["A_log"],
                        d["dt_bias"], None, **dims)
    torch.cuda.synchronize()
    _check(got, want, "bf16")


@pytest.mark.parametrize("K", [2, 3])
def test_prepare_shorter_conv_kernels(native_lib, K):
    t, dims = _inputs(B=1, S=5, Hk=1, Hv=2, Dk=128, Dv=64, K=K, seed=80 + K)
    want = O.gdn_prepare(**t, **dims, dtype="bf16")
    d = _dev(t, torch.bfloat16)
    got = G.gdn_prepare(d["qkv"], d["conv_state"], d["conv_w"], d["a"], d["b"], d["A_log"], d["dt_bias"], None, **dims)
    torch.cuda.synchronize()
    assert tuple(got[0].shape) == (1, K - 1, 2 * 128 + 2 * 64)
    _check(got, want, "bf16")


def test_prepare_takes_the_array_ops_for_other_head_sizes(native_lib):
    t, dims = _inputs(B=1, S=4, Hk=1, Hv=2, Dk=32, Dv=96, seed=60)
    want = O.gdn_prepare(**t, **dims, dtype="bf16")
    d = _dev(t, torch.bfloat16)
    got = G.gdn_prepare(d["qkv"], d["conv_state"], d["conv_w"], d["a"], d["b"], d["A_log"], d["dt_bias"], None, **dims)
    _check(got, want, "bf16")
    with pytest.raises(ValueError):
        G.gdn_prepare(d["qkv"][..., :-1], d["conv_state"], d["conv_w"], d["a"], d["b"], d["A_log"], d["dt_bias"],
                      None, **dims)


def test_prepare_rejects_bad_shapes_through_the_c_abi(native_lib):
    import dflash_mlx_amd._native as nat
    x = torch.zeros(4096, dtype=torch.bfloat16, device=DEV)
    g = torch.zeros(64, dtype=torch.float32, device=DEV)
    ptr = x.data_ptr()
    args = [ptr] * 7 + [None] + [ptr] * 4 + [g.data_ptr(), ptr]
    rc = native_lib.dflash_gdn_prepare(*args, 1, 1, 1, 1, 96, 64, 4, nat.BF16, nat.BF16, 1e-6, None)
    assert rc != 0 and b"multiples of 64" in native_lib.dflash_last_error()
    rc = native_lib.dflash_gdn_prepare(*args, 1, 1, 1, 1, 64, 64, 1, nat.BF16, nat.BF16, 1e-6, None)
    assert rc != 0
    rc = native_lib.dflash_gdn_gated_norm(ptr, ptr, ptr, ptr, 4, 100, nat.BF16, nat.BF16, 1e-6, None)
    assert rc != 0 and b"multiple of 64" in native_lib.dflash_last_error()
    torch.cuda.synchronize()


@pytest.mark.parametrize("name", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("D", [64, 128, 256])
def test_gated_norm_against_the_oracle(native_lib, name, D):
    rng = np.random.default_rng(70 + D)
    r = lambda x: O.round_to(np.asarray(x, np.float32), name)
    x, z, w = r(rng.standard_normal((3, 16, 4, D)) * 3), r(rng.standard_normal((3, 16, 4, D))), r(1 + 0.1 * rng.standard_normal(D))
    want = O.gdn_gated_norm(x, z, w, name)
    got = G.gated_norm(*(torch.from_numpy(v).to(TORCH[name]).to(DEV) for v in (x, z, w)))
    torch.cuda.synchronize()
    a = got.float().cpu().numpy()
    assert np.all(np.abs(a - want) <= 2 * ULP[name] * np.abs(want) + TINY[name])
    assert np.mean(a == want) > 0.97 or name == "fp32"


def test_speculative_layer_call_on_the_device_matches_the_host(native_lib, monkeypatch):
    """The same layer, the same tokens: device kernels (projections through the verify qmm,
    fused glue, block recurrence) against the array operators on the host, then a rollback."""
    monkeypatch.setenv("DFLASH_VERIFY_QMM", "1")
    host = _layer(seed=8, hidden=512, Hk=2, Hv=4, D=128, dtype=torch.bfloat16, quantized=True)
    G._install_exact_small_proj_hooks(host)
    G._install_speculative_linear_cache_hook(host)
    import copy
    dev = copy.deepcopy(host).to(DEV)
    gen = torch.Generator().manual_seed(9)
    prompt = torch.randn((1, 7, 512), generator=gen).to(torch.bfloat16)
    block = torch.randn((1, 16, 512), generator=gen).to(torch.bfloat16)

    outs, caches = [], []
    for layer, to in ((host, lambda t: t), (dev, lambda t: t.to(DEV))):
        cache = RecurrentRollbackCache()
        layer(to(prompt), cache=cache)
        cache[1] = cache[1].float()                 # the serving configuration keeps S in fp32
        cache.arm_rollback(prefix_len=7)
        y = layer(to(block), cache=cache)
        tape = cache._tape.float().cpu()
        cache.rollback(9)
        outs.append((y.float().cpu(), tape))
        caches.append((cache[0].float().cpu(), cache[1].float().cpu()))
    torch.cuda.synchronize()
    rel = lambda a, b: float((a - b).norm() / b.norm())
    assert rel(outs[1][0], outs[0][0]) < 2e-2       # bf16 activations through five matmuls
    assert rel(outs[1][1], outs[0][1]) < 2e-2
    assert rel(caches[1][1], caches[0][1]) < 2e-2
    assert rel(caches[1][0], caches[0][0]) < 1e-2


def test_layer_hook_with_an_arena_cache_matches_the_per_layer_cache(native_lib, monkeypatch):
    """The documented set-up - RollbackArena with its defaults, the layer's speculative hook
    recording its fp32 tape into it, rollback_all - against a plain RecurrentRollbackCache."""
    import copy

    from dflash_mlx_amd.recurrent_rollback_cache import RollbackArena

    monkeypatch.setenv("DFLASH_VERIFY_QMM", "1")
    host = _layer(seed=18, hidden=512, Hk=2, Hv=4, D=128, dtype=torch.bfloat16, quantized=True)
    G._install_exact_small_proj_hooks(host)
    G._install_speculative_linear_cache_hook(host)
    layer = copy.deepcopy(host).to(DEV)
    gen = torch.Generator().manual_seed(19)
    prompt = torch.randn((1, 7, 512), generator=gen).to(torch.bfloat16).to(DEV)
    block = torch.randn((1, 16, 512), generator=gen).to(torch.bfloat16).to(DEV)
    conv_dim = 2 * 2 * 128 + 4 * 128

    plain = RecurrentRollbackCache()
    layer(prompt, cache=plain)
    plain[1] = plain[1].float()
    conv0, state0 = plain[0].clone(), plain[1].clone()
    plain.arm_rollback(prefix_len=7)
    y_plain = layer(block, cache=plain)
    plain.rollback(9)

    arena = RollbackArena(1, Hk=2, Hv=4, Dk=128, Dv=128, conv_dim=conv_dim, device=DEV)
    cache = arena.caches()[0]
    cache[0].copy_(conv0); cache[1].copy_(state0)
    arena.arm_all(prefix_len=7)
    y_arena = layer(block, cache=cache)
    assert cache._tape.dtype == torch.float32
    arena.rollback_all(torch.tensor(9, dtype=torch.int32, device=DEV))
    torch.cuda.synchronize()
    assert torch.equal(y_arena, y_plain)
    assert torch.equal(cache[1], plain[1]) and torch.equal(cache[0], plain[0])
