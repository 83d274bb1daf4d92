"""Parity of the gfx950 16-query attention kernel (dflash_sdpa_q16) against the fp64 oracle.

Bar: the kernel keeps scores, softmax state and outputs in fp32 but feeds the probabilities
to the matrix cores in the input dtype, so |out - exact| <= 4 eps (|exact| + max |v| of the
head), eps = 2^-9 for bf16, 2^-12 for fp16 (output rounding included); rows without keys are
exactly 0."""
import numpy as np
import pytest
import torch

import dflash_mlx_amd._native as nat
from dflash_mlx_amd.kernels import batched_sdpa_2pass_exact
from oracle import dflash_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TORCH = {"bf16": torch.bfloat16, "fp16": torch.float16}
EPS = {"bf16": 2.0 ** -9, "fp16": 2.0 ** -12}


def _case(B, Hq, Hk, N, D, seed, name):
    rng = np.random.default_rng(0xDF1A + seed)
    r = lambda x: O.round_to(np.asarray(x, np.float32), name)
    return r(rng.standard_normal((B, Hq, 16, D))), r(rng.standard_normal((B, Hk, N, D))), r(rng.standard_normal((B, Hk, N, D)))


def _check(out, exact, v, name, Hq):
    a = out.float().cpu().numpy().astype(np.float64)
    G = Hq // v.shape[1]
    vmax = np.repeat(np.abs(v).max(axis=(2, 3)), G, axis=1)[:, :, None, None]
    assert np.all(np.isfinite(a))
    assert np.all(np.abs(a - exact) <= 4 * EPS[name] * (np.abs(exact) + vmax))


def _dev(t, name):
    return torch.from_numpy(t).to(TORCH[name]).to(DEV)


@pytest.mark.parametrize("name", ["bf16", "fp16"])
@pytest.mark.parametrize("B,Hq,Hk,N,D", [(1, 4, 1, 300, 128), (2, 8, 2, 1000, 256), (1, 2, 2, 16, 128),
                                         (1, 6, 1, 17, 256), (1, 8, 1, 33, 128), (1, 16, 4, 1025, 256),
                                         (1, 3, 1, 4000, 128), (1, 32, 8, 4112, 256), (1, 5, 1, 289, 128),
                                         (1, 8, 8, 145, 256), (3, 7, 7, 81, 256),
                                         (1, 8, 2, 33000, 128), (1, 4, 1, 70001, 256)])  # long caches: dozens of tiles per key range
def test_against_the_oracle(native_lib, name, B, Hq, Hk, N, D):
    q, k, v = _case(B, Hq, Hk, N, D, N + D, name)
    out = batched_sdpa_2pass_exact(_dev(q, name), _dev(k, name), _dev(v, name), D ** -0.5)
    torch.cuda.synchronize()
    assert out is not None and out.dtype == TORCH[name] and tuple(out.shape) == q.shape
    _check(out, O.sdpa_q16_exact(q, k, v, D ** -0.5, dtype=name), v, name, Hq)


@pytest.mark.parametrize("D,N", [(128, 700), (256, 500)])
@pytest.mark.parametrize("splits", [1, 2, 5, 64])
def test_any_number_of_key_ranges_gives_the_same_attention(native_lib, splits, D, N):
    q, k, v = _case(1, 4, 2, N, D, 77, "bf16")
    assert native_lib.dflash_set_option(nat.OPT_SDPA_SPLITS, splits) == 0
    try:
        out = batched_sdpa_2pass_exact(_dev(q, "bf16"), _dev(k, "bf16"), _dev(v, "bf16"), 0.1)
        torch.cuda.synchronize()
    finally:
        native_lib.dflash_set_option(nat.OPT_SDPA_SPLITS, 0)
    _check(out, O.sdpa_q16_exact(q, k, v, 0.1), v, "bf16", 4)


def test_config2_cache_shape_read_in_place(native_lib):
    """8 key/value heads of 256 over 4096 + 16 positions, queried through the view of a larger
    cache buffer (capacity 4352), 32 query heads."""
    B, Hq, Hk, N, D, cap = 1, 32, 8, 4112, 256, 4352
    q, k, v = _case(B, Hq, Hk, N, D, 5, "bf16")
    kbuf = torch.zeros((B, Hk, cap, D), dtype=torch.bfloat16, device=DEV)
    vbuf = torch.full((B, Hk, cap, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    kbuf[:, :, :N], vbuf[:, :, :N] = _dev(k, "bf16"), _dev(v, "bf16")
    out = batched_sdpa_2pass_exact(_dev(q, "bf16"), kbuf[:, :, :N], vbuf[:, :, :N], D ** -0.5)
    torch.cuda.synchronize()
    _check(out, O.sdpa_q16_exact(q, k, v, D ** -0.5), v, "bf16", Hq)


@pytest.mark.parametrize("kind", ["bool", "additive"])
def test_masks(native_lib, kind):
    B, Hq, Hk, N, D = 2, 4, 2, 200, 128
    q, k, v = _case(B, Hq, Hk, N, D, 9, "bf16")
    rng = np.random.default_rng(3)
    if kind == "bool":
        keep = rng.random((B, 1, 16, N)) > 0.3
        keep[0, 0, 5, :] = False                     # every key carries the lowest finite value: still used
        mask_dev = torch.from_numpy(keep).to(DEV)
        mask = np.broadcast_to(np.where(keep, 0.0, O._lowest("bf16")), (B, Hq, 16, N))
    else:
        mask = O.round_bf16(rng.standard_normal((B, Hq, 16, N)).astype(np.float32))
        mask[1, 2, 7, :] = -np.inf                   # a query without keys: 0
        mask[0, 1, :, 40:90] = -np.inf
        mask_dev = _dev(mask, "bf16")
    out = batched_sdpa_2pass_exact(_dev(q, "bf16"), _dev(k, "bf16"), _dev(v, "bf16"), D ** -0.5, mask=mask_dev)
    torch.cuda.synchronize()
    _check(out, O.sdpa_q16_exact(q, k, v, D ** -0.5, mask), v, "bf16", Hq)
    if kind == "additive":
        assert torch.all(out[1, 2, 7] == 0)


def test_gates_and_errors(native_lib):
    import dflash_mlx_amd._native as nat
    bf = torch.bfloat16
    q = torch.zeros(1, 4, 16, 128, dtype=bf, device=DEV)
    kv = torch.zeros(1, 2, 64, 128, dtype=bf, device=DEV)
    assert batched_sdpa_2pass_exact(q[:, :, :8], kv, kv, 1.0) is None            # q_len != 16
    assert batched_sdpa_2pass_exact(q.float(), kv.float(), kv.float(), 1.0) is None
    assert batched_sdpa_2pass_exact(q[..., :64], kv[..., :64], kv[..., :64], 1.0) is None
    assert batched_sdpa_2pass_exact(torch.zeros(1, 18, 16, 128, dtype=bf, device=DEV), kv, kv, 1.0) is None
    assert batched_sdpa_2pass_exact(q, kv[:, :, :8], kv[:, :, :8], 1.0) is None  # fewer keys than queries
    out = batched_sdpa_2pass_exact(q, kv, kv, 1.0)
    assert out is not None and torch.all(out == 0)
    rc = native_lib.dflash_sdpa_q16(q.data_ptr(), kv.data_ptr(), kv.data_ptr(), None, out.data_ptr(), None, 0,
                                    1, 4, 2, 64, 96, 0, 64 * 96, 96, 0, 64 * 96, 96, 1.0, nat.BF16, None)
    assert rc != 0 and b"head dim" in native_lib.dflash_last_error()
    need = native_lib.dflash_sdpa_q16_workspace_bytes(1, 4, 2, 4096, 128)
    assert need > 0
    rc = native_lib.dflash_sdpa_q16(q.data_ptr(), kv.data_ptr(), kv.data_ptr(), None, out.data_ptr(), None, 0,
                                    1, 4, 2, 4096, 128, 0, 4096 * 128, 128, 0, 4096 * 128, 128, 1.0, nat.BF16, None)
    assert rc == nat.ERR_WORKSPACE if hasattr(nat, "ERR_WORKSPACE") else rc != 0
    torch.cuda.synchronize()


def test_attention_layer_takes_the_kernel_for_a_verify_block_over_a_long_prefix(native_lib, monkeypatch):
    """The layer hook (dflash_mlx/runtime.py:508-616) on the device: 16 new tokens over 1100 cached
    ones go through the kernel and agree with the layer's plain causal call."""
    from dflash_mlx_amd import attention_layer as A
    from dflash_mlx_amd import kernels as K
    from dflash_mlx_amd.cache import KVCache
    from test_attention_layer import _Layer, _attn

    attn = _attn(dtype=torch.bfloat16, heads=8, kv_heads=2, head_dim=128, hidden=256, seed=5).to(DEV)
    A.configure_full_attention_split([_Layer(attn)], enabled=True)
    original = type(attn)._dflash_original_call
    calls = []
    real = K.batched_sdpa_2pass_exact
    monkeypatch.setattr(A, "batched_sdpa_2pass_exact",
                        lambda **kw: calls.append(tuple(kw["keys"].shape)) or real(**kw))
    gen = torch.Generator().manual_seed(1)
    prefix = torch.randn((1, 1100, 256), generator=gen).to(torch.bfloat16).to(DEV)
    block = torch.randn((1, 16, 256), generator=gen).to(torch.bfloat16).to(DEV)
    outs = []
    with torch.no_grad():
        for call in (lambda x, c: attn(x, mask="causal", cache=c), lambda x, c: original(attn, x, mask="causal", cache=c)):
            cache = KVCache()
            call(prefix, cache)
            outs.append(call(block, cache).float())
    torch.cuda.synchronize()
    assert calls == [(1, 2, 1116, 128)]              # the cache view, read in place; the prefill took the plain path
    rel = float((outs[0] - outs[1]).norm() / outs[1].norm())
    assert rel < 1e-2
