"""The full-attention layer hook (dflash_mlx/runtime.py:456-652) on the host: off by default,
exact query-by-query attention over long cached prefixes when enabled, and equal to the plain
causal call - the property the hook exists to preserve."""
import torch

from dflash_mlx_amd import attention_layer as A
from dflash_mlx_amd.cache import KVCache


def _attn(dtype=torch.float32, heads=4, kv_heads=2, head_dim=32, hidden=64, seed=0, gated=True):
    g = torch.Generator().manual_seed(0xDF1A + seed)

    def lin(n_in, n_out):
        m = torch.nn.Linear(n_in, n_out, bias=False)
        m.weight.data = torch.randn((n_out, n_in), generator=g) * n_in ** -0.5
        return m.to(dtype)

    q_out = heads * head_dim * (2 if gated else 1)
    attn = A.GatedAttention(num_attention_heads=heads, num_key_value_heads=kv_heads, head_dim=head_dim,
                            q_proj=lin(hidden, q_out), k_proj=lin(hidden, kv_heads * head_dim),
                            v_proj=lin(hidden, kv_heads * head_dim), o_proj=lin(heads * head_dim, hidden), dtype=dtype)
    attn.q_norm.weight.data = (1 + 0.1 * torch.randn(head_dim, generator=g)).to(dtype)
    return attn


class _Layer:
    is_linear = False

    def __init__(self, attn):
        self.self_attn = attn


def test_hook_is_off_until_configured_and_installed_once():
    attn = _attn()
    original = type(attn).forward if not getattr(type(attn), "_dflash_split_full_attention_installed", False) \
        else type(attn)._dflash_original_call
    A._install_split_full_attention_hook(attn)
    patched = type(attn).forward
    A._install_split_full_attention_hook(attn)
    assert type(attn).forward is patched and type(attn)._dflash_original_call is original
    x = torch.randn(1, 5, 64)
    assert torch.equal(attn(x, mask="causal", cache=KVCache()), original(attn, x, mask="causal", cache=KVCache()))
    assert A._attention_has_gated_q_proj(attn) and not A._attention_has_gated_q_proj(_attn(gated=False, seed=1))
    assert A._attention_num_heads(attn) == 4 and A._attention_num_kv_heads(attn) == 2


def test_exact_path_over_a_long_prefix_equals_the_plain_causal_call():
    attn = _attn(seed=2)
    A.configure_full_attention_split([_Layer(attn)], enabled=True)
    attn._dflash_split_sdpa_exact_kv_threshold = 8
    original = type(attn)._dflash_original_call
    prefix, block = torch.randn(1, 20, 64), torch.randn(1, 16, 64)
    outs = []
    for call in (lambda x, c: attn(x, mask="causal", cache=c), lambda x, c: original(attn, x, mask="causal", cache=c)):
        cache = KVCache()
        call(prefix, cache)
        outs.append(call(block, cache))
        assert cache.offset == 36
    torch.testing.assert_close(outs[0], outs[1], rtol=1e-5, atol=1e-6)
    # the same tokens one at a time: what "exact" means
    cache = KVCache()
    original(attn, prefix, mask="causal", cache=cache)
    steps = torch.cat([original(attn, block[:, t:t + 1], mask=None, cache=cache) for t in range(16)], dim=1)
    torch.testing.assert_close(outs[0], steps, rtol=1e-5, atol=1e-6)


def test_array_masks_are_cut_per_query_chunk():
    attn = _attn(seed=3)
    A.configure_full_attention_split([_Layer(attn)], enabled=True)
    attn._dflash_split_sdpa_exact_kv_threshold = 4
    original = type(attn)._dflash_original_call
    prefix, block = torch.randn(1, 10, 64), torch.randn(1, 16, 64)
    allow = torch.arange(26)[None, :] <= (10 + torch.arange(16))[:, None]
    allow[:, 3] = False
    outs = []
    for call in (lambda x, m, c: attn(x, mask=m, cache=c), lambda x, m, c: original(attn, x, mask=m, cache=c)):
        cache = KVCache()
        call(prefix, "causal", cache)
        outs.append(call(block, allow, cache))
    torch.testing.assert_close(outs[0], outs[1], rtol=1e-5, atol=1e-6)
