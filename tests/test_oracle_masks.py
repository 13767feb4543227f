"""Pins of the oracle's score modifiers (soft-capping, local window, ALiBi) against library
routines: SDPA with an additive bias, and plain torch ops for the tanh cap."""
import pytest
import torch
import torch.nn.functional as F

from flash_attention_factory_amd import workloads as W
from _torch_ref import call_oracle, dense_kv


def _reference(w, alibi=None, softcap=0.0, window_left=-1):
    S, H, D = w.query.shape
    G = H // w.num_kv_heads
    k = (dense_kv(w, w.key_cache) * w.fp8_scale).repeat_interleave(G, dim=2).permute(0, 2, 1, 3)  # [S,H,T,D]
    v = (dense_kv(w, w.value_cache) * w.fp8_scale).repeat_interleave(G, dim=2).permute(0, 2, 1, 3)
    T = k.shape[2]
    q = w.query.float().unsqueeze(2)
    pos = torch.arange(T)[None, :]
    n = w.context_lens[:, None].long()
    bias = torch.zeros(S, H, 1, T)
    dead = pos >= n
    if window_left >= 0:
        dead = dead | (pos < n - 1 - window_left)
    bias.masked_fill_(dead[:, None, None, :], float("-inf"))
    if alibi is not None:
        bias = bias - alibi.view(1, H, 1, 1) * (n - 1 - pos).clamp(min=0)[:, None, None, :].float()
    if softcap > 0:   # SDPA has no cap: softmax(cap * tanh(qk / cap) + bias) v with torch ops
        s = torch.einsum("shqd,shtd->shqt", q * w.scale, k)
        s = softcap * torch.tanh(s / softcap) + bias
        if w.sinks is not None:
            s = torch.cat([s, w.sinks.float().view(1, H, 1, 1).expand(S, H, 1, 1)], dim=3)
            v = torch.cat([v, torch.zeros(S, H, 1, D)], dim=2)
        return torch.einsum("shqt,shtd->shqd", torch.softmax(s, dim=-1), v).squeeze(2)
    if w.sinks is not None:
        k = torch.cat([k, torch.zeros(S, H, 1, D)], dim=2)
        v = torch.cat([v, torch.zeros(S, H, 1, D)], dim=2)
        bias = torch.cat([bias, w.sinks.float().view(1, H, 1, 1).expand(S, H, 1, 1)], dim=3)
    return F.scaled_dot_product_attention(q, k, v, attn_mask=bias, scale=w.scale).squeeze(2)


CASES = [
    dict(window_left=100),
    dict(window_left=0),
    dict(alibi=True),
    dict(softcap=5.0),
    dict(softcap=0.7, alibi=True, window_left=64),
    dict(alibi=True, window_left=5000),   # wider than any context: no effect
]


@pytest.mark.parametrize("mk", CASES)
@pytest.mark.parametrize("sinks", [False, True])
@pytest.mark.parametrize("fp8", [False, True])
def test_masked_attention_ref_matches_torch(oracle, mk, sinks, fp8):
    w = W.make_test_shaped(batch_size=3, nheads=6, nheads_k=2, d=64, seqlen_k=300, varlen=True, has_sinks=sinks,
                           fp8=fp8, seed=7)
    w.context_lens[0] = 1
    alibi = torch.rand(6, generator=torch.Generator().manual_seed(1)) * 0.3 if mk.get("alibi") else None
    kw = dict(alibi_slopes=alibi, softcap=mk.get("softcap", 0.0), window_left=mk.get("window_left", -1))
    _, got = call_oracle(oracle.attention_ref, w, want_f32=True, **kw)
    want = _reference(w, alibi, kw["softcap"], kw["window_left"])
    torch.testing.assert_close(got, want, rtol=2e-5, atol=2e-6)
    plain = call_oracle(oracle.attention_ref, w, want_f32=True)[1]
    if mk == dict(alibi=True, window_left=5000):
        assert not torch.equal(got, plain)   # the bias acts although the window does not
    if mk == dict(window_left=0):            # only the last key is visible: out = its value row, sink-weighted
        assert torch.isfinite(got).all()


def _reference_multi(w, query4, alibi=None, window_left=-1):
    """SDPA over [S, H, QL, T] with the causal rule of upstream's reference: the QL query tokens
    are the last QL positions and token j of them sees keys 0 .. n - QL + j."""
    S, QL, H, D = query4.shape
    G = H // w.num_kv_heads
    k = (dense_kv(w, w.key_cache) * w.fp8_scale).repeat_interleave(G, dim=2).permute(0, 2, 1, 3)
    v = (dense_kv(w, w.value_cache) * w.fp8_scale).repeat_interleave(G, dim=2).permute(0, 2, 1, 3)
    T = k.shape[2]
    q = query4.float().permute(0, 2, 1, 3)                                   # [S, H, QL, D]
    pos = torch.arange(T)[None, None, :]
    last = (w.context_lens[:, None].long() - QL + torch.arange(QL)[None, :])[:, :, None]   # [S, QL, 1]
    dead = pos > last
    if window_left >= 0:
        dead = dead | (pos < last - window_left)
    bias = torch.zeros(S, 1, QL, T).masked_fill(dead[:, None], float("-inf")).expand(S, H, QL, T).clone()
    if alibi is not None:
        bias = bias - alibi.view(1, H, 1, 1) * (last - pos).clamp(min=0)[:, None].float()
    if w.sinks is not None:
        k = torch.cat([k, torch.zeros(S, H, 1, D)], dim=2)
        v = torch.cat([v, torch.zeros(S, H, 1, D)], dim=2)
        bias = torch.cat([bias, w.sinks.float().view(1, H, 1, 1).expand(S, H, QL, 1)], dim=3)
    out = F.scaled_dot_product_attention(q, k, v, attn_mask=bias, scale=w.scale)
    return out.permute(0, 2, 1, 3)                                           # [S, QL, H, D]


@pytest.mark.parametrize("QL", [2, 4, 8])
@pytest.mark.parametrize("mods", [dict(), dict(alibi=True, window_left=50)])
@pytest.mark.parametrize("sinks", [False, True])
def test_multi_token_queries_match_sdpa(oracle, QL, mods, sinks):
    w = W.make_test_shaped(batch_size=3, nheads=4, nheads_k=2, d=64, seqlen_k=200, varlen=True, has_sinks=sinks,
                           fp8=False, seed=11)
    w.context_lens[0] = QL          # the query tokens are the whole context
    g = torch.Generator().manual_seed(3)
    query4 = torch.randn(3, QL, 4, 64, generator=g).to(torch.float16)
    alibi = torch.rand(4, generator=g) * 0.2 if mods.get("alibi") else None
    wl = mods.get("window_left", -1)
    got = oracle.attention_ref(query4, w.key_cache, w.value_cache, w.block_tables, w.context_lens, scale=w.scale,
                               block_size=w.block_size, kv_strides=w.kv_strides(), num_kv_heads=w.num_kv_heads,
                               sinks=w.sinks, want_f32=True, alibi_slopes=alibi, window_left=wl)[1]
    want = _reference_multi(w, query4, alibi, wl)
    torch.testing.assert_close(got, want, rtol=2e-5, atol=2e-6)
    # the last query token is plain decode on the same cache
    plain = oracle.attention_ref(query4[:, -1].contiguous(), w.key_cache, w.value_cache, w.block_tables,
                                 w.context_lens, scale=w.scale, block_size=w.block_size, kv_strides=w.kv_strides(),
                                 num_kv_heads=w.num_kv_heads, sinks=w.sinks, want_f32=True, alibi_slopes=alibi,
                                 window_left=wl)[1]
    torch.testing.assert_close(got[:, -1], plain, rtol=1e-6, atol=1e-7)


@pytest.mark.parametrize("sinks", [False, True])
def test_query_tokens_before_the_first_key_see_nothing(oracle, sinks):
    """A context shorter than the query block: the leading query tokens lie before key 0.  With a
    sink upstream's formula (test_paged.py:107-121) gives them zeros (all weight on the sink, whose
    value row is zero); without one it divides 0 by 0 -- the oracle returns zeros there too, which
    is what attention kernels (SDPA included) store for a row without keys."""
    QL = 4
    w = W.make_test_shaped(batch_size=2, nheads=4, nheads_k=2, d=64, seqlen_k=100, varlen=True, has_sinks=sinks,
                           fp8=False, seed=12)
    w.context_lens[0] = 2            # tokens 0 and 1 see nothing, token 2 key 0, token 3 keys 0..1
    g = torch.Generator().manual_seed(5)
    query4 = torch.randn(2, QL, 4, 64, generator=g).to(torch.float16)
    got = oracle.attention_ref(query4, w.key_cache, w.value_cache, w.block_tables, w.context_lens, scale=w.scale,
                               block_size=w.block_size, kv_strides=w.kv_strides(), num_kv_heads=w.num_kv_heads,
                               sinks=w.sinks, want_f32=True)[1]
    assert (got[0, :2] == 0).all()
    want = _reference_multi(w, query4)
    # this torch's SDPA stores zeros for a row whose keys are all masked, with or without a sink
    torch.testing.assert_close(got, want, rtol=2e-5, atol=2e-6)
    if not sinks:
        # token 2 sees exactly one key: its output is that key's value row
        v0 = dense_kv(w, w.value_cache)[0, 0]                        # [Hk, D]
        torch.testing.assert_close(got[0, 2], v0.repeat_interleave(2, dim=0), rtol=1e-6, atol=1e-7)
