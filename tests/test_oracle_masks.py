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
