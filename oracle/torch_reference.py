"""The upstream tests' PyTorch reference, restated in PyTorch (TEST INFRASTRUCTURE ONLY).

Only ``tests/`` and the ``cpu_baseline`` leg of ``bench.py`` may import this module: it is what
gets timed on the host cores beside the kernels, and a second checker next to the C oracle.  It
never produces a result the package returns.

Two forms of ``attention_ref`` (test_paged.py:40-168, called as at :408-431 with upcast=True):

``attention_ref_padded``  the literal one: K/V gathered from the pool through the block table into
    dense ``[batch, max_len, kv_heads, d]`` tensors (test_paged.py:184-193), repeated over the query
    group (:85-86), fp32 scores of the scaled query against every key (:82-89), positions at or
    beyond a sequence's length set to -inf (:96-97), the explicit max / exp / sum softmax in fp32
    with the sink in the denominator only (:112-123), probabilities times V (:165), cast back (:168).
    Its dense tensors are ``batch x max_len x heads x d`` fp32: fine for the small configurations,
    137 GB for the large-batch serving mix.
``attention_ref_per_sequence``  the same arithmetic one sequence and one kv head at a time, straight
    from the pool: no padded or repeated tensor, so every configuration fits in memory.

FP8 pools are dequantised to the query dtype first, as test_paged_fp8cache.py:80-81 does.
Inputs are CPU tensors; the result is ``[num_seqs, num_heads, head_size]`` in the query dtype.
"""
from __future__ import annotations


import torch

_FP8 = (torch.float8_e5m2, torch.float8_e4m3fn)


def _token_major(cache: torch.Tensor, layout: str) -> torch.Tensor:
    """[blocks, block_size, kv_heads, d] view of a pool stored in either layout."""
    return cache.permute(0, 2, 1, 3) if layout == "head_major" else cache


def _gather(cache: torch.Tensor, index) -> torch.Tensor:
    """cache[index] (FP8 tensors are indexed as bytes: not every build indexes them directly)."""
    if cache.dtype in _FP8:
        return cache.view(torch.uint8)[index].view(cache.dtype)
    return cache[index]


def _softmax_with_sink(scores: torch.Tensor, sinks) -> torch.Tensor:
    """scores [..., heads, keys] fp32, sinks [heads] or None -> probabilities (test_paged.py:112-123)."""
    m = scores.max(dim=-1, keepdim=True).values
    if sinks is None:
        e = torch.exp(scores - m)
        return e / e.sum(dim=-1, keepdim=True)
    sk = sinks.float().view(*([1] * (scores.dim() - 2)), -1, 1)
    m = torch.maximum(sk, m)
    e = torch.exp(scores - m)
    return e / (e.sum(dim=-1, keepdim=True) + torch.exp(sk - m))


def attention_ref_padded(query, key_cache, value_cache, block_tables, context_lens, *, scale, layout,
                         sinks=None, fp8_scale: float = 1.0) -> torch.Tensor:
    S, H, D = query.shape
    kc, vc = _token_major(key_cache, layout), _token_major(value_cache, layout)
    B, Hk = kc.shape[1], kc.shape[2]
    G = H // Hk
    max_len = int(context_lens.max())
    nb = -(-max_len // B)
    idx = block_tables[:, :nb].long().reshape(-1)

    def dense(c):  # [S, max_len, H, D] fp32, gathered, dequantised, repeated over the group
        c = _gather(c, idx).reshape(S, nb * B, Hk, D)[:, :max_len]
        c = c.to(query.dtype) if c.dtype in _FP8 else c
        return (c.float() * fp8_scale).repeat_interleave(G, dim=2)

    k, v = dense(kc), dense(vc)
    scores = torch.einsum("bhd,bshd->bhs", query.float() * scale, k)
    pad = torch.arange(max_len)[None, :] >= context_lens[:, None].long()
    scores.masked_fill_(pad[:, None, :], float("-inf"))
    attention = _softmax_with_sink(scores, sinks)
    return torch.einsum("bhs,bshd->bhd", attention, v).to(query.dtype)


def attention_ref_per_sequence(query, key_cache, value_cache, block_tables, context_lens, *, scale, layout,
                               sinks=None, fp8_scale: float = 1.0) -> torch.Tensor:
    S, H, D = query.shape
    kc, vc = _token_major(key_cache, layout), _token_major(value_cache, layout)
    B, Hk = kc.shape[1], kc.shape[2]
    G = H // Hk
    out = torch.zeros((S, H, D), dtype=query.dtype)
    for s in range(S):
        n = int(context_lens[s])
        if n <= 0:
            continue
        idx = block_tables[s, : -(-n // B)].long()
        q = (query[s].float() * scale).view(Hk, G, D)
        for kh in range(Hk):
            k = _gather(kc, (idx, slice(None), kh)).reshape(-1, D)[:n]
            v = _gather(vc, (idx, slice(None), kh)).reshape(-1, D)[:n]
            if k.dtype in _FP8:
                k, v = k.to(query.dtype), v.to(query.dtype)
            k, v = k.float() * fp8_scale, v.float() * fp8_scale
            scores = q[kh] @ k.T                                   # [G, n]
            sk = None if sinks is None else sinks[kh * G:(kh + 1) * G]
            out[s, kh * G:(kh + 1) * G] = (_softmax_with_sink(scores, sk) @ v).to(query.dtype)
    return out


def run_workload(w, padded: bool = False) -> torch.Tensor:
    fn = attention_ref_padded if padded else attention_ref_per_sequence
    return fn(w.query, w.key_cache, w.value_cache, w.block_tables, w.context_lens, scale=w.scale, layout=w.layout,
              sinks=w.sinks, fp8_scale=w.fp8_scale)


def padded_bytes(w) -> int:
    """Size of the dense fp32 K and V tensors the padded form builds."""
    S, H, D = w.query.shape
    return 2 * S * int(w.context_lens.max()) * H * D * 4
