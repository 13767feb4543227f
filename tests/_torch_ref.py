"""Independent checks for the oracle, built from library routines only.

``sdpa_reference`` gathers each sequence's K/V through its block table into dense
tensors and calls ``torch.nn.functional.scaled_dot_product_attention`` in fp32.
A sink is one extra key whose logit is the sink value (additive bias on a zero
key row) and whose value row is zero -- the identity behind the sink branch of
the upstream reference (test_paged.py:114-119).
"""
import math

import torch
import torch.nn.functional as F


def dense_kv(w, cache):
    """[S, max_ctx, Hk, D] fp32 (dequantised, unscaled) gathered through the block tables."""
    S = w.num_seqs
    B = w.block_size
    max_ctx = int(w.context_lens.max())
    nb = (max_ctx + B - 1) // B
    c = cache.to(w.query.dtype).float() if cache.dtype in (torch.float8_e5m2, torch.float8_e4m3fn) else cache.float()
    if w.layout == "head_major":
        c = c.permute(0, 2, 1, 3)  # -> [NB, B, Hk, D]
    idx = w.block_tables[:, :nb].long()
    g = c[idx.reshape(-1)].reshape(S, nb * B, c.shape[2], c.shape[3])
    return g[:, :max_ctx]


def sdpa_reference(w):
    S, H, D = w.query.shape
    Hk = w.num_kv_heads
    G = H // Hk
    k = dense_kv(w, w.key_cache) * w.fp8_scale
    v = dense_kv(w, w.value_cache) * w.fp8_scale
    max_ctx = k.shape[1]
    k = k.repeat_interleave(G, dim=2).permute(0, 2, 1, 3)  # [S, H, T, D]
    v = v.repeat_interleave(G, dim=2).permute(0, 2, 1, 3)
    q = w.query.float().unsqueeze(2)  # [S, H, 1, D]
    pos = torch.arange(max_ctx)[None, :]
    bias = torch.zeros(S, 1, 1, max_ctx)
    bias.masked_fill_((pos >= w.context_lens[:, None].long())[:, None, None, :], float("-inf"))
    if w.sinks is not None:
        k = torch.cat([k, torch.zeros(S, H, 1, D)], dim=2)
        v = torch.cat([v, torch.zeros(S, H, 1, D)], dim=2)
        bias = torch.cat([bias.expand(S, H, 1, max_ctx), w.sinks.float().view(1, H, 1, 1).expand(S, H, 1, 1)], dim=3)
    out = F.scaled_dot_product_attention(q, k, v, attn_mask=bias, scale=w.scale)
    return out.squeeze(2)  # [S, H, D] fp32


def brute_force(w):
    """float64, plain Python loops; tiny shapes only."""
    S, H, D = w.query.shape
    G = H // w.num_kv_heads
    B = w.block_size
    out = torch.zeros(S, H, D, dtype=torch.float64)

    def row(cache, s, t, kh):
        blk = int(w.block_tables[s, t // B])
        r = cache[blk, kh, t % B] if w.layout == "head_major" else cache[blk, t % B, kh]
        if r.dtype in (torch.float8_e5m2, torch.float8_e4m3fn):
            r = r.to(w.query.dtype)
        return r.double() * w.fp8_scale

    for s in range(S):
        n = int(w.context_lens[s])
        for h in range(H):
            kh = h // G
            q = w.query[s, h].double()
            logits = [sum(float(q[d]) * float(row(w.key_cache, s, t, kh)[d]) for d in range(D)) * w.scale
                      for t in range(n)]
            extra = [float(w.sinks[h])] if w.sinks is not None else []
            m = max(logits + extra)
            es = [math.exp(x - m) for x in logits]
            den = sum(es) + sum(math.exp(x - m) for x in extra)
            for t in range(n):
                out[s, h] += (es[t] / den) * row(w.value_cache, s, t, kh)
    return out


def call_oracle(fn, w, **kw):
    return fn(w.query, w.key_cache, w.value_cache, w.block_tables, w.context_lens, scale=w.scale,
              block_size=w.block_size, kv_strides=w.kv_strides(), num_kv_heads=w.num_kv_heads,
              sinks=w.sinks, fp8_scale=w.fp8_scale, **kw)


def assert_close_to_reference(got, ref, what="", atol=1e-2, rtol=1e-2):
    """The benchmark contract's gate (atol = rtol = 1e-2 on the outputs as they are) AND the same gate
    on outputs brought to unit magnitude, sequence by sequence.  With a large sink logit or a narrow
    window |out| is 1e-3 .. 1e-1 and the absolute gate alone would pass almost anything; normalised by
    each sequence's max |ref| a kernel that ignored a mask or a modifier fails.  Rows of all-zero
    reference (query tokens that see no key) must be zero."""
    got = got.float().cpu()
    ref = ref.float()
    assert torch.isfinite(got).all(), what
    torch.testing.assert_close(got, ref, atol=atol, rtol=rtol, msg=lambda m: f"{what}: {m}")
    flat_ref = ref.reshape(ref.shape[0], -1)
    unit = flat_ref.abs().amax(dim=1)
    dead = unit == 0
    assert (got.reshape(got.shape[0], -1)[dead] == 0).all(), f"{what}: rows with an all-zero reference"
    unit = torch.where(dead, torch.ones_like(unit), unit).view(-1, *([1] * (ref.dim() - 1)))
    torch.testing.assert_close(got / unit, ref / unit, atol=atol, rtol=rtol, msg=lambda m: f"{what} (normalised): {m}")


def out_pt_reference(w):
    """Upstream's second evaluation of its reference, `out_pt` (test_paged.py:432-447: upcast=False,
    reorder_ops=True): the same maths without the fp32 upcast -- K scaled by 1/sqrt(d) and rounded,
    scores rounded to the 16-bit type, the softmax in fp32 (:112-123), the probabilities rounded,
    P.V rounded.  Its distance from the upcast reference is upstream's yardstick for a kernel's error
    (:603-604).  The 16-bit matrix products are modelled as fp32 accumulation with one rounding of
    each output, which is what a GPU GEMM does; upstream evaluates them on an XPU whose summation
    order nobody can reproduce.  FP8 caches are dequantised first (test_paged_fp8cache.py:80-81).
    Returns [S, H, D] in the query dtype."""
    qd = w.query.dtype
    S, H, D = w.query.shape
    G = H // w.num_kv_heads
    k_all, v_all = dense_kv(w, w.key_cache), dense_kv(w, w.value_cache)  # fp32 images of the 16-bit values
    out = torch.zeros((S, H, D), dtype=qd)
    for s in range(S):
        n = int(w.context_lens[s])
        if n <= 0:
            continue
        k = (k_all[s, :n] * w.fp8_scale).to(qd).repeat_interleave(G, dim=1)   # [n, H, D]
        v = (v_all[s, :n] * w.fp8_scale).to(qd).repeat_interleave(G, dim=1)
        k = (k / math.sqrt(D)).to(qd)                                          # reorder_ops: K is scaled, in 16 bits
        scores = torch.einsum("hd,nhd->hn", w.query[s].float(), k.float()).to(qd).float()
        m = scores.max(dim=-1, keepdim=True).values
        if w.sinks is not None:
            sk = w.sinks.float().view(H, 1)
            m = torch.maximum(m, sk)
            e = torch.exp(scores - m)
            p = e / (e.sum(dim=-1, keepdim=True) + torch.exp(sk - m))
        else:
            e = torch.exp(scores - m)
            p = e / e.sum(dim=-1, keepdim=True)
        out[s] = torch.einsum("hn,nhd->hd", p.to(qd).float(), v.float()).to(qd)
    return out
