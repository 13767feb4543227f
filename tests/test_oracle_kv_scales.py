"""Pins of the oracle's per-head and per-block FP8 scales against independent routines:
torch dequantisation + gather + scaled_dot_product_attention for the attention reference,
torch's own fp32 -> FP8 casts with torch indexing for the writer.  CPU only.

Upstream has one scalar scale (paged_attention_kernel_fp8_loop.hpp:328-333,540-545) and its
tests pass 1.0; finer scales have no upstream counterpart, so what is pinned here is the
stated reading K^ = dequant(K) * k_scale, V^ = dequant(V) * v_scale."""
import pytest
import torch
import torch.nn.functional as F

from flash_attention_factory_amd import workloads as W


def _scaled_dense(w, cache, scales):
    """[S, max_ctx, Hk, D] fp32: every row dequantised and multiplied with the scale of its
    kv head ([Hk]) or of its physical block and kv head ([NB, Hk])."""
    S, B = w.num_seqs, w.block_size
    max_ctx = int(w.context_lens.max())
    nb = (max_ctx + B - 1) // B
    c = cache.to(w.query.dtype).float()
    if w.layout == "head_major":
        c = c.permute(0, 2, 1, 3)                     # [NB, B, Hk, D]
    if scales.dim() == 1:
        c = c * scales.view(1, 1, -1, 1)
    else:
        c = c * scales.view(scales.shape[0], 1, scales.shape[1], 1)
    idx = w.block_tables[:, :nb].long()
    return c[idx.reshape(-1)].reshape(S, nb * B, c.shape[2], c.shape[3])[:, :max_ctx]


def _sdpa(w, k_scales, v_scales):
    S, H, D = w.query.shape
    G = H // w.num_kv_heads
    k = _scaled_dense(w, w.key_cache, k_scales).repeat_interleave(G, dim=2).permute(0, 2, 1, 3)
    v = _scaled_dense(w, w.value_cache, v_scales).repeat_interleave(G, dim=2).permute(0, 2, 1, 3)
    T = k.shape[2]
    bias = torch.zeros(S, 1, 1, T)
    bias.masked_fill_((torch.arange(T)[None, :] >= w.context_lens[:, None].long())[:, None, None, :], float("-inf"))
    if w.sinks is not None:
        k = torch.cat([k, torch.zeros(S, H, 1, D)], dim=2)
        v = torch.cat([v, torch.zeros(S, H, 1, D)], dim=2)
        bias = torch.cat([bias.expand(S, H, 1, T), w.sinks.float().view(1, H, 1, 1).expand(S, H, 1, 1)], dim=3)
    return F.scaled_dot_product_attention(w.query.float().unsqueeze(2), k, v, attn_mask=bias, scale=w.scale).squeeze(2)


def _scales(shape, seed, lo=0.25, hi=4.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.rand(shape, generator=g) * (hi - lo) + lo).float()


def _oracle(oracle, w, **kw):
    return oracle.attention_ref(w.query, w.key_cache, w.value_cache, w.block_tables, w.context_lens, scale=w.scale,
                                block_size=w.block_size, kv_strides=w.kv_strides(), num_kv_heads=w.num_kv_heads,
                                sinks=w.sinks, want_f32=True, **kw)[1]


@pytest.mark.parametrize("fp8_dtype", [torch.float8_e5m2, torch.float8_e4m3fn])
@pytest.mark.parametrize("per_block", [False, True])
@pytest.mark.parametrize("layout", [W.TOKEN_MAJOR, W.HEAD_MAJOR])
@pytest.mark.parametrize("sinks", [False, True])
def test_scaled_attention_matches_sdpa(oracle, fp8_dtype, per_block, layout, sinks):
    w = W.make_test_shaped(batch_size=3, nheads=6, nheads_k=2, d=64, seqlen_k=150, varlen=True, has_sinks=sinks,
                           fp8=True, block_size=16, seed=21, layout=layout, fp8_dtype=fp8_dtype)
    NB = w.key_cache.shape[0]
    shape = (NB, 2) if per_block else (2,)
    ks, vs = _scales(shape, 1), _scales(shape, 2)
    got = _oracle(oracle, w, k_scales=ks, v_scales=vs)
    want = _sdpa(w, ks, vs)
    torch.testing.assert_close(got, want, rtol=3e-5, atol=3e-6)
    # and the scales matter: without them the result is another one
    plain = _oracle(oracle, w)
    assert (plain - got).abs().max() > 1e-2


def test_equal_scales_reduce_to_the_scalar(oracle):
    """Per-head and per-block arrays that hold one value s everywhere are upstream's fp8_scale = s."""
    w = W.make_test_shaped(batch_size=2, nheads=4, nheads_k=2, d=64, seqlen_k=90, varlen=True, has_sinks=True,
                           fp8=True, block_size=16, seed=22)
    NB = w.key_cache.shape[0]
    s = 0.375
    want = _oracle(oracle, w, fp8_scale=s)
    for shape in ((2,), (NB, 2)):
        full = torch.full(shape, s, dtype=torch.float32)
        got = _oracle(oracle, w, k_scales=full, v_scales=full.clone())
        assert torch.equal(got, want)


def test_v_scale_is_linear_and_k_scale_is_a_softmax_temperature(oracle):
    w = W.make_test_shaped(batch_size=2, nheads=4, nheads_k=2, d=64, seqlen_k=70, varlen=False, has_sinks=False,
                           fp8=True, block_size=16, seed=23)
    one = torch.ones(2)
    base = _oracle(oracle, w, k_scales=one, v_scales=one.clone())
    # V scale per head multiplies that head group's output
    vs = torch.tensor([2.0, 0.5])
    got = _oracle(oracle, w, k_scales=one, v_scales=vs)
    torch.testing.assert_close(got[:, :2], base[:, :2] * 2.0, rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(got[:, 2:], base[:, 2:] * 0.5, rtol=1e-6, atol=1e-7)
    # K scale c on every head = softmax scale multiplied by c
    ks = torch.full((2,), 3.0)
    got = _oracle(oracle, w, k_scales=ks, v_scales=one.clone())
    want = oracle.attention_ref(w.query, w.key_cache, w.value_cache, w.block_tables, w.context_lens, scale=w.scale * 3.0,
                                block_size=w.block_size, kv_strides=w.kv_strides(), num_kv_heads=w.num_kv_heads,
                                want_f32=True)[1]
    torch.testing.assert_close(got, want, rtol=2e-5, atol=2e-6)


@pytest.mark.parametrize("per_block", [False, True])
@pytest.mark.parametrize("fp8_dtype", [torch.float8_e5m2, torch.float8_e4m3fn])
@pytest.mark.parametrize("src", [torch.float16, torch.bfloat16])
def test_scaled_writer_matches_torch_cast_and_indexing(oracle, per_block, fp8_dtype, src):
    g = torch.Generator().manual_seed(31)
    N, Hk, D, B, NB = 41, 3, 64, 16, 5
    key = (torch.randn(N, Hk, D, generator=g) * 4).to(src)
    value = (torch.randn(N, Hk, D, generator=g) * 4).to(src)
    slots = torch.randperm(NB * B, generator=g)[:N].to(torch.int64)
    slots[7] = -1
    shape = (NB, Hk) if per_block else (Hk,)
    ks, vs = _scales(shape, 3, 0.05, 2.0), _scales(shape, 4, 0.05, 2.0)
    kc = torch.full((NB, B, Hk, D), 9, dtype=torch.uint8)
    vc = torch.full((NB, B, Hk, D), 9, dtype=torch.uint8)
    want_k, want_v = kc.clone(), vc.clone()
    for n in range(N):
        s = int(slots[n])
        if s < 0:
            continue
        b = s // B
        for pool, srct, sc in ((want_k, key, ks), (want_v, value, vs)):
            row_scale = sc[b] if per_block else sc                     # [Hk]
            q = srct[n].float() * (1.0 / row_scale).view(Hk, 1)         # fp32 product, rounded once by the cast
            pool[b, s % B] = q.to(fp8_dtype).view(torch.uint8)
    oracle.kv_cache_write(key, value, kc, vc, slots, block_size=B, kv_strides=(B * Hk * D, Hk * D, D),
                          e4m3=fp8_dtype == torch.float8_e4m3fn, k_scales=ks, v_scales=vs)
    assert torch.equal(kc, want_k) and torch.equal(vc, want_v)


def test_write_then_read_recovers_the_rows(oracle):
    """Quantise with per-block scales, attend with the same scales: the result is attention over
    the original rows up to the format's rounding (E4M3: 2^-4 relative per element)."""
    g = torch.Generator().manual_seed(33)
    S, H, Hk, D, B = 2, 4, 2, 64, 16
    lens = torch.tensor([40, 23], dtype=torch.int32)
    nblk = [3, 2]
    NB = 6
    tables = torch.tensor([[4, 1, 5], [0, 3, 0]], dtype=torch.int32)
    mags = torch.tensor([0.01, 30.0, 1.0, 200.0, 0.3, 5.0])           # very different blocks
    kc = torch.zeros((NB, B, Hk, D), dtype=torch.uint8)
    vc = torch.zeros((NB, B, Hk, D), dtype=torch.uint8)
    keys, values, slots = [], [], []
    for s in range(S):
        for t in range(int(lens[s])):
            b = int(tables[s, t // B])
            keys.append(torch.randn(Hk, D, generator=g) * mags[b])
            values.append(torch.randn(Hk, D, generator=g) * mags[b])
            slots.append(b * B + t % B)
    key = torch.stack(keys).to(torch.float16)
    value = torch.stack(values).to(torch.float16)
    slots = torch.tensor(slots, dtype=torch.int64)
    # amax scaling per block and kv head, as a serving engine would choose it
    ks = torch.ones(NB, Hk)
    vs = torch.ones(NB, Hk)
    for b in range(NB):
        sel = (slots // B) == b
        if sel.any():
            ks[b] = key[sel].float().abs().amax(dim=(0, 2)) / 448.0
            vs[b] = value[sel].float().abs().amax(dim=(0, 2)) / 448.0
    oracle.kv_cache_write(key, value, kc, vc, slots, block_size=B, kv_strides=(B * Hk * D, Hk * D, D), e4m3=True,
                          k_scales=ks, v_scales=vs)
    query = torch.randn(S, H, D, generator=g).to(torch.float16)
    kc8, vc8 = kc.view(torch.float8_e4m3fn), vc.view(torch.float8_e4m3fn)
    got = oracle.attention_ref(query, kc8, vc8, tables, lens, scale=D ** -0.5, block_size=B,
                               kv_strides=(B * Hk * D, Hk * D, D), num_kv_heads=Hk, want_f32=True,
                               k_scales=ks, v_scales=vs)[1]
    # attention over the unquantised rows
    k16 = torch.zeros((NB, B, Hk, D), dtype=torch.float16)
    v16 = torch.zeros((NB, B, Hk, D), dtype=torch.float16)
    k16.view(NB * B, Hk, D)[slots] = key
    v16.view(NB * B, Hk, D)[slots] = value
    want = oracle.attention_ref(query, k16, v16, tables, lens, scale=D ** -0.5, block_size=B,
                                kv_strides=(B * Hk * D, Hk * D, D), num_kv_heads=Hk, want_f32=True)[1]
    err = (got - want).abs().max() / want.abs().max()
    assert err < 0.08, err
    # with one scalar for everything the small blocks are flushed away or the large ones overflow
    assert torch.isfinite(got).all()
