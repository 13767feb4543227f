"""GPU parity of per-head and per-block FP8 scales: the decode entry points against the oracle
(atol = rtol = 1e-2 on outputs brought to unit magnitude), the KV-cache writer bit-exact, and
the two together as a write -> attend round trip."""
import pytest
import torch

from flash_attention_factory_amd import lib, workloads as W
from flash_attention_factory_amd.lib import kv_cache_write

pytestmark = pytest.mark.gpu
ATOL = RTOL = 1e-2


def _dev():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch.device("cuda:0")


def _scales(shape, seed, lo, hi):
    """Log-uniform in [lo, hi]."""
    g = torch.Generator().manual_seed(seed)
    u = torch.rand(shape, generator=g)
    return (torch.tensor(lo).log() + u * (torch.tensor(hi).log() - torch.tensor(lo).log())).exp().float()


def _views(w):
    return (w.key_cache.permute(0, 2, 1, 3), w.value_cache.permute(0, 2, 1, 3)) if w.layout == W.HEAD_MAJOR \
        else (w.key_cache, w.value_cache)


def _call(w, kernel, query=None, **kw):
    """lib.paged_attention_<kernel>.run with upstream's positional arguments; `query` may be 4-D."""
    mod = getattr(lib, "paged_attention_" + kernel)
    q = w.query if query is None else query
    rows = q.shape[0] * (q.shape[1] if q.dim() == 4 else 1)
    H, D = q.shape[-2], q.shape[-1]
    NP = -(-int(w.context_lens.max()) // w.partition_size)
    dev = q.device
    ml = torch.full((rows, H, NP), float("nan"), dtype=torch.float32, device=dev)
    es = torch.full_like(ml, float("nan"))
    tmp = torch.full((rows, H, NP, D), float("nan"), dtype=torch.float32, device=dev)
    out = torch.zeros_like(q)
    kv, vv = _views(w)
    extra = dict(partition_size=w.partition_size) if "reduce" in kernel else {}
    args = (ml, es, tmp, out, None, q, kv, vv, w.block_tables, w.context_lens, H // w.num_kv_heads, w.scale,
            w.fp8_scale, w.block_size, int(w.context_lens.max()), None, w.sinks, 0.0)
    times = mod.run(*args, **extra, **kw)
    if "reduce" in kernel and times[1] == 0.0:
        # rows so short that the split entry ran the single-pass kernel; this test is after the split kernels
        mod.run(*args, **extra, **dict(kw, schedule=3))
    torch.cuda.synchronize()
    return out


def _ref(oracle, w, query=None, **kw):
    return oracle.attention_ref(w.query if query is None else query, w.key_cache, w.value_cache, w.block_tables,
                                w.context_lens, scale=w.scale, block_size=w.block_size, kv_strides=w.kv_strides(),
                                num_kv_heads=w.num_kv_heads, sinks=w.sinks, want_f32=True, **kw)[1]


def _close(got, ref, what):
    unit = ref.abs().max()
    torch.testing.assert_close(got.float().cpu() / unit, ref / unit, atol=ATOL, rtol=RTOL, msg=lambda m: f"{what}: {m}")


@pytest.mark.parametrize("per_block", [False, True], ids=["head", "block"])
@pytest.mark.parametrize("fp8_dtype", [torch.float8_e5m2, torch.float8_e4m3fn], ids=["e5m2", "e4m3"])
@pytest.mark.parametrize("layout", [W.TOKEN_MAJOR, W.HEAD_MAJOR])
def test_scaled_caches_match_oracle(oracle, per_block, fp8_dtype, layout):
    w = W.make_test_shaped(batch_size=4, nheads=8, nheads_k=2, d=128, seqlen_k=1500, varlen=True, has_sinks=True,
                           fp8=True, block_size=16, seed=41, layout=layout, fp8_dtype=fp8_dtype)
    w.context_lens[0] = 1
    w.context_lens[1] = 513
    NB = w.key_cache.shape[0]
    shape = (NB, 2) if per_block else (2,)
    ks, vs = _scales(shape, 1, 0.3, 3.0), _scales(shape, 2, 0.3, 3.0)
    ref = _ref(oracle, w, k_scales=ks, v_scales=vs)
    wd = w.to(_dev())
    for kernel in ("fp8_loop", "fp8_reduce"):
        got = _call(wd, kernel, k_scales=ks.to(_dev()), v_scales=vs.to(_dev()))
        _close(got, ref, kernel)


@pytest.mark.parametrize("qdtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("fp8_dtype", [torch.float8_e5m2, torch.float8_e4m3fn], ids=["e5m2", "e4m3"])
def test_amax_sized_block_scales(oracle, qdtype, fp8_dtype):
    """Scales as amax scaling produces them: around 1e-4 for E5M2 (amax / 57344), 1e-2 for E4M3,
    and three orders of magnitude apart between blocks.  The probabilities carry the V scale
    relative to the sequence's first block, so nothing leaves the 16-bit normal range."""
    w = W.make_config(4, num_seqs=3, pool_blocks=400, lens=[2100, 40, 1030], fp8_dtype=fp8_dtype)   # bf16 q, G = 8
    w.query = w.query.to(qdtype)
    NB, Hk = w.key_cache.shape[0], w.num_kv_heads
    top = 57344.0 if fp8_dtype == torch.float8_e5m2 else 448.0
    ks = _scales((NB, Hk), 5, 0.5 / top, 4.0 / top)     # keys: amax 0.5 .. 4
    vs = _scales((NB, Hk), 6, 0.02 / top, 20.0 / top)   # values: amax 0.02 .. 20
    # the caches hold N(0,1) bytes; bring the products back to O(1) logits
    w.scale = w.scale * top / 4.0
    ref = _ref(oracle, w, k_scales=ks, v_scales=vs)
    wd = w.to(_dev())
    for kernel in ("fp8_loop", "fp8_reduce"):
        got = _call(wd, kernel, k_scales=ks.to(_dev()), v_scales=vs.to(_dev()))
        assert torch.isfinite(got).all()
        _close(got, ref, kernel)


def test_block_scales_with_query_tokens_and_window(oracle):
    w = W.make_test_shaped(batch_size=3, nheads=8, nheads_k=2, d=128, seqlen_k=1300, varlen=True, has_sinks=False,
                           fp8=True, block_size=16, seed=43, fp8_dtype=torch.float8_e4m3fn)
    NB = w.key_cache.shape[0]
    ks, vs = _scales((NB, 2), 7, 0.2, 2.0), _scales((NB, 2), 8, 0.2, 2.0)
    g = torch.Generator().manual_seed(9)
    query4 = torch.randn(3, 4, 8, 128, generator=g).to(torch.float16)
    ref = _ref(oracle, w, query=query4, k_scales=ks, v_scales=vs, window_left=600)
    wd = w.to(_dev())
    for kernel in ("fp8_loop", "fp8_reduce"):
        got = _call(wd, kernel, query=query4.to(_dev()), k_scales=ks.to(_dev()), v_scales=vs.to(_dev()),
                    window_left=600)
        _close(got, ref, kernel)


def test_equal_scales_equal_the_scalar_path(oracle):
    """Arrays holding one value everywhere give what upstream's scalar fp8_scale gives (other
    kernels underneath, so equal within rounding, not bit for bit)."""
    w = W.make_config(3, num_seqs=4, pool_blocks=500, lens=[1200, 600, 77, 1999])
    NB, Hk = w.key_cache.shape[0], w.num_kv_heads
    w.fp8_scale = 0.5
    wd = w.to(_dev())
    want = {k: _call(wd, k).float() for k in ("fp8_loop", "fp8_reduce")}
    for shape in ((Hk,), (NB, Hk)):
        full = torch.full(shape, 0.5, dtype=torch.float32, device=_dev())
        for kernel in ("fp8_loop", "fp8_reduce"):
            got = _call(wd, kernel, k_scales=full, v_scales=full.clone()).float()
            torch.testing.assert_close(got, want[kernel], atol=2e-3, rtol=2e-2)


# ---- writer --------------------------------------------------------------------------------

@pytest.mark.parametrize("per_block", [False, True], ids=["head", "block"])
@pytest.mark.parametrize("fp8_dtype", [torch.float8_e5m2, torch.float8_e4m3fn], ids=["e5m2", "e4m3"])
@pytest.mark.parametrize("src", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("layout", [W.TOKEN_MAJOR, W.HEAD_MAJOR])
def test_scaled_writer_is_bit_exact(oracle, per_block, fp8_dtype, src, layout):
    g = torch.Generator().manual_seed(51)
    N, Hk, D, B, NB = 700, 4, 128, 16, 60
    key = (torch.randn(N, Hk, D, generator=g) * 6).to(src)
    value = (torch.randn(N, Hk, D, generator=g) * 6).to(src)
    slots = torch.randperm(NB * B, generator=g)[:N].to(torch.int64)
    slots[::19] = -1
    shape = (NB, Hk) if per_block else (Hk,)
    ks, vs = _scales(shape, 3, 0.01, 3.0), _scales(shape, 4, 0.01, 3.0)
    pshape = (NB, B, Hk, D) if layout == W.TOKEN_MAJOR else (NB, Hk, B, D)
    kc, vc = torch.full(pshape, 9, dtype=torch.uint8), torch.full(pshape, 9, dtype=torch.uint8)
    view = (lambda t: t) if layout == W.TOKEN_MAJOR else (lambda t: t.permute(0, 2, 1, 3))
    dev = _dev()
    kc_d, vc_d = kc.to(dev).view(fp8_dtype), vc.to(dev).view(fp8_dtype)
    v = view(kc)
    oracle.kv_cache_write(key, value, kc, vc, slots, block_size=B, kv_strides=(v.stride(0), v.stride(1), v.stride(2)),
                          e4m3=fp8_dtype == torch.float8_e4m3fn, k_scales=ks, v_scales=vs)
    kv_cache_write.run(key.to(dev), value.to(dev), view(kc_d), view(vc_d), slots.to(dev),
                       k_scales=ks.to(dev), v_scales=vs.to(dev))
    torch.cuda.synchronize()
    assert torch.equal(kc_d.view(torch.uint8).cpu(), kc) and torch.equal(vc_d.view(torch.uint8).cpu(), vc)


def test_write_then_attend_with_block_scales(oracle):
    """Blocks of very different magnitude, amax scaling per block and kv head, E4M3 bytes: the
    device writer and the device decode kernels together reproduce attention over the original
    16-bit rows to the format's precision, and agree with the oracle doing the same."""
    g = torch.Generator().manual_seed(61)
    S, H, Hk, D, B, NB = 3, 16, 2, 128, 16, 200
    lens = torch.tensor([1500, 33, 700], dtype=torch.int32)
    perm = torch.randperm(NB, generator=g).to(torch.int32)
    nb = [(int(n) + B - 1) // B for n in lens]
    tables = torch.zeros((S, max(nb)), dtype=torch.int32)
    off = 0
    for s in range(S):
        tables[s, :nb[s]] = perm[off:off + nb[s]]
        off += nb[s]
    mags = torch.rand(NB, generator=g) * 3 - 1.5                      # 10^-1.5 .. 10^1.5
    mags = 10.0 ** mags
    slots = torch.cat([tables[s, torch.arange(int(lens[s])) // B].long() * B + torch.arange(int(lens[s])) % B
                       for s in range(S)])
    N = slots.numel()
    key = (torch.randn(N, Hk, D, generator=g) * mags[slots // B].view(N, 1, 1) * 0.3).to(torch.float16)
    value = (torch.randn(N, Hk, D, generator=g) * mags[slots // B].view(N, 1, 1)).to(torch.float16)
    blk = slots // B
    ks, vs = torch.ones(NB, Hk), torch.ones(NB, Hk)
    at = blk.view(N, 1).expand(N, Hk)
    ks.scatter_reduce_(0, at, key.float().abs().amax(dim=2), "amax", include_self=False)
    vs.scatter_reduce_(0, at, value.float().abs().amax(dim=2), "amax", include_self=False)
    used = torch.zeros(NB, dtype=torch.bool)
    used[blk] = True
    ks = torch.where(used[:, None], ks / 448.0, torch.ones(()))
    vs = torch.where(used[:, None], vs / 448.0, torch.ones(()))
    query = torch.randn(S, H, D, generator=g).to(torch.float16)
    scale = 0.02

    dev = _dev()
    kc = torch.zeros((NB, Hk, B, D), dtype=torch.float8_e4m3fn, device=dev)          # head-major pools
    vc = torch.zeros_like(kc)
    kv_cache_write.run(key.to(dev), value.to(dev), kc.permute(0, 2, 1, 3), vc.permute(0, 2, 1, 3), slots.to(dev),
                       k_scales=ks.to(dev), v_scales=vs.to(dev))
    w = W.Workload(name="roundtrip", query=query.to(dev), key_cache=kc, value_cache=vc, block_tables=tables.to(dev),
                   context_lens=lens.to(dev), scale=scale, block_size=B, num_kv_heads=Hk, layout=W.HEAD_MAJOR,
                   partition_size=512)
    # the oracle on the bytes the device wrote
    wc = w.to("cpu")
    ref = _ref(oracle, wc, k_scales=ks, v_scales=vs)
    # attention over the unquantised rows
    k16 = torch.zeros((NB * B, Hk, D), dtype=torch.float16)          # token-major pools of the 16-bit rows
    v16 = torch.zeros_like(k16)
    k16[slots] = key
    v16[slots] = value
    exact = oracle.attention_ref(query, k16.view(NB, B, Hk, D), v16.view(NB, B, Hk, D), tables, lens, scale=scale,
                                 block_size=B, kv_strides=(B * Hk * D, Hk * D, D), num_kv_heads=Hk, want_f32=True)[1]
    for kernel in ("fp8_loop", "fp8_reduce"):
        got = _call(w, kernel, k_scales=ks.to(dev), v_scales=vs.to(dev))
        _close(got, ref, kernel)
        err = (got.float().cpu() - exact).abs().max() / exact.abs().max()
        assert err < 0.1, (kernel, float(err))


def test_block_scales_in_every_scheduling_form(oracle):
    """Per-block scales on a batch the persistent kernels take whole (100 sequences, several items
    per work-group), on one they take as sub-batches (300 sequences) and on one left to the grid
    form (a table of 2^24 tokens per sequence)."""
    for S, seed, wide in ((100, 71, False), (300, 72, False), (7, 73, True)):
        gen = torch.Generator().manual_seed(seed)
        lens = torch.randint(1, 1200, (S,), generator=gen)
        lens[::11] = 0
        w = W.make_test_shaped(batch_size=S, nheads=4, nheads_k=2, d=64, seqlen_k=1200, varlen=False, has_sinks=True,
                               fp8=True, block_size=16, seed=seed, fp8_dtype=torch.float8_e4m3fn)
        w.context_lens = lens.to(torch.int32)
        w.partition_size = 256
        if wide:
            table = torch.zeros((S, (1 << 24) // w.block_size), dtype=torch.int32)
            table[:, :w.block_tables.shape[1]] = w.block_tables
            w.block_tables = table
        NB = w.key_cache.shape[0]
        ks, vs = _scales((NB, 2), seed, 0.2, 3.0), _scales((NB, 2), seed + 1, 0.01, 3.0)
        ref = _ref(oracle, w, k_scales=ks, v_scales=vs)
        wd = w.to(_dev())
        live = lens > 0
        for kernel in ("fp8_loop", "fp8_reduce"):
            got = _call(wd, kernel, k_scales=ks.to(_dev()), v_scales=vs.to(_dev())).float().cpu()
            assert (got[~live] == 0).all(), (S, kernel)
            unit = ref[live].abs().max()
            torch.testing.assert_close(got[live] / unit, ref[live] / unit, atol=ATOL, rtol=RTOL,
                                       msg=lambda m: f"S={S} {kernel}: {m}")


def test_scales_of_unused_blocks_may_be_anything(oracle):
    """A tile wholly past a context takes its block id from a clamped or padding column of the table;
    that block's scales (and bytes) belong to nobody and may be NaN.  The V scale is applied by
    select, like the K/V tail itself: loop, segment and grid forms, block sizes 16 and 32."""
    for S, seed, block_size, schedule in ((40, 81, 16, 0), (40, 82, 32, 0), (9, 83, 16, 1), (300, 84, 16, 0)):
        gen = torch.Generator().manual_seed(seed)
        lens = torch.randint(1, 900, (S,), generator=gen)
        lens[0], lens[1], lens[2] = 1, 17, 16 * 7 + 3  # contexts that end inside the first tile of a chunk
        w = W.make_test_shaped(batch_size=S, nheads=8, nheads_k=2, d=128, seqlen_k=900, varlen=False, has_sinks=False,
                               fp8=True, block_size=block_size, seed=seed)
        w.context_lens = lens.to(torch.int32)
        NB = w.key_cache.shape[0]
        used = torch.zeros(NB, dtype=torch.bool)
        cols = torch.arange(w.block_tables.shape[1])
        spare = None
        for s in range(S):
            n = -(-int(lens[s]) // block_size)
            used[w.block_tables[s, :n].long()] = True
        spare = int((~used).nonzero()[0])
        for s in range(S):  # every column past the context points at a block nobody uses
            n = -(-int(lens[s]) // block_size)
            w.block_tables[s, n:] = spare
        ks, vs = _scales((NB, 2), seed, 0.2, 3.0), _scales((NB, 2), seed + 1, 0.01, 3.0)
        ks[~used], vs[~used] = float("nan"), float("nan")
        kb, vb = w.key_cache.view(torch.uint8), w.value_cache.view(torch.uint8)
        kb[~used], vb[~used] = 0x7f, 0x7f  # NaN bytes
        ref = _ref(oracle, w, k_scales=ks, v_scales=vs)
        assert torch.isfinite(ref).all()
        wd = w.to(_dev())
        for kernel in ("fp8_loop", "fp8_reduce"):
            got = _call(wd, kernel, k_scales=ks.to(_dev()), v_scales=vs.to(_dev()), schedule=schedule).float().cpu()
            assert torch.isfinite(got).all(), (S, block_size, kernel)
            unit = ref.abs().max()
            torch.testing.assert_close(got / unit, ref / unit, atol=ATOL, rtol=RTOL,
                                       msg=lambda m: f"S={S} B={block_size} {kernel}: {m}")
