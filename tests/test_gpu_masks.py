"""GPU parity of the opt-in score modifiers (soft-capping, local window, ALiBi) with the oracle,
through all four entry points; and the default stays upstream's: slopes and cap are ignored."""
import pytest
import torch

from flash_attention_factory_amd import lib, runner, workloads as W
from _torch_ref import assert_close_to_reference, call_oracle

pytestmark = pytest.mark.gpu
ATOL = RTOL = 1e-2

CASES = [
    dict(window_left=100),
    dict(window_left=0),
    dict(window_left=700),
    dict(alibi=True),
    dict(softcap=5.0),
    dict(softcap=0.7, alibi=True, window_left=64),
    dict(softcap=30.0, alibi=True, window_left=1300),
]


def _dev():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch.device("cuda:0")


def _call(w, kernel, **mods):
    """One call of lib.<kernel>.run with upstream's positional arguments plus the opt-in keywords."""
    mod = getattr(lib, "paged_attention_" + kernel)
    bufs = runner.alloc_buffers(w)
    H, Hk = w.query.shape[1], w.num_kv_heads
    kv, vv = (w.key_cache.permute(0, 2, 1, 3), w.value_cache.permute(0, 2, 1, 3)) if w.layout == W.HEAD_MAJOR \
        else (w.key_cache, w.value_cache)
    head = [bufs.max_logits, bufs.exp_sums, bufs.tmp_out, bufs.out, None, w.query, kv, vv, w.block_tables,
            w.context_lens, H // Hk, w.scale]
    if kernel.startswith("fp8"):
        head.append(w.fp8_scale)
    alibi, softcap = mods.pop("alibi_slopes", None), mods.pop("softcap", 0.0)
    extra = dict(partition_size=w.partition_size) if "reduce" in kernel else {}
    times = mod.run(*head, w.block_size, int(w.context_lens.max()), alibi, w.sinks, softcap, **extra, **mods)
    if "reduce" in kernel and times[1] == 0.0:
        # rows so short that the split entry ran the single-pass kernel; this test is after the split kernels
        mod.run(*head, w.block_size, int(w.context_lens.max()), alibi, w.sinks, softcap, schedule=3, **extra, **mods)
    torch.cuda.synchronize()
    return bufs.out


@pytest.mark.parametrize("mk", CASES, ids=lambda m: "_".join(f"{k}{v}" for k, v in m.items()))
@pytest.mark.parametrize("fp8", [False, True])
def test_modifiers_match_oracle(oracle, mk, fp8):
    w = W.make_test_shaped(batch_size=4, nheads=8, nheads_k=2, d=128, seqlen_k=1500, varlen=True, has_sinks=True,
                           fp8=fp8, seed=5)
    w.context_lens[0] = 1
    w.context_lens[1] = 513          # one token into the second partition
    H = w.query.shape[1]
    w.sinks = torch.linspace(-3, 3, H).to(w.query.dtype)  # modest: the keys keep most of the softmax mass
    alibi = torch.rand(H, generator=torch.Generator().manual_seed(2)) * 0.05 if mk.get("alibi") else None
    okw = dict(alibi_slopes=alibi, softcap=mk.get("softcap", 0.0), window_left=mk.get("window_left", -1))
    ref = call_oracle(oracle.attention_ref, w, want_f32=True, **okw)[1]
    # the modifier must matter: against plain attention the result moves by far more than the tolerance
    plain = call_oracle(oracle.attention_ref, w, want_f32=True)[1]
    moved = ((ref - plain)[2:].abs().amax() / plain[2:].abs().amax()).item()
    assert moved > 0.3, moved
    wd = w.to(_dev())
    mods = dict(alibi_slopes=None if alibi is None else alibi.to(_dev()), softcap=okw["softcap"],
                apply_alibi=alibi is not None, apply_softcap=okw["softcap"] > 0,
                window_left=mk.get("window_left"))
    for kernel in (("fp8_loop", "fp8_reduce") if fp8 else ("loop", "reduce")):
        got = _call(wd, kernel, **dict(mods)).float().cpu()
        assert torch.isfinite(got).all()
        assert_close_to_reference(got, ref, f"{kernel} {mk}")


def test_modifiers_on_a_measured_shape(oracle):
    """bf16 queries, E5M2 pools, G = 8, block 16, head-major, window across many partitions."""
    w = W.make_config(4, num_seqs=3, pool_blocks=1200, lens=[5000, 64, 2049])
    H = w.query.shape[1]
    alibi = torch.linspace(0.001, 0.02, H)
    ref = call_oracle(oracle.attention_ref, w, want_f32=True, alibi_slopes=alibi, softcap=20.0, window_left=1500)[1]
    wd = w.to(_dev())
    for kernel in ("fp8_loop", "fp8_reduce"):
        got = _call(wd, kernel, alibi_slopes=alibi.to(_dev()), softcap=20.0, apply_alibi=True, apply_softcap=True,
                    window_left=1500).float().cpu()
        assert_close_to_reference(got, ref)


def test_default_ignores_slopes_and_cap(oracle):
    """Upstream's tests hand the kernels alibi_slopes = ones and expect plain attention
    (test_paged.py:456,480): without the opt-in keywords that is what comes out."""
    w = W.make_test_shaped(batch_size=2, nheads=8, nheads_k=2, d=64, seqlen_k=400, varlen=True, has_sinks=False)
    ref = call_oracle(oracle.attention_ref, w, want_f32=True)[1]
    wd = w.to(_dev())
    ones = torch.ones(8, dtype=torch.float32, device=_dev())
    for kernel in ("loop", "reduce"):
        got = _call(wd, kernel, alibi_slopes=ones, softcap=3.0).float().cpu()
        assert_close_to_reference(got, ref)


def _call_multi(w, query4, kernel, **mods):
    """lib.<kernel>.run with query/out of shape [S, query_len, H, D] and scratch rows to match."""
    dev = query4.device
    mod = getattr(lib, "paged_attention_" + kernel)
    S, QL, H, D = query4.shape
    Hk = w.num_kv_heads
    NP = -(-int(w.context_lens.max()) // w.partition_size)
    out = torch.zeros_like(query4)
    ml = torch.full((S * QL, H, NP), float("nan"), dtype=torch.float32, device=dev)
    es = torch.full_like(ml, float("nan"))
    tmp = torch.full((S * QL, H, NP, D), float("nan"), dtype=torch.float32, device=dev)
    kv, vv = (w.key_cache.permute(0, 2, 1, 3), w.value_cache.permute(0, 2, 1, 3)) if w.layout == W.HEAD_MAJOR \
        else (w.key_cache, w.value_cache)
    head = [ml, es, tmp, out, None, query4, kv, vv, w.block_tables, w.context_lens, H // Hk, w.scale]
    if kernel.startswith("fp8"):
        head.append(w.fp8_scale)
    alibi, softcap = mods.pop("alibi_slopes", None), mods.pop("softcap", 0.0)
    extra = dict(partition_size=w.partition_size) if "reduce" in kernel else {}
    times = mod.run(*head, w.block_size, int(w.context_lens.max()), alibi, w.sinks, softcap, **extra, **mods)
    if "reduce" in kernel and times[1] == 0.0:
        # rows so short that the split entry ran the single-pass kernel; this test is after the split kernels
        mod.run(*head, w.block_size, int(w.context_lens.max()), alibi, w.sinks, softcap, schedule=3, **extra, **mods)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("QL,nheads,nheads_k", [(2, 8, 2), (4, 8, 2), (8, 4, 2), (16, 2, 2), (3, 10, 2)])
@pytest.mark.parametrize("fp8", [False, True])
def test_several_query_tokens_per_sequence(oracle, QL, nheads, nheads_k, fp8):
    """Speculative-decoding shaped calls: QL query tokens per sequence, causal among themselves,
    (query token, head) pairs filling the 16 MFMA columns."""
    w = W.make_test_shaped(batch_size=4, nheads=nheads, nheads_k=nheads_k, d=128, seqlen_k=1400, varlen=True,
                           has_sinks=True, fp8=fp8, seed=13)
    w.context_lens[0] = QL                 # the query tokens are the whole context
    w.context_lens[1] = 512 + 1            # the last query token opens a new partition
    w.context_lens[2] = 1024               # the query tokens end exactly on a partition boundary
    g = torch.Generator().manual_seed(4)
    query4 = torch.randn(4, QL, nheads, 128, generator=g).to(torch.float16)
    ref = oracle.attention_ref(query4, w.key_cache, w.value_cache, w.block_tables, w.context_lens, scale=w.scale,
                               block_size=w.block_size, kv_strides=w.kv_strides(), num_kv_heads=w.num_kv_heads,
                               sinks=w.sinks, fp8_scale=w.fp8_scale, want_f32=True)[1]
    wd = w.to(_dev())
    for kernel in (("fp8_loop", "fp8_reduce") if fp8 else ("loop", "reduce")):
        got = _call_multi(wd, query4.to(_dev()), kernel).float().cpu()
        assert torch.isfinite(got).all(), kernel
        assert_close_to_reference(got, ref, f"{kernel} QL={QL}")


def test_query_tokens_with_modifiers_and_last_token_equals_decode(oracle):
    w = W.make_config(4, num_seqs=3, pool_blocks=1200, lens=[3000, 70, 1537])      # bf16, E5M2, G = 8
    H = w.query.shape[1]
    QL = 2
    g = torch.Generator().manual_seed(6)
    query4 = torch.randn(3, QL, H, 128, generator=g).to(torch.bfloat16)
    alibi = torch.linspace(0.001, 0.02, H)
    okw = dict(alibi_slopes=alibi, softcap=25.0, window_left=900)
    ref = oracle.attention_ref(query4, w.key_cache, w.value_cache, w.block_tables, w.context_lens, scale=w.scale,
                               block_size=w.block_size, kv_strides=w.kv_strides(), num_kv_heads=w.num_kv_heads,
                               fp8_scale=w.fp8_scale, want_f32=True, **okw)[1]
    wd = w.to(_dev())
    mods = dict(alibi_slopes=alibi.to(_dev()), softcap=25.0, apply_alibi=True, apply_softcap=True, window_left=900)
    for kernel in ("fp8_loop", "fp8_reduce"):
        got = _call_multi(wd, query4.to(_dev()), kernel, **dict(mods))
        assert_close_to_reference(got, ref)
        # the last query token alone is a plain decode call with the same modifiers
        wq = W.Workload(**{**wd.__dict__})
        wq.query = query4[:, -1].contiguous().to(_dev())
        single = _call(wq, kernel, **dict(mods))
        torch.testing.assert_close(got[:, -1].float(), single.float(), atol=2e-3, rtol=2e-2)


@pytest.mark.parametrize("sinks", [False, True])
def test_query_block_longer_than_the_context(oracle, sinks):
    """Leading query tokens that lie before key 0 see nothing: zeros, never NaN."""
    QL = 4
    w = W.make_test_shaped(batch_size=3, nheads=8, nheads_k=2, d=128, seqlen_k=700, varlen=True, has_sinks=sinks,
                           seed=17)
    w.context_lens[0] = 2
    w.context_lens[1] = 1
    g = torch.Generator().manual_seed(8)
    query4 = torch.randn(3, QL, 8, 128, generator=g).to(torch.float16)
    ref = oracle.attention_ref(query4, w.key_cache, w.value_cache, w.block_tables, w.context_lens, scale=w.scale,
                               block_size=w.block_size, kv_strides=w.kv_strides(), num_kv_heads=w.num_kv_heads,
                               sinks=w.sinks, want_f32=True)[1]
    assert (ref[0, :2] == 0).all() and (ref[1, :3] == 0).all()
    wd = w.to(_dev())
    for kernel in ("loop", "reduce"):
        got = _call_multi(wd, query4.to(_dev()), kernel).float().cpu()
        assert (got[0, :2] == 0).all() and (got[1, :3] == 0).all(), kernel
        assert_close_to_reference(got, ref)


def test_query_tokens_head_major_e4m3(oracle):
    """The measured pool layout and the second FP8 format with several query tokens."""
    w = W.make_config(3, num_seqs=4, pool_blocks=400, lens=[1500, 513, 16, 1024], fp8_dtype=torch.float8_e4m3fn)
    H = w.query.shape[1]
    QL = 8
    g = torch.Generator().manual_seed(9)
    query4 = torch.randn(4, QL, H, 128, generator=g).to(torch.float16)
    ref = oracle.attention_ref(query4, w.key_cache, w.value_cache, w.block_tables, w.context_lens, scale=w.scale,
                               block_size=w.block_size, kv_strides=w.kv_strides(), num_kv_heads=w.num_kv_heads,
                               fp8_scale=w.fp8_scale, want_f32=True)[1]
    wd = w.to(_dev())
    for kernel in ("fp8_loop", "fp8_reduce"):
        got = _call_multi(wd, query4.to(_dev()), kernel).float().cpu()
        assert_close_to_reference(got, ref, kernel)


def test_extended_instances_in_every_scheduling_form(oracle):
    """Modifiers + two query tokens on a batch that the persistent kernels take whole (120
    sequences, several items per work-group, empty sequences in between), on one they take as
    sub-batches (300 sequences) and on one left to the grid form (a table of 2^24 tokens per
    sequence)."""
    for S, seed, wide in ((120, 31, False), (300, 32, False), (9, 33, True)):
        gen = torch.Generator().manual_seed(seed)
        lens = torch.randint(1, 1500, (S,), generator=gen)
        lens[::9] = 0
        lens[1] = 1                                    # shorter than the query block
        w = W.make_config(0, num_seqs=S, pool_blocks=S * 94, lens=lens.tolist())     # D 64, G 1
        w.partition_size = 256
        w.sinks = torch.linspace(-2, 2, w.num_heads).to(w.query.dtype)
        if wide:
            table = torch.zeros((S, (1 << 24) // w.block_size), dtype=torch.int32)
            table[:, :w.block_tables.shape[1]] = w.block_tables
            w.block_tables = table
        H = w.query.shape[1]
        QL = 2
        query4 = torch.randn(S, QL, H, 64, generator=gen).to(torch.float16)
        alibi = torch.linspace(0.001, 0.03, H)
        okw = dict(alibi_slopes=alibi, softcap=20.0, window_left=400)
        ref = oracle.attention_ref(query4, w.key_cache, w.value_cache, w.block_tables, w.context_lens, scale=w.scale,
                                   block_size=w.block_size, kv_strides=w.kv_strides(), num_kv_heads=w.num_kv_heads,
                                   sinks=w.sinks, want_f32=True, **okw)[1]
        wd = w.to(_dev())
        mods = dict(alibi_slopes=alibi.to(_dev()), softcap=20.0, apply_alibi=True, apply_softcap=True, window_left=400)
        live = lens > 0
        for kernel in ("loop", "reduce"):
            got = _call_multi(wd, query4.to(_dev()), kernel, **dict(mods)).float().cpu()
            assert (got[~live] == 0).all(), (S, kernel)          # empty sequences: rows untouched
            assert_close_to_reference(got[live], ref[live], f"S={S} {kernel}")


@pytest.mark.parametrize("QL,nheads,nheads_k", [(4, 16, 2), (7, 8, 2), (33, 2, 2), (3, 16, 1)])
@pytest.mark.parametrize("fp8", [False, True])
def test_more_query_tokens_than_the_mfma_columns_hold(oracle, QL, nheads, nheads_k, fp8):
    """QL x (heads per kv head) beyond 16: the call runs as several launches, each covering the
    query tokens that fit the 16 columns (8+8 heads x 2+2 tokens; 4 heads x 4+3 tokens; 16 + 16 + 1
    tokens of one head; 16 heads x 1+1+1 tokens), with a window and ALiBi placed per token."""
    w = W.make_test_shaped(batch_size=3, nheads=nheads, nheads_k=nheads_k, d=128, seqlen_k=1100, varlen=True,
                           has_sinks=True, fp8=fp8, seed=19)
    w.context_lens[0] = QL - 1             # the first query token lies before key 0
    w.context_lens[1] = 512 + 2
    g = torch.Generator().manual_seed(5)
    query4 = torch.randn(3, QL, nheads, 128, generator=g).to(torch.float16)
    alibi = torch.linspace(0.002, 0.02, nheads)
    ref = oracle.attention_ref(query4, w.key_cache, w.value_cache, w.block_tables, w.context_lens, scale=w.scale,
                               block_size=w.block_size, kv_strides=w.kv_strides(), num_kv_heads=w.num_kv_heads,
                               sinks=w.sinks, fp8_scale=w.fp8_scale, want_f32=True, alibi_slopes=alibi,
                               window_left=300)[1]
    wd = w.to(_dev())
    for kernel in (("fp8_loop", "fp8_reduce") if fp8 else ("loop", "reduce")):
        got = _call_multi(wd, query4.to(_dev()), kernel, alibi_slopes=alibi.to(_dev()), apply_alibi=True,
                          window_left=300).float().cpu()
        assert torch.isfinite(got).all(), kernel
        assert_close_to_reference(got, ref, f"{kernel} QL={QL}")


@pytest.mark.parametrize("fp8,qdtype,block_scales", [(False, torch.float16, False), (True, torch.bfloat16, False),
                                                      (True, torch.float16, True)])
def test_two_tile_kernels_at_the_edges_of_their_item_lists(oracle, fp8, qdtype, block_scales):
    """Two column tiles (2 heads x 16 tokens) over 100 sequences -- more than the 64 a wavefront's
    lanes hold at once -- whose lengths give a wavefront every number of chunks from none to a few
    more than the steady loop needs: 0, less than the query block, 1 .. 5 chunks of 32 tokens per
    wavefront with and without a ragged end, on and one past partition and chunk boundaries.  With
    soft-capping, a window and sinks; with per-block FP8 scales in the third case.  Both paths."""
    S, QL, H, Hk, D = 100, 16, 4, 2, 128
    edge = [0, 5, 16, 17, 31, 32, 33, 127, 128, 129, 160, 255, 256, 257, 384, 385, 500, 511, 512, 513, 640, 641, 700,
            768, 769, 896, 1000, 1023, 1024, 1025, 1100]
    w = W.make_test_shaped(batch_size=S, nheads=H, nheads_k=Hk, d=D, seqlen_k=1100, varlen=False, has_sinks=True,
                           fp8=fp8, block_size=16, seed=23, dtype=qdtype)
    w.context_lens = torch.tensor([edge[(7 * s) % len(edge)] for s in range(S)], dtype=torch.int32)
    w.sinks = torch.linspace(-2, 2, H).to(qdtype)
    g = torch.Generator().manual_seed(9)
    query4 = torch.randn(S, QL, H, D, generator=g).to(qdtype)
    kw, okw = {}, {}
    if block_scales:
        NB = w.key_cache.shape[0]
        ks = (torch.rand(NB, Hk, generator=g) * 1.5 + 0.5).float()
        vs = (torch.rand(NB, Hk, generator=g) * 1.5 + 0.5).float()
        okw = dict(k_scales=ks, v_scales=vs)
        kw = dict(k_scales=ks.to(_dev()), v_scales=vs.to(_dev()))
    ref = oracle.attention_ref(query4, w.key_cache, w.value_cache, w.block_tables, w.context_lens, scale=w.scale,
                               block_size=w.block_size, kv_strides=w.kv_strides(), num_kv_heads=w.num_kv_heads,
                               sinks=w.sinks, fp8_scale=w.fp8_scale, want_f32=True, softcap=15.0, window_left=600,
                               **okw)[1]
    wd = w.to(_dev())
    live = w.context_lens > 0
    for kernel in (("fp8_loop", "fp8_reduce") if fp8 else ("loop", "reduce")):
        got = _call_multi(wd, query4.to(_dev()), kernel, softcap=15.0, apply_softcap=True, window_left=600,
                          **kw).float().cpu()
        assert torch.isfinite(got).all(), kernel
        assert (got[~live] == 0).all(), kernel          # empty sequences: rows untouched
        assert_close_to_reference(got[live], ref[live], f"{kernel} fp8={fp8} block_scales={block_scales}")


@pytest.mark.parametrize("cache", ["e5m2", "fp16_head_size_64"])
def test_two_tile_kernels_with_two_kv_heads_per_work_group(oracle, cache):
    """Pools in upstream's layout with token rows of 128 bytes and enough pairs of kv heads to give
    every compute unit one: the two-tile kernels of both paths then hand a work-group two adjacent
    kv heads, two wavefronts each.  280 pairs, two column tiles (2 heads x 16 tokens), lengths from
    empty to three partitions, a window, ALiBi and sinks."""
    fp8 = cache == "e5m2"
    D = 128 if fp8 else 64
    S, QL, H, Hk = 140, 16, 8, 4
    qdtype = torch.bfloat16 if fp8 else torch.float16
    w = W.make_test_shaped(batch_size=S, nheads=H, nheads_k=Hk, d=D, seqlen_k=700, varlen=False, has_sinks=True,
                           fp8=fp8, block_size=16, seed=31, dtype=qdtype)
    g = torch.Generator().manual_seed(19)
    w.context_lens = torch.randint(1, 701, (S,), generator=g).to(torch.int32)
    w.context_lens[3], w.context_lens[4], w.context_lens[11] = 0, 7, 700
    w.sinks = torch.linspace(-2, 2, H).to(qdtype)
    query4 = torch.randn(S, QL, H, D, generator=g).to(qdtype)
    alibi = torch.linspace(0.001, 0.02, H)
    ref = oracle.attention_ref(query4, w.key_cache, w.value_cache, w.block_tables, w.context_lens, scale=w.scale,
                               block_size=w.block_size, kv_strides=w.kv_strides(), num_kv_heads=w.num_kv_heads,
                               sinks=w.sinks, fp8_scale=w.fp8_scale, want_f32=True, alibi_slopes=alibi,
                               window_left=300)[1]
    wd = w.to(_dev())
    live = w.context_lens > 0
    for kernel in (("fp8_loop", "fp8_reduce") if fp8 else ("loop", "reduce")):
        got = _call_multi(wd, query4.to(_dev()), kernel, alibi_slopes=alibi.to(_dev()), apply_alibi=True,
                          window_left=300).float().cpu()
        assert torch.isfinite(got).all(), kernel
        assert (got[~live] == 0).all(), kernel
        assert_close_to_reference(got[live], ref[live], f"{kernel} {cache}")


@pytest.mark.parametrize("index,QL", [(4, 4), (1, 32), (2, 8)])
def test_full_size_query_blocks_with_modifiers(oracle, index, QL):
    """The measured configurations at full size with a query block of two column tiles (G x QL =
    32 columns), a local window and ALiBi, through the loop and the split entry: whole output
    against the oracle, and loop == split within two 16-bit roundings."""
    dev = _dev()
    wd = W.make_config(index, device=dev, pools_on_device=True)
    w = wd.to("cpu")
    S, H, D = w.query.shape
    g = torch.Generator().manual_seed(40 + index)
    query4 = torch.randn(S, QL, H, D, generator=g).to(w.query.dtype)
    alibi = torch.linspace(0.0005, 0.01, H)
    window = int(w.context_lens.max()) // 2
    ref = oracle.attention_ref(query4, w.key_cache, w.value_cache, w.block_tables, w.context_lens, scale=w.scale,
                               block_size=w.block_size, kv_strides=w.kv_strides(), num_kv_heads=w.num_kv_heads,
                               fp8_scale=w.fp8_scale, want_f32=True, alibi_slopes=alibi, window_left=window)[1]
    outs = {}
    for kernel in (("fp8_loop", "fp8_reduce") if w.is_fp8 else ("loop", "reduce")):
        got = _call_multi(wd, query4.to(dev), kernel, alibi_slopes=alibi.to(dev), apply_alibi=True,
                          window_left=window).float().cpu()
        assert_close_to_reference(got, ref, f"config {index} {kernel}")
        outs[kernel] = got
    a, b = outs.values()
    ulps = 2.0 ** (-7 if w.query.dtype == torch.bfloat16 else -10)
    assert (a - b).abs().max().item() <= ulps * ref.abs().max().item() + 1e-5


def test_more_rows_than_one_grid_dimension_holds(oracle):
    """2100 sequences x 32 query tokens = 67200 rows of out and scratch: more than the 65535 a
    second grid dimension could address; both entry points, tiny contexts."""
    S, QL = 2100, 32
    gen = torch.Generator().manual_seed(77)
    lens = torch.randint(1, 40, (S,), generator=gen)
    w = W.make_config(0, num_seqs=S, pool_blocks=S * 3, lens=lens.tolist())      # D 64, G 1, 8 heads
    H = w.query.shape[1]
    query4 = torch.randn(S, QL, H, 64, generator=gen).to(torch.float16)
    ref = oracle.attention_ref(query4, w.key_cache, w.value_cache, w.block_tables, w.context_lens, scale=w.scale,
                               block_size=w.block_size, kv_strides=w.kv_strides(), num_kv_heads=w.num_kv_heads,
                               want_f32=True)[1]
    wd = w.to(_dev())
    for kernel in ("loop", "reduce"):
        got = _call_multi(wd, query4.to(_dev()), kernel).float().cpu()
        assert_close_to_reference(got, ref, kernel)
