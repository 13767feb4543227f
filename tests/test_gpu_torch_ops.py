"""The stream-ordered torch.library operators: same results as the timed ``lib.*.run`` calls,
and a HIP graph holding a whole decode step (KV-cache append, FP8 loop decode, FP8 split
decode) replays correctly.  The graph is replayed several times with the program's own eager
work and synchronisations between the replays, and every replay is checked against eager."""
import pytest
import torch

from flash_attention_factory_amd import runner, workloads as W

pytestmark = pytest.mark.gpu


def _dev():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch.device("cuda:0")


def _views(w, kc, vc):
    """[blocks, block_size, kv_heads, head_size] views of pools stored in the workload's layout."""
    if w.layout == W.HEAD_MAJOR:
        return kc.permute(0, 2, 1, 3), vc.permute(0, 2, 1, 3)
    return kc, vc


@pytest.mark.parametrize("index", [0, 3])
def test_operators_match_the_run_functions(index):
    from flash_attention_factory_amd import torch_ops  # noqa: F401  (registers the operators)
    dev = _dev()
    w = W.make_config(index, num_seqs=4, pool_blocks=300, lens=[100, 700, 33, 512]).to(dev)
    fp8 = w.is_fp8
    kv, vv = _views(w, w.key_cache, w.value_cache)
    ref_loop = runner.alloc_buffers(w)
    runner.run_workload(w, "fp8_loop" if fp8 else "loop", ref_loop)
    ref_split = runner.alloc_buffers(w)
    runner.run_workload(w, "fp8_reduce" if fp8 else "reduce", ref_split)
    got = runner.alloc_buffers(w)
    ops = torch.ops.fa_amd
    if fp8:
        ops.paged_attention_fp8_loop(got.out, w.query, kv, vv, w.block_tables, w.context_lens, w.scale, w.fp8_scale, w.sinks)
    else:
        ops.paged_attention_loop(got.out, w.query, kv, vv, w.block_tables, w.context_lens, w.scale, w.sinks)
    torch.cuda.synchronize()
    assert torch.equal(got.out, ref_loop.out)
    got.out.zero_()
    if fp8:
        ops.paged_attention_fp8_reduce(got.out, got.exp_sums, got.max_logits, got.tmp_out, w.query, kv, vv,
                                       w.block_tables, w.context_lens, w.scale, w.fp8_scale, w.partition_size, w.sinks)
    else:
        ops.paged_attention_reduce(got.out, got.exp_sums, got.max_logits, got.tmp_out, w.query, kv, vv,
                                   w.block_tables, w.context_lens, w.scale, w.partition_size, w.sinks)
    torch.cuda.synchronize()
    assert torch.equal(got.out, ref_split.out)


def test_decode_step_in_a_hip_graph():
    from flash_attention_factory_amd import torch_ops  # noqa: F401
    dev = _dev()
    ops = torch.ops.fa_amd
    w = W.make_config(3, num_seqs=4, pool_blocks=300, lens=[100, 700, 33, 512]).to(dev)   # E5M2 pools, fp16 queries
    S, H, D = w.query.shape
    Hk, B = w.num_kv_heads, w.block_size
    gen = torch.Generator(device=dev).manual_seed(1)

    def fresh_state():
        kc, vc = w.key_cache.clone(), w.value_cache.clone()
        bufs_a, bufs_b = runner.alloc_buffers(w), runner.alloc_buffers(w)
        return dict(kc=kc, vc=vc, views=_views(w, kc, vc), ctx=w.context_lens.clone(), query=w.query.clone(),
                    key=torch.zeros((S, Hk, D), dtype=torch.float16, device=dev),
                    value=torch.zeros((S, Hk, D), dtype=torch.float16, device=dev),
                    slots=torch.zeros(S, dtype=torch.int64, device=dev), loop=bufs_a, split=bufs_b)

    def step(st):  # append one token per sequence, then decode it twice (loop and split kernels)
        ops.kv_cache_write(st["key"], st["value"], st["views"][0], st["views"][1], st["slots"], 1.0)
        ops.paged_attention_fp8_loop(st["loop"].out, st["query"], st["views"][0], st["views"][1], w.block_tables,
                                     st["ctx"], w.scale, 1.0, None)
        ops.paged_attention_fp8_reduce(st["split"].out, st["split"].exp_sums, st["split"].max_logits,
                                       st["split"].tmp_out, st["query"], st["views"][0], st["views"][1],
                                       w.block_tables, st["ctx"], w.scale, 1.0, w.partition_size, None)

    def new_inputs(st):  # in place, so that a graph holding these tensors sees them
        old = st["ctx"].clone()
        st["slots"].copy_(w.block_tables.gather(1, (old // B).long()[:, None]).squeeze(1).long() * B + old % B)
        st["ctx"].add_(1)
        st["key"].copy_(torch.randn((S, Hk, D), generator=gen, device=dev).half())
        st["value"].copy_(torch.randn((S, Hk, D), generator=gen, device=dev).half())
        st["query"].copy_(torch.randn((S, H, D), generator=gen, device=dev).half())

    eager, graphed = fresh_state(), fresh_state()
    # warm-up outside the capture (first calls query occupancy and create nothing afterwards)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        warm = fresh_state()
        step(warm)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(graphed)
    for replay in range(4):
        gen.manual_seed(100 + replay)
        new_inputs(eager)
        gen.manual_seed(100 + replay)
        new_inputs(graphed)
        step(eager)
        scratch = torch.randn(1 << 20, device=dev).sum()   # the program's own eager work between replays
        graph.replay()
        torch.cuda.synchronize()
        assert torch.isfinite(scratch)
        assert torch.equal(graphed["loop"].out, eager["loop"].out), f"loop kernel, replay {replay}"
        assert torch.equal(graphed["split"].out, eager["split"].out), f"split kernels, replay {replay}"
        assert torch.equal(graphed["kc"].view(torch.uint8), eager["kc"].view(torch.uint8)), f"key pool, replay {replay}"
        a, b = eager["loop"].out.float(), eager["split"].out.float()
        assert (a - b).abs().max().item() <= 2.0 ** -9 * a.abs().max().item() + 1e-5


def test_operators_with_modifiers_query_tokens_and_block_scales(oracle):
    """The optional arguments of the operators against the oracle, eagerly and as a HIP graph
    replayed with fresh inputs: window + ALiBi + soft-capping, three query tokens per sequence,
    E4M3 pools with per-block scales."""
    from flash_attention_factory_amd import torch_ops  # noqa: F401
    dev = _dev()
    ops = torch.ops.fa_amd
    w = W.make_test_shaped(batch_size=3, nheads=8, nheads_k=2, d=128, seqlen_k=900, varlen=True, has_sinks=True,
                           fp8=True, block_size=16, seed=81, fp8_dtype=torch.float8_e4m3fn)
    S, H, D, QL = 3, 8, 128, 3
    NB = w.key_cache.shape[0]
    g = torch.Generator().manual_seed(2)
    ks = torch.rand((NB, 2), generator=g) * 2 + 0.2
    vs = torch.rand((NB, 2), generator=g) * 2 + 0.2
    alibi = torch.linspace(0.002, 0.02, H)
    NP = -(-int(w.context_lens.max()) // 512)
    wd = w.to(dev)
    query = torch.zeros((S, QL, H, D), dtype=torch.float16, device=dev)
    out_a, out_b = torch.zeros_like(query), torch.zeros_like(query)
    es = torch.zeros((S * QL, H, NP), dtype=torch.float32, device=dev)
    ml, tmp = torch.zeros_like(es), torch.zeros((S * QL, H, NP, D), dtype=torch.float32, device=dev)
    ks_d, vs_d, alibi_d = ks.to(dev), vs.to(dev), alibi.to(dev)

    def step():
        ops.paged_attention_fp8_loop(out_a, query, wd.key_cache, wd.value_cache, wd.block_tables, wd.context_lens,
                                     w.scale, 1.0, wd.sinks, alibi_d, 15.0, 500, ks_d, vs_d)
        ops.paged_attention_fp8_reduce(out_b, es, ml, tmp, query, wd.key_cache, wd.value_cache, wd.block_tables,
                                       wd.context_lens, w.scale, 1.0, 512, wd.sinks, alibi_d, 15.0, 500, ks_d, vs_d)

    def check(q_cpu, what):
        ref = oracle.attention_ref(q_cpu, w.key_cache, w.value_cache, w.block_tables, w.context_lens, scale=w.scale,
                                   block_size=16, kv_strides=w.kv_strides(), num_kv_heads=2, sinks=w.sinks,
                                   want_f32=True, alibi_slopes=alibi, softcap=15.0, window_left=500,
                                   k_scales=ks, v_scales=vs)[1]
        unit = ref.abs().max()
        for name, out in (("loop", out_a), ("split", out_b)):
            torch.testing.assert_close(out.float().cpu() / unit, ref / unit, atol=1e-2, rtol=1e-2,
                                       msg=lambda m: f"{what} {name}: {m}")

    q0 = torch.randn((S, QL, H, D), generator=g).to(torch.float16)
    query.copy_(q0)
    step()                      # eager (and warm-up for the capture)
    torch.cuda.synchronize()
    check(q0, "eager")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for it in range(3):
        qn = torch.randn((S, QL, H, D), generator=g).to(torch.float16)
        query.copy_(qn)
        out_a.zero_(); out_b.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        check(qn, f"replay {it}")


def test_reduce_operators_report_scratch_overflow_when_told_the_longest_context():
    """exp_sums.size(-1) partitions must cover the longest context; with max_context_len the operators
    fail instead of attending over a truncated context."""
    from flash_attention_factory_amd import _cabi, torch_ops  # noqa: F401
    dev = _dev()
    ops = torch.ops.fa_amd
    for index in (0, 3):
        w = W.make_config(index, num_seqs=2, pool_blocks=300, lens=[1300, 40]).to(dev)
        kv, vv = _views(w, w.key_cache, w.value_cache)
        bufs = runner.alloc_buffers(w, max_num_partitions=2)  # 2 x 512 tokens < 1300
        args = (bufs.out, bufs.exp_sums, bufs.max_logits, bufs.tmp_out, w.query, kv, vv, w.block_tables, w.context_lens,
                w.scale) + ((w.fp8_scale,) if w.is_fp8 else ()) + (512,)
        op = ops.paged_attention_fp8_reduce if w.is_fp8 else ops.paged_attention_reduce
        with pytest.raises(_cabi.PagedAttentionError, match="partitions"):
            op(*args, max_context_len=1300)
        fits = runner.alloc_buffers(w, max_num_partitions=3)
        op(fits.out, fits.exp_sums, fits.max_logits, fits.tmp_out, *args[4:], max_context_len=1300)
        torch.cuda.synchronize()
        assert torch.isfinite(fits.out.float()).all()
