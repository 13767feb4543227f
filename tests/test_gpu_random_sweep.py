"""Seeded random sweep over shapes, dtypes, layouts and optional features: every case through
the loop and the split entry point of its cache type, against the oracle.  Small cases (the
oracle takes milliseconds each), many of them: this is where odd combinations meet -- a window
that ends inside the first partition of a sequence with a sink, a query block longer than a
context next to an empty sequence, a group of 5 heads with 3 query tokens in two launches."""
import random

import pytest
import torch

from flash_attention_factory_amd import lib, workloads as W

pytestmark = pytest.mark.gpu
ATOL = RTOL = 1e-2
CASES_PER_SEED = 12


def _dev():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch.device("cuda:0")


def _draw_case(rng):
    D = rng.choice([64, 128])
    Hk = rng.choice([1, 2, 4, 8])
    G = rng.choice([1, 1, 2, 3, 4, 5, 7, 8, 16])
    B = rng.choice([16, 16, 32, 64, 128])
    S = rng.randint(1, 7)
    cache = rng.choice(["16", "16", "e5m2", "e4m3"])
    qdtype = rng.choice([torch.float16, torch.bfloat16])
    layout = rng.choice([W.TOKEN_MAJOR, W.HEAD_MAJOR])
    psize = rng.choice([64, 128, 256, 512])
    top = rng.choice([40, 300, 1200, 3000])
    lens = []
    for _ in range(S):
        kind = rng.random()
        if kind < 0.1:
            lens.append(0)
        elif kind < 0.25:
            lens.append(rng.randint(1, 5))
        elif kind < 0.45:
            lens.append(max(1, min(top, psize * rng.randint(1, 4) + rng.choice([-1, 0, 1]))))
        else:
            lens.append(rng.randint(1, top))
    if max(lens) == 0:
        lens[0] = rng.randint(1, top)
    feats = {}
    if rng.random() < 0.6:
        if rng.random() < 0.5:
            feats["window_left"] = rng.choice([0, 1, 17, 200, 1000, 5000])
        if rng.random() < 0.4:
            feats["alibi"] = True
        if rng.random() < 0.3:
            feats["softcap"] = rng.choice([0.5, 5.0, 30.0])
        if rng.random() < 0.5:
            feats["query_len"] = rng.choice([2, 3, 5])
        if cache != "16" and rng.random() < 0.5:
            feats["scales"] = rng.choice(["head", "block"])
    fp8_scale = rng.choice([1.0, 1.0, 0.5, 2.0]) if cache != "16" and "scales" not in feats else 1.0
    return dict(D=D, Hk=Hk, G=G, B=B, S=S, cache=cache, qdtype=qdtype, layout=layout, psize=psize, lens=lens,
                sinks=rng.random() < 0.5, feats=feats, fp8_scale=fp8_scale, seed=rng.randint(0, 1 << 30))


def _draw_large_case(rng):
    """Batches of more (sequence, kv head) items than the GPU has compute units, short contexts:
    where the kernels rank more than 64 sequences, deal several items to a work-group, put two or
    three work-groups on a unit and give a work-group two kv heads (pools in upstream's layout with
    128-byte token rows)."""
    D, cache = rng.choice([(128, "e5m2"), (128, "e4m3"), (64, "16"), (128, "16"), (64, "e5m2")])
    Hk = rng.choice([8, 16, 32])
    G = rng.choice([1, 1, 2, 4, 5])
    S = rng.choice([rng.randint(17, 64), rng.randint(65, 128), rng.randint(129, 256), rng.randint(257, 300)])
    psize = rng.choice([256, 512])
    budget = (24 << 20) // (Hk * D)  # tokens in the pools: the oracle and the random draw stay quick
    top = min(rng.choice([90, 400, 1500]), max(30, 2 * budget // S))
    lens = []
    for _ in range(S):
        kind = rng.random()
        if kind < 0.05:
            lens.append(0)
        elif kind < 0.15:
            lens.append(rng.randint(1, 20))
        elif kind < 0.25:
            lens.append(max(1, min(top, psize * rng.randint(1, 3) + rng.choice([-1, 0, 1]))))
        else:
            lens.append(rng.randint(1, top))
    if rng.random() < 0.3:   # one sequence far longer than the others
        lens[rng.randrange(S)] = rng.randint(budget // 4, budget // 2)
    feats = {}
    if rng.random() < 0.4:
        if rng.random() < 0.5:
            feats["window_left"] = rng.choice([17, 200, 1000])
        if rng.random() < 0.4:
            feats["alibi"] = True
        if rng.random() < 0.5 and S * G * Hk <= 8192:
            feats["query_len"] = rng.choice([2, 3])
        if cache != "16" and rng.random() < 0.4:
            feats["scales"] = rng.choice(["head", "block"])
    return dict(D=D, Hk=Hk, G=G, B=rng.choice([16, 16, 64]), S=S, cache=cache,
                qdtype=rng.choice([torch.float16, torch.bfloat16]),
                layout=rng.choice([W.TOKEN_MAJOR, W.TOKEN_MAJOR, W.HEAD_MAJOR]), psize=psize, lens=lens,
                sinks=rng.random() < 0.5, feats=feats, fp8_scale=1.0, seed=rng.randint(0, 1 << 30), compact=True)


def _compact_pools(w, c, fp8_dtype):
    """Pools of just the blocks the lengths need (make_test_shaped sizes them for the longest
    length times the batch), dealt to the sequences in random order."""
    gen = torch.Generator().manual_seed(c["seed"] + 2)
    B, Hk, D = c["B"], c["Hk"], c["D"]
    NB = sum(-(-n // B) for n in c["lens"]) + 3
    w.block_tables = W._deal_block_tables(c["lens"], B, torch.randperm(NB, generator=gen).to(torch.int32))
    shape = (NB, B, Hk, D) if c["layout"] == W.TOKEN_MAJOR else (NB, Hk, B, D)
    w.key_cache = W._randn16(shape, gen, c["qdtype"])
    w.value_cache = W._randn16(shape, gen, c["qdtype"])
    if c["cache"] != "16":
        w.key_cache, w.value_cache = w.key_cache.to(fp8_dtype), w.value_cache.to(fp8_dtype)


def _run_case(oracle, c):
    dev = _dev()
    fp8 = c["cache"] != "16"
    fp8_dtype = torch.float8_e4m3fn if c["cache"] == "e4m3" else torch.float8_e5m2
    w = W.make_test_shaped(batch_size=c["S"], nheads=c["Hk"] * c["G"], nheads_k=c["Hk"], d=c["D"],
                           seqlen_k=c["B"] if c.get("compact") else max(c["lens"]), varlen=False, has_sinks=c["sinks"],
                           fp8=fp8, block_size=c["B"], seed=c["seed"], dtype=c["qdtype"], layout=c["layout"],
                           fp8_dtype=fp8_dtype)
    if c.get("compact"):
        _compact_pools(w, c, fp8_dtype)
    w.context_lens = torch.tensor(c["lens"], dtype=torch.int32)
    w.partition_size = c["psize"]
    w.fp8_scale = c["fp8_scale"]
    if c["sinks"]:
        w.sinks = torch.linspace(-3, 3, w.num_heads).to(w.query.dtype)
    g = torch.Generator().manual_seed(c["seed"] + 1)
    H, Hk, D = w.num_heads, w.num_kv_heads, c["D"]
    f = c["feats"]
    QL = f.get("query_len", 1)
    query = w.query if QL == 1 else torch.randn(c["S"], QL, H, D, generator=g).to(c["qdtype"])
    okw, kw = {}, {}
    if f.get("alibi"):
        okw["alibi_slopes"] = (torch.rand(H, generator=g) * 0.05).float()
        kw["apply_alibi"] = True
    if "softcap" in f:
        okw["softcap"] = f["softcap"]
        kw["apply_softcap"] = True
    if "window_left" in f:
        okw["window_left"] = kw["window_left"] = f["window_left"]
    if "scales" in f:
        shape = (w.key_cache.shape[0], Hk) if f["scales"] == "block" else (Hk,)
        okw["k_scales"] = (torch.rand(shape, generator=g) * 2 + 0.1).float()
        okw["v_scales"] = (torch.rand(shape, generator=g) * 2 + 0.1).float()
        kw["k_scales"], kw["v_scales"] = okw["k_scales"].to(dev), okw["v_scales"].to(dev)
    ref = oracle.attention_ref(query, w.key_cache, w.value_cache, w.block_tables, w.context_lens, scale=w.scale,
                               block_size=w.block_size, kv_strides=w.kv_strides(), num_kv_heads=Hk, sinks=w.sinks,
                               fp8_scale=w.fp8_scale, want_f32=True, **okw)[1]
    live = w.context_lens > 0
    unit = ref[live].abs().max().clamp_min(1e-6)
    wd = w.to(dev)
    q = query.to(dev)
    rows = c["S"] * QL
    NP = max(1, -(-max(c["lens"]) // c["psize"]))
    alibi = okw["alibi_slopes"].to(dev) if "alibi_slopes" in okw else None
    kv, vv = (wd.key_cache.permute(0, 2, 1, 3), wd.value_cache.permute(0, 2, 1, 3)) if w.layout == W.HEAD_MAJOR \
        else (wd.key_cache, wd.value_cache)
    kernels = ("fp8_loop", "fp8_reduce") if fp8 else ("loop", "reduce")
    if c.get("dot_schedules"):
        # the loop kernels without the matrix cores (schedules FA_SCHEDULE_GRID_VALU, FA_SCHEDULE_VALU)
        kernels = tuple((kernels[0], sched) for sched in c["dot_schedules"])
    for kernel in kernels:
        if isinstance(kernel, tuple):
            kernel, kw["schedule"] = kernel
        ml = torch.full((rows, H, NP), float("nan"), dtype=torch.float32, device=dev)
        es = torch.full_like(ml, float("nan"))
        tmp = torch.full((rows, H, NP, D), float("nan"), dtype=torch.float32, device=dev)
        out = torch.zeros_like(q)
        head = [ml, es, tmp, out, None, q, kv, vv, wd.block_tables, wd.context_lens, c["G"], w.scale]
        if fp8:
            head.append(w.fp8_scale)
        extra = dict(partition_size=c["psize"]) if "reduce" in kernel else {}
        run = getattr(lib, "paged_attention_" + kernel).run
        times = run(*head, w.block_size, max(c["lens"]), alibi, wd.sinks, okw.get("softcap", 0.0), **extra, **kw)
        torch.cuda.synchronize()
        got = out.float().cpu()
        if "reduce" in kernel and times[1] == 0.0:
            # rows so short that the split entry ran the single-pass kernel: that result is checked below
            # against the one of the split kernels themselves, which then goes on to the oracle
            assert torch.isfinite(got).all(), (kernel, c)
            single = got
            out.zero_()
            times = run(*head, w.block_size, max(c["lens"]), alibi, wd.sinks, okw.get("softcap", 0.0),
                        schedule=3, **extra, **kw)
            torch.cuda.synchronize()
            assert times[1] > 0.0
            got = out.float().cpu()
            torch.testing.assert_close(single[live] / unit, got[live] / unit, atol=ATOL, rtol=RTOL,
                                       msg=lambda m: f"{kernel} single-pass against split kernels {c}: {m}")
        assert torch.isfinite(got).all(), (kernel, c)
        assert (got[~live] == 0).all(), (kernel, c)          # empty sequences: rows untouched
        torch.testing.assert_close(got[live] / unit, ref[live] / unit, atol=ATOL, rtol=RTOL,
                                   msg=lambda m: f"{kernel} {c}: {m}")


@pytest.mark.parametrize("seed", range(16))
def test_random_cases(oracle, seed):
    rng = random.Random(1000 + seed)
    for _ in range(CASES_PER_SEED):
        c = _draw_case(rng)
        print(c, flush=True)
        _run_case(oracle, c)


@pytest.mark.parametrize("seed", range(4))
def test_random_single_head_groups_by_dot_products(oracle, seed):
    """The shapes the dot-product kernels take (one query head per kv head, head size 128, fp16 queries, plain
    decode) drawn like the other cases -- cache formats, layouts, block sizes, sinks, scales, empty and tiny
    sequences -- through both of their schedules."""
    rng = random.Random(9000 + seed)
    for k in range(CASES_PER_SEED):
        c = _draw_case(rng)
        c.update(D=128, G=1, qdtype=torch.float16, feats={}, dot_schedules=(4, 5))
        c["Hk"] = rng.choice([1, 2, 8, 32])
        if k % 4 == 3:  # more items than work-groups stay resident, several per work-group
            c["S"] = rng.randint(20, 60)
            c["Hk"] = 32
            c["lens"] = [rng.choice([0, rng.randint(1, 40), rng.randint(1, 700)]) for _ in range(c["S"])]
            c["lens"][0] = max(c["lens"][0], 1)
        print(c, flush=True)
        _run_case(oracle, c)


@pytest.mark.parametrize("seed", range(6))
def test_random_large_batches(oracle, seed):
    rng = random.Random(5000 + seed)
    for _ in range(5):
        c = _draw_large_case(rng)
        print({k: (v if k != "lens" else (len(v), max(v))) for k, v in c.items()}, flush=True)
        _run_case(oracle, c)
