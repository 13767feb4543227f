"""Which kernels a call of the split path runs is decided on the host, from the call's arguments alone
(fa_paged_attention_reduce_plan; upstream's launcher has one form, launch_kernels_reduce.h:18-78).
The rule that turns a call into the single-pass kernel rests on an upper bound of the rows' lengths
that the host can prove -- max_context_len, the block table's width, the scratch arrays' capacity --
and is checked here without a GPU: on upstream's own perf shapes (test_paged.py:607-631,
test_paged_fp8cache.py:612-636), on the benchmark configurations, and as a property over random shapes."""
import ctypes
import math
import random

import pytest

from flash_attention_factory_amd import _cabi

GRID, SEGMENT, LOOP = _cabi.FA_SPLIT_FORM_GRID, _cabi.FA_SPLIT_FORM_SEGMENT, _cabi.FA_SPLIT_FORM_LOOP
CUS = 256


@pytest.fixture(scope="module")
def L():
    return _cabi.load()


def _plan(L, *, S, H, Hk, D, B, ctx_bound, max_context_len=0, fp8=False, token_major=True, NP=None, P=0,
          pool_blocks=4096, cus=CUS, **options):
    psize = P or (256 if D == 64 else 512)
    sh = _cabi.Shape()
    sh.num_seqs, sh.num_heads, sh.num_kv_heads, sh.head_size, sh.block_size = S, H, Hk, D, B
    sh.max_blocks_per_seq = math.ceil(ctx_bound / B)
    sh.max_num_partitions = NP if NP is not None else math.ceil(ctx_bound / psize)
    sh.partition_size = P
    if token_major:
        sh.kv_block_stride, sh.kv_token_stride, sh.kv_head_stride = B * Hk * D, Hk * D, D
    else:
        sh.kv_block_stride, sh.kv_token_stride, sh.kv_head_stride = Hk * B * D, D, B * D
    sh.q_dtype, sh.num_pool_blocks = _cabi.FA_DTYPE_F16, pool_blocks
    op = _cabi.Options()
    for k, v in options.items():
        setattr(op, k, v)
    plan = _cabi.SplitPlan()
    rc = L.fa_paged_attention_reduce_plan(ctypes.byref(sh), ctypes.byref(op), max_context_len, int(fp8), cus, ctypes.byref(plan))
    assert rc == _cabi.FA_OK, L.fa_last_error()
    assert plan.compute_units == cus and plan.work_groups == 0  # made without a device
    return plan.form


def test_upstreams_perf_shapes_run_as_the_single_pass_kernel(L):
    # batch 64, 1500 keys, head size 64, block 64, 64 (FP8: 40) query heads over 8 kv heads; upstream
    # passes seqlen_k as max_context_len and sizes the scratch for it
    recipe = dict(S=64, Hk=8, D=64, B=64, ctx_bound=1500)
    assert _plan(L, H=64, max_context_len=1500, **recipe) == LOOP
    assert _plan(L, H=40, max_context_len=1500, fp8=True, **recipe) == LOOP
    # without max_context_len the block table's width (24 blocks of 64) is the bound: still short
    assert _plan(L, H=64, **recipe) == LOOP
    # half the sequences: no row for every compute unit, and 1536 keys are worth splitting then
    assert _plan(L, H=64, max_context_len=1500, **dict(recipe, S=32)) == SEGMENT
    # a caller who asks for upstream's decomposition, or fixes the segment length, gets the split kernels
    assert _plan(L, H=64, max_context_len=1500, schedule=_cabi.FA_SCHEDULE_GRID, **recipe) == GRID
    assert _plan(L, H=64, max_context_len=1500, segment_partitions=2, **recipe) == SEGMENT
    assert _plan(L, H=64, max_context_len=1500, schedule=_cabi.FA_SCHEDULE_SPLIT, **recipe) == SEGMENT


def test_benchmark_configurations(L):
    # long contexts and the serving mix are split; the Llama-7B-shaped batch through the split entry is not
    assert _plan(L, S=8, H=32, Hk=8, D=128, B=16, ctx_bound=32768, token_major=False, pool_blocks=16384) == SEGMENT
    assert _plan(L, S=128, H=64, Hk=8, D=128, B=16, ctx_bound=32768, fp8=True, token_major=False, pool_blocks=65536) == SEGMENT
    assert _plan(L, S=32, H=32, Hk=32, D=128, B=16, ctx_bound=2048, token_major=False) == LOOP
    assert _plan(L, S=4, H=8, Hk=8, D=64, B=16, ctx_bound=256, token_major=False, pool_blocks=128) == LOOP


def test_what_the_bound_rests_on(L):
    base = dict(S=64, H=32, Hk=8, D=128, B=16)
    # the table is wide, max_context_len says the rows are short
    assert _plan(L, ctx_bound=32768, max_context_len=1000, **base) == LOOP
    assert _plan(L, ctx_bound=32768, max_context_len=0, **base) == SEGMENT
    assert _plan(L, ctx_bound=32768, max_context_len=2048, **base) == LOOP      # 512 rows for 256 units
    assert _plan(L, ctx_bound=32768, max_context_len=2049, **base) == SEGMENT
    assert _plan(L, ctx_bound=32768, max_context_len=2048, **dict(base, S=16)) == SEGMENT  # 128 rows
    assert _plan(L, ctx_bound=32768, max_context_len=1024, **dict(base, S=1)) == LOOP
    assert _plan(L, ctx_bound=32768, max_context_len=1025, **dict(base, S=1)) == SEGMENT
    # scratch that cannot hold what the table could: the split kernels cut such rows, so they keep the call
    assert _plan(L, ctx_bound=1024, NP=1, **base) == SEGMENT
    assert _plan(L, ctx_bound=1024, NP=2, **base) == LOOP
    # no pool size: no persistent kernel of either kind
    assert _plan(L, ctx_bound=1024, pool_blocks=0, **base) == GRID
    # more sequences than the single-pass kernel ranks in one launch
    assert _plan(L, ctx_bound=1024, **dict(base, S=129)) == SEGMENT
    # pairs (FP8, head size 64) and teams (128-byte rows in upstream's layout) of kv heads count once
    assert _plan(L, ctx_bound=2048, **dict(base, S=32)) == LOOP                       # 256 rows
    assert _plan(L, ctx_bound=2048, fp8=True, **dict(base, S=32)) == SEGMENT          # 128 teams
    assert _plan(L, ctx_bound=2048, fp8=True, token_major=False, **dict(base, S=32)) == LOOP


def test_loop_form_implies_the_proven_bound(L):
    rng = random.Random(0)
    seen = {GRID: 0, SEGMENT: 0, LOOP: 0}
    for _ in range(400):
        D = rng.choice((64, 128))
        B = rng.choice((16, 32, 64))
        Hk = rng.choice((1, 2, 4, 8, 32))
        G = rng.choice((1, 2, 4, 8))
        S = rng.choice((1, 2, 8, 32, 64, 128, 200))
        fp8 = rng.random() < 0.5
        token_major = rng.random() < 0.5
        psize = 256 if D == 64 else 512
        ctx_bound = rng.choice((300, 1000, 1024, 1500, 2048, 2100, 5000))
        max_ctx = rng.choice((0, 0, 700, 1024, 1500, 2048, 4000))
        max_ctx = min(max_ctx, math.ceil(ctx_bound / B) * B)
        NP = math.ceil(ctx_bound / psize) + rng.choice((-1, 0, 0, 1))
        if NP < 1 or (max_ctx > 0 and NP * psize < max_ctx):
            continue
        cus = rng.choice((64, 256, 304))
        schedule = rng.choice((0, 0, 0, 1))
        form = _plan(L, S=S, H=Hk * G, Hk=Hk, D=D, B=B, ctx_bound=ctx_bound, max_context_len=max_ctx, fp8=fp8,
                     token_major=token_major, NP=NP, cus=cus, schedule=schedule)
        seen[form] += 1
        table = math.ceil(ctx_bound / B) * B
        bound = min(max_ctx, table) if max_ctx > 0 else table
        if form == LOOP:
            assert schedule == 0 and S <= 128
            assert bound <= NP * psize          # the scratch arrays could have held every row
            rows = S * Hk
            paired = fp8 and D == 64 and token_major and Hk % 2 == 0 and 2 * G <= 16
            teams = not paired and D * (1 if fp8 else 2) == 128 and token_major and Hk % 2 == 0
            if paired or teams:
                rows //= 2
            assert bound <= 1024 or (bound <= 2048 and rows >= cus)
        if schedule == 1:
            assert form == GRID
    assert all(n > 20 for n in seen.values()), seen


def test_plan_argument_checks(L):
    sh = _cabi.Shape()
    plan = _cabi.SplitPlan()
    assert L.fa_paged_attention_reduce_plan(None, None, 0, 0, CUS, ctypes.byref(plan)) == _cabi.FA_ERR_NULL_POINTER
    assert L.fa_paged_attention_reduce_plan(ctypes.byref(sh), None, 0, 0, CUS, None) == _cabi.FA_ERR_NULL_POINTER
    assert L.fa_paged_attention_reduce_plan(ctypes.byref(sh), None, 0, 0, CUS, ctypes.byref(plan)) != _cabi.FA_OK  # empty shape
    plan.struct_size = 8
    sh.struct_size = ctypes.sizeof(sh)
    rc = L.fa_paged_attention_reduce_plan(ctypes.byref(sh), None, 0, 0, CUS, ctypes.byref(plan))
    assert rc == _cabi.FA_ERR_BAD_SHAPE and b"plan.struct_size" in L.fa_last_error()
