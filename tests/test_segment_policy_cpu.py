"""The segment-length rule of the split path, replayed on the host (tests/_segment_policy.py follows
csrc/paged_attention_segment_policy.h statement by statement) against the lengths an MI355X chose
for 39 recorded batches (tests/golden/segment_policy_cases.json), and against what the rule is meant
to guarantee.  Upstream has one partial per partition (paged_attention_policy_v2.hpp:28,50); the
rule, and so these vectors, are this library's own."""
import importlib.util
import json
import math
import os
import random

import pytest

import _segment_policy as P

HERE = os.path.dirname(os.path.abspath(__file__))
spec = importlib.util.spec_from_file_location("make_segment_policy_cases",
                                              os.path.join(HERE, "golden", "make_segment_policy_cases.py"))
mk = importlib.util.module_from_spec(spec)
spec.loader.exec_module(mk)

with open(os.path.join(HERE, "golden", "segment_policy_cases.json")) as f:
    CASES = json.load(f)["cases"]


def test_the_recorded_batches_are_the_generators():
    # the fixture holds what batches(seed=0) draws (those that ran in the segment form)
    drawn = {json.dumps(b, sort_keys=True) for b in mk.batches(seed=0)}
    assert len(CASES) >= 35
    for c in CASES:
        b = {k: v for k, v in c.items() if k not in ("plan", "partitions_per_segment")}
        assert json.dumps(b, sort_keys=True) in drawn


@pytest.mark.parametrize("index", range(len(CASES)))
def test_replay_gives_the_length_the_gpu_chose(index):
    c = CASES[index]
    assert mk.replay(c, c["plan"]) == c["partitions_per_segment"]


def test_the_constants_in_the_header_are_the_ones_replayed():
    src = open(os.path.join(os.path.dirname(HERE), "flash_attention_factory_amd", "csrc", "paged_attention_segment_policy.h")).read()
    for literal in ("return 1147;", "563 *", "584 -", "205 *", "379 -", "19 *", "return 360;", "(768 << 10)",
                    "#define FA_SEGMENT_MAX_PARTS 64", "5 * items_all", "n * 20 < (long long)groups * 17"):
        assert literal in src, literal
    assert [P.segment_share_of_load(x) for x in (0, 1024, 1536, 2048, 3072, 4096, 8192, 9000)] == \
        [1147, 1147, 866, 584, 482, 379, 360, 360]


def _args(**kw):
    base = dict(partition_size=512, max_num_partitions=64, max_ctx=32768, num_kv_heads=8, groups=512, cus=256,
                rows_apart=False, partition_bytes=2 * 512 * 256)
    base.update(kw)
    return base


def test_known_choices():
    # eight equal sequences of 40 partitions, 8 kv heads, 512 work-groups on 256 units: 2560 partitions,
    # ten per unit; one segment per unit means 64 rows of 4 segments each
    assert P.partitions_per_segment([40 * 512] * 8, **_args()) == 10
    # a batch in which no row has a second partition has nothing to cut, whatever the length
    m = P.partitions_per_segment([300] * 200, **_args())
    assert len(P.segments_of([300] * 200, m, partition_size=512, max_num_partitions=64, max_ctx=32768)) == 200
    # upstream's FP8 perf shape (pairs of kv heads, 64 KB partitions, 0.4 MB per unit): rows stay whole
    recipe = _args(partition_size=256, max_num_partitions=6, max_ctx=1536, num_kv_heads=4, rows_apart=True,
                   partition_bytes=2 * 256 * 128)
    assert P.partitions_per_segment([1500] * 64, **recipe) >= 6
    # ... and the same rows in a batch of 32 get half a row each: two segments for every unit's worth
    assert P.partitions_per_segment([1500] * 32, **recipe) == 3
    # rows apart with a large load per unit: four segments per unit, as fitted on such batches
    big = _args(rows_apart=True)
    assert P.partitions_per_segment([40 * 512] * 8, **big) == 3  # ten partitions per unit over four (2.5)


def test_even_shares_cover_every_partition_once_and_are_even():
    """Even shares (on request): every live partition of every row lies in exactly one piece, pieces of a
    work-group are contiguous on the tape, and no work-group has many more keys than it aims at (a
    stretch of many short rows holds fewer: every piece has a cost of its own)."""
    rng = random.Random(4)
    for _ in range(120):
        S = rng.choice((1, 5, 40, 128, 256))
        psize = rng.choice((64, 256, 512))
        lens = [rng.choice((0, rng.randint(1, 64 * psize))) for _ in range(S)]
        hk = rng.choice((1, 4, 8))
        cus = 256
        groups = rng.choice((7, cus, 2 * cus))
        kw = dict(partition_size=psize, max_num_partitions=64, max_ctx=64 * psize, num_kv_heads=hk, groups=groups, cus=cus)
        pieces = P.even_shares_pieces(lens, **kw)
        _, parts = P.live_partitions(lens, psize, 64, 64 * psize)
        keys = [0] * groups
        for s, p in enumerate(parts):
            for k in range(hk):
                if p == 0:
                    assert (s, k) not in pieces
                    continue
                covered = []
                for first, count, g in pieces[(s, k)]:
                    covered += list(range(first, first + count))
                    keys[g] += min(lens[s], (first + count) * psize) - first * psize
                assert covered == list(range(p)), (lens[s], pieces[(s, k)])
        total = sum(keys)
        if total >= 64 * psize * groups:  # enough for the rounding to partitions not to matter
            share = [k / total * groups for k in keys]
            weight = [1.08, 0.92] if groups == 2 * cus else [1.0, 1.0]
            half = groups // 2 if groups == 2 * cus else groups
            assert all(x < weight[g >= half] + 0.08 for g, x in enumerate(share)), (min(share), max(share))


def test_properties_over_random_batches():
    rng = random.Random(1)
    for _ in range(300):
        S = rng.choice((1, 3, 8, 40, 128, 256))
        psize = rng.choice((256, 512))
        lens = [rng.randint(0, 64 * psize) if rng.random() < 0.7 else rng.randint(0, 3 * psize) for _ in range(S)]
        hk = rng.choice((1, 4, 8, 32))
        cus = 256
        groups = rng.choice((cus, 2 * cus, 3 * cus))
        groups = min(groups, max(1, S * hk * 64))
        kw = _args(partition_size=psize, max_ctx=64 * psize, num_kv_heads=hk, groups=groups, cus=cus,
                   rows_apart=rng.random() < 0.5, partition_bytes=2 * psize * rng.choice((128, 256)))
        m = P.partitions_per_segment(lens, **kw)
        assert 1 <= m <= P.SEGMENT_MAX_PARTITIONS
        segs = P.segments_of(lens, m, partition_size=psize, max_num_partitions=64, max_ctx=64 * psize)
        assert sum(segs) == sum(min(c, 64 * psize) for c in lens)       # every key in exactly one segment
        assert all(0 < s <= m * psize for s in segs)
        total = sum(math.ceil(min(c, 64 * psize) / psize) for c in lens) * hk
        if total <= groups and m == 1:
            continue
        # the rule aims at a share of a compute unit's load: a segment is never longer than twice a
        # unit's mean load (in partitions, rounded up) unless one partition already is
        per_unit = total / min(groups, cus)
        assert m <= max(1, math.ceil(2 * per_unit)), (m, per_unit, kw)
