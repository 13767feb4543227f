"""Batches for the segment-length rule of the split path, and the lengths the GPU chose for them.

`batches(seed)` draws seeded batches over the shapes the rule distinguishes (head sizes, cache
types, pool layouts, 1 to 256 sequences, uniform / long / log-normal lengths).  `device_choice`
runs one through `lib.paged_attention_*reduce.run` on the GPU and reads, from the mark the
attention kernel leaves in slot 1 of max_logits (csrc/paged_attention_segment_policy.h:
segment_mark), how many partitions a partial covers; the launch geometry comes from
fa_paged_attention_reduce_plan.  Run as a script ON A GPU BOX it writes
tests/golden/segment_policy_cases.json, which the CPU test replays with tests/_segment_policy.py;
tests/test_gpu_segment_policy.py compares the two on batches of another seed.

    python tests/golden/make_segment_policy_cases.py [output.json]         # needs the GPU

Upstream has no such rule (one partial per partition, paged_attention_policy_v2.hpp:28,50) and so
no vectors: these are this library's own choices, frozen so that a change of the fitted constants
shows.
"""
from __future__ import annotations

import ctypes
import json
import math
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

MARK_BITS, MARK_MASK = 0x7FD3A600, 0xFFFFFF00

# (head_size, kv heads, group, fp8, token_major, block_size)
SHAPES = [
    (128, 8, 4, False, False, 16),   # 16-bit, head-major: the long-context configuration's shape
    (128, 8, 8, True, False, 16),    # byte cache, head-major: the serving mix's shape
    (128, 8, 4, False, True, 16),    # 16-bit, upstream's layout: rows apart, two work-groups per unit
    (128, 8, 8, True, True, 16),     # byte cache, upstream's layout: teams of two kv heads
    (64, 8, 8, False, True, 64),     # upstream's own perf shape: 128-byte rows, teams
    (64, 8, 5, True, True, 64),      # its FP8 twin: pairs of kv heads
    (64, 8, 2, False, False, 16),    # head size 64, head-major: three work-groups per unit
]


def batches(seed: int, per_shape: int = 9):
    g = torch.Generator().manual_seed(seed)
    out = []
    for shape_index, (d, hk, group, fp8, token_major, block) in enumerate(SHAPES):
        psize = 256 if d == 64 else 512
        for k in range(per_shape):
            S = [1, 2, 4, 8, 16, 32, 64, 128, 256][(k + shape_index) % 9]
            kind = k % 3
            if kind == 0:    # long contexts
                lens = torch.randint(16 * psize, 64 * psize + 1, (S,), generator=g)
            elif kind == 1:  # log-normal around 8 partitions, clipped
                lens = torch.exp(torch.randn(S, generator=g) * 0.75 + math.log(8 * psize)).long().clamp(64, 64 * psize)
            else:            # a few partitions each
                lens = torch.randint(1, 6 * psize + 1, (S,), generator=g)
            out.append(dict(head_size=d, num_kv_heads=hk, group=group, fp8=fp8, token_major=token_major,
                            block_size=block, partition_size=psize, lens=[int(x) for x in lens]))
    return out


def device_choice(case, dev, segment_partitions=0):
    """(how the attention kernel cut the batch, plan, the slots of every (sequence, kv-head item) row that
    hold partials) for one batch.  The cut: m, the partitions per segment; 0 for even shares
    (segment_partitions = -1); None if the call did not run in the segment form or no slot holds a mark
    (no piece covers two partitions)."""
    from flash_attention_factory_amd import _cabi, lib
    d, hk, group, block, psize = (case[k] for k in ("head_size", "num_kv_heads", "group", "block_size", "partition_size"))
    lens = torch.tensor(case["lens"], dtype=torch.int32)
    S, H = lens.numel(), hk * group
    mb = max(1, math.ceil(int(lens.max()) / block))
    npart = max(1, math.ceil(int(lens.max()) / psize))
    nb = 2048
    shape = (nb, block, hk, d) if case["token_major"] else (nb, hk, block, d)
    kv_dtype = torch.uint8 if case["fp8"] else torch.float16
    key = torch.zeros(shape, dtype=kv_dtype, device=dev)
    value = torch.zeros(shape, dtype=kv_dtype, device=dev)
    view = (lambda t: t) if case["token_major"] else (lambda t: t.permute(0, 2, 1, 3))
    tables = torch.randint(0, nb, (S, mb), generator=torch.Generator().manual_seed(0), dtype=torch.int32).to(dev)
    query = torch.zeros((S, H, d), dtype=torch.float16, device=dev)
    out = torch.zeros_like(query)
    ml = torch.full((S, H, npart), float("nan"), dtype=torch.float32, device=dev)
    es = torch.full_like(ml, float("nan"))
    tmp = torch.empty((S, H, npart, d), dtype=torch.float32, device=dev)
    mod = lib.paged_attention_fp8_reduce if case["fp8"] else lib.paged_attention_reduce
    head = [ml, es, tmp, out, None, query, view(key), view(value), tables, lens.to(dev), group, d ** -0.5]
    if case["fp8"]:
        head.append(1.0)
    mod.run(*head, block, 0, None, None, 0.0, partition_size=psize, timed=False, segment_partitions=segment_partitions)
    torch.cuda.synchronize()
    # the plan of the same call
    sh = _cabi.Shape()
    sh.num_seqs, sh.num_heads, sh.num_kv_heads, sh.head_size, sh.block_size = S, H, hk, d, block
    sh.max_blocks_per_seq, sh.max_num_partitions, sh.partition_size = mb, npart, psize
    kc = view(key)
    sh.kv_block_stride, sh.kv_token_stride, sh.kv_head_stride = kc.stride(0), kc.stride(1), kc.stride(2)
    sh.q_dtype, sh.num_pool_blocks = _cabi.FA_DTYPE_F16, nb
    plan = _cabi.SplitPlan()
    _cabi.check(_cabi.load().fa_paged_attention_reduce_plan(ctypes.byref(sh), None, 0, int(case["fp8"]), 0, ctypes.byref(plan)))
    m, slots = None, {}
    if plan.form == _cabi.FA_SPLIT_FORM_SEGMENT:
        bits = ml.view(torch.int32).cpu()
        marks = bits[(bits & MARK_MASK) == MARK_BITS]
        if marks.numel():
            low = set((marks & 0xFF).tolist())
            assert len(low) == 1, low  # every mark of a launch carries the same byte
            m = low.pop()
        first_head = plan.kv_heads_per_item * group  # query heads per kv-head item
        written = ~torch.isnan(ml.cpu())
        for s in range(S):
            for k in range(hk // plan.kv_heads_per_item):
                if case["lens"][s] > 0:
                    slots[(s, k)] = torch.nonzero(written[s, k * first_head]).flatten().tolist()
    return m, dict(form=plan.form, compute_units=plan.compute_units, work_groups=plan.work_groups,
                   kv_heads_per_item=plan.kv_heads_per_item), slots


def _policy():
    sys.path.insert(0, os.path.dirname(HERE))
    import _segment_policy
    return _segment_policy


def _geometry(case, plan):
    d, hk, block, psize = (case[k] for k in ("head_size", "num_kv_heads", "block_size", "partition_size"))
    lens = case["lens"]
    mb = max(1, math.ceil(max(lens) / block))
    npart = max(1, math.ceil(max(lens) / psize))
    per_item = plan["kv_heads_per_item"]
    return dict(partition_size=psize, max_num_partitions=npart, max_ctx=mb * block, num_kv_heads=hk // per_item,
                groups=plan["work_groups"])


def replay(case, plan):
    """The same choice by the host restatement of the rule: partitions per segment."""
    P = _policy()
    geo = _geometry(case, plan)
    row_bytes = case["head_size"] * (1 if case["fp8"] else 2) * plan["kv_heads_per_item"]
    return P.partitions_per_segment(case["lens"], cus=plan["compute_units"], rows_apart=case["token_major"],
                                    partition_bytes=2 * case["partition_size"] * row_bytes, **geo)


def replay_slots(case, plan, m):
    """The slots that hold partials, per (sequence, kv-head item) row, for a cut of m (0: even shares)."""
    P = _policy()
    geo = _geometry(case, plan)
    if m == 0:
        pieces = P.even_shares_pieces(case["lens"], cus=plan["compute_units"], **geo)
        return {row: [first for first, _, _ in cut] for row, cut in pieces.items()}
    _, parts = P.live_partitions(case["lens"], geo["partition_size"], geo["max_num_partitions"], geo["max_ctx"])
    return {(s, k): list(range(0, p, m)) for s, p in enumerate(parts) if p > 0 for k in range(geo["num_kv_heads"])}


def main():
    dev = torch.device("cuda:0")
    cases = []
    for case in batches(seed=0):
        m, plan, _ = device_choice(case, dev)
        if m is None:
            continue
        cases.append(dict(case, plan=plan, partitions_per_segment=m))
        print(f"S={len(case['lens']):3d} d={case['head_size']} fp8={int(case['fp8'])} tm={int(case['token_major'])} "
              f"groups={plan['work_groups']} per_item={plan['kv_heads_per_item']} -> m={m} (replay {replay(case, plan)})", flush=True)
    path = sys.argv[1] if len(sys.argv) > 1 else os.path.join(HERE, "segment_policy_cases.json")
    with open(path, "w") as f:
        json.dump(dict(note="lengths chosen on an MI355X by the attention kernels of the segment form; written by "
                            "tests/golden/make_segment_policy_cases.py", cases=cases), f, separators=(",", ":"))
        f.write("\n")
    print(f"wrote {len(cases)} cases to {path}")


if __name__ == "__main__":
    main()
