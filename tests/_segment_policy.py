"""The segment-length rule of the split path, restated on the host for the tests.

The attention kernels of the segment form choose on the device, from the batch's context lengths,
how many partitions one partial covers (csrc/paged_attention_segment_policy.h:
partitions_per_segment; the role upstream gives to a compile-time constant,
include/paged_attention_policy_v2.hpp:28,50 -- one partial per partition).  This file follows that
function statement by statement, in the same integer and fp32 arithmetic, so that the constants in
it are guarded by CPU tests (recorded batches with the lengths the GPU chose) and by a GPU test that
compares the two on fresh batches.  Test infrastructure: nothing in the product imports it.
"""
from __future__ import annotations

import math

import numpy as np

F = np.float32
SEGMENT_MAX_PARTITIONS = 64
SEGMENT_BYTES_WORTH_CUTTING = 768 << 10


def segment_share_of_load(x: int) -> int:
    if x <= 1024:
        return 1147
    if x <= 2048:
        return 1147 - ((563 * (x - 1024)) >> 10)
    if x <= 4096:
        return 584 - ((205 * (x - 2048)) >> 11)
    if x <= 8192:
        return 379 - ((19 * (x - 4096)) >> 12)
    return 360


def live_partitions(lens, partition_size: int, max_num_partitions: int, max_ctx: int):
    ctx = [max(0, min(int(c), max_ctx)) for c in lens]
    parts = [min((c + partition_size - 1) // partition_size, max_num_partitions) for c in ctx]
    return ctx, parts


def count_segments(ctx, parts, partition_size: int, m: int):
    seg = m * partition_size
    whole = tails = 0
    for c, p in zip(ctx, parts):
        cut = min(c, p * partition_size)
        whole += cut // seg
        tails += cut % seg > 0
    return whole, whole + tails


def partitions_per_segment(lens, *, partition_size: int, max_num_partitions: int, max_ctx: int, num_kv_heads: int,
                           groups: int, cus: int, rows_apart: bool, partition_bytes: int) -> int:
    """num_kv_heads: kv-head items per sequence as the kernel deals them (pairs or teams of heads
    count once); groups: work-groups of the launch; partition_bytes: K and V bytes of one partition
    of one item."""
    ctx, parts = live_partitions(lens, partition_size, max_num_partitions, max_ctx)
    total_partitions = sum(parts)
    units = max(1, min(groups, cus))
    sharing = 1 if groups <= units else 2 if groups <= 2 * units else (groups + units - 1) // units
    live = sum(p > 0 for p in parts)
    items = F(total_partitions) * F(num_kv_heads)
    per_unit = F(1.0) / F(units)
    seqs_per_cu = min(F(live) * F(num_kv_heads) * per_unit, F(1024.0))
    share = segment_share_of_load(int(F(seqs_per_cu) * F(1024.0)))
    halves = sharing > 2 or (rows_apart and sharing > 1)
    if halves:
        load_bytes = F(items * per_unit) * F(partition_bytes)
        n = max(1, min(int(F(load_bytes * F(1.0 / SEGMENT_BYTES_WORTH_CUTTING)) + F(0.5)), 2 * sharing))
        share = 1024 // n
    elif sharing == 2:
        share = min(share, 512)
    m = int(min(F(F(items * per_unit) * F(F(share) * F(1.0 / 1024.0))) + F(0.5), F(SEGMENT_MAX_PARTITIONS)))
    m = max(m, 1)
    if m == 1 and items <= F(groups):
        return 1
    if halves:
        return m
    items_all = total_partitions * num_kv_heads
    few = sharing > 1 and 2 * live * num_kv_heads <= units
    aimed = m
    phase = 1
    if sharing > 1 and live * num_kv_heads <= units and items_all > units:
        phase = 0
        m = int(min(F(math.ceil(F(items * per_unit))), F(SEGMENT_MAX_PARTITIONS)))
    before = tries = 0
    for _ in range(12):
        if phase == 0 and (tries >= 4 or m > SEGMENT_MAX_PARTITIONS or 4 * m * units > 5 * items_all):
            phase, m, tries = 1, aimed, 0
        whole, every = count_segments(ctx, parts, partition_size, m)
        n = every * num_kv_heads
        if phase == 0:
            if n <= units:
                return m
            m += 1
            tries += 1
            continue
        if phase == 1:
            if whole * num_kv_heads > groups and tries < 3 and m < SEGMENT_MAX_PARTITIONS:
                m += 1
                tries += 1
                continue
            if not (few and n > units and n * 20 < groups * 17):
                return m
            phase, before = 2, m
        elif n <= units:
            return m
        if m - before >= 4 or m >= SEGMENT_MAX_PARTITIONS:
            return before
        m += 1
    return before if before > 0 else m


SHARE_TOKENS = 32
SHARE_PIECE_COST = 4


def even_shares_pieces(lens, *, partition_size: int, max_num_partitions: int, max_ctx: int, num_kv_heads: int,
                       groups: int, cus: int):
    """The pieces even shares cut the batch into: {(sequence, kv-head item): [(first partition, partitions,
    work-group), ...]} -- what options->segment_partitions = -1 asks for.  A row costs its keys in steps
    of 32 plus 4 steps; the rows' costs lie end to end, sequences in order and kv heads within a sequence;
    the work-groups take equal stretches of that tape in turn (to within a step; with two work-groups on
    every compute unit the older half of them takes 54 % of it), and what a work-group holds of a row
    runs between the partition boundaries nearest to its stretch's ends
    (csrc/paged_attention_items.h: build_even_shares, next_of_share)."""
    ctx, parts = live_partitions(lens, partition_size, max_num_partitions, max_ctx)
    ctx = [min(c, p * partition_size) for c, p in zip(ctx, parts)]
    cost = [(c + SHARE_TOKENS - 1) // SHARE_TOKENS + SHARE_PIECE_COST if c > 0 else 0 for c in ctx]
    n = sum(cost) * num_kv_heads
    # two work-groups per compute unit (g and g + cus): the older half takes 540 / 1000 of the tape
    halves = [(0, n, groups)]
    if groups == 2 * cus:
        older = int(F(n) * (F(540) * F(0.001)))
        halves = [(0, older, cus), (older, n - older, cus)]
    bounds = []
    for begin, length, count in halves:
        each, extra = divmod(length, count)
        bounds += [begin + g * each + min(g, extra) for g in range(count)]
    bounds.append(n)
    steps = partition_size // SHARE_TOKENS

    def nearest_cut(x, parts_of_row):
        return min(parts_of_row, (x + steps // 2) // steps)

    pieces = {}
    row_begin = 0
    for s, (c, p) in enumerate(zip(cost, parts)):
        for k in range(num_kv_heads if c else 0):
            row_end = row_begin + c
            row = []
            for g in range(groups):
                lo, hi = bounds[g], bounds[g + 1]
                if hi <= row_begin or lo >= row_end or lo == hi:
                    continue
                first = 0 if lo <= row_begin else nearest_cut(lo - row_begin, p)
                last = p if hi >= row_end else nearest_cut(hi - row_begin, p)
                if last > first:
                    row.append((first, last - first, g))
            pieces[(s, k)] = row
            row_begin = row_end
    return pieces


def segments_of(lens, m: int, *, partition_size: int, max_num_partitions: int, max_ctx: int):
    """Token lengths of the segments a length of m partitions cuts the batch into (per kv head)."""
    ctx, parts = live_partitions(lens, partition_size, max_num_partitions, max_ctx)
    seg = m * partition_size
    out = []
    for c, p in zip(ctx, parts):
        cut = min(c, p * partition_size)
        out += [seg] * (cut // seg)
        if cut % seg:
            out.append(cut % seg)
    return out
