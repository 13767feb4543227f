"""Drives a ``Workload`` through the ``lib.paged_attention_*`` modules the way the
upstream test functions drive theirs (test_paged.py:449-483, test_paged_fp8cache.py:
476-516): allocate outputs and scratch, call ``run`` positionally, return the result."""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional

import torch

from . import lib
from .workloads import HEAD_MAJOR, Workload

_MODULES = {
    "loop": lib.paged_attention_loop,
    "reduce": lib.paged_attention_reduce,
    "fp8_loop": lib.paged_attention_fp8_loop,
    "fp8_reduce": lib.paged_attention_fp8_reduce,
}


@dataclass
class Buffers:
    out: torch.Tensor
    max_logits: torch.Tensor
    exp_sums: torch.Tensor
    tmp_out: torch.Tensor
    debug: torch.Tensor
    alibi: torch.Tensor


def logical_cache_view(w: Workload, cache: torch.Tensor) -> torch.Tensor:
    """The [blocks, block_size, kv_heads, head_size] view ``run`` expects."""
    return cache.permute(0, 2, 1, 3) if w.layout == HEAD_MAJOR else cache


def alloc_buffers(w: Workload, max_num_partitions: Optional[int] = None, fill: float = float("nan")) -> Buffers:
    S, H, D = w.query.shape
    dev = w.query.device
    NP = max_num_partitions or w.max_num_partitions
    return Buffers(
        out=torch.zeros((S, H, D), dtype=w.query.dtype, device=dev),
        max_logits=torch.full((S, H, NP), fill, dtype=torch.float32, device=dev),
        exp_sums=torch.full((S, H, NP), fill, dtype=torch.float32, device=dev),
        tmp_out=torch.full((S, H, NP, D), fill, dtype=torch.float32, device=dev),
        debug=torch.zeros(1, dtype=torch.float32, device=dev),
        alibi=torch.ones(H, dtype=torch.float32, device=dev),
    )


def run_workload(w: Workload, kernel: str, bufs: Optional[Buffers] = None, *,
                 key_cache: Optional[torch.Tensor] = None,
                 value_cache: Optional[torch.Tensor] = None, timed: bool = True,
                 max_context_len: Optional[int] = None, schedule: int = 0, spin_limit: int = 0,
                 segment_partitions: int = 0) -> List[float]:
    """One call of ``lib.paged_attention_<kernel>.run``; returns its kernel times (us).
    ``key_cache``/``value_cache`` substitute pool clones of the same layout.  ``max_context_len``
    defaults to what the block table can hold (no device read needed to know it).  ``schedule``:
    0 = the library's choice, 1 = the grid form (one work-group per (sequence, kv head[, partition])),
    2 = the grid form with K/V staged through LDS."""
    if kernel.startswith("fp8") != w.is_fp8:
        raise ValueError(f"kernel {kernel} does not match the workload's cache dtype")
    bufs = bufs or alloc_buffers(w)
    mod = _MODULES[kernel]
    kc = logical_cache_view(w, w.key_cache if key_cache is None else key_cache)
    vc = logical_cache_view(w, w.value_cache if value_cache is None else value_cache)
    G = w.num_heads // w.num_kv_heads
    max_ctx = max_context_len if max_context_len is not None else int(w.block_tables.shape[1]) * w.block_size
    head = (bufs.max_logits, bufs.exp_sums, bufs.tmp_out, bufs.out, bufs.debug, w.query, kc, vc,
            w.block_tables, w.context_lens, G, w.scale)
    tail = (w.block_size, max_ctx, bufs.alibi, w.sinks, -1.0)
    kw = dict(timed=timed, schedule=schedule, spin_limit=spin_limit)
    if "reduce" in kernel:
        kw["partition_size"] = w.partition_size
        kw["segment_partitions"] = segment_partitions
    if w.is_fp8:
        return mod.run(*head, w.fp8_scale, *tail, **kw)
    return mod.run(*head, *tail, **kw)
