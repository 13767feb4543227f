"""Stream-ordered ``torch.library`` operators over the C ABI.

Upstream's launchers build a queue of their own and block on every kernel
(launch_kernels_reduce.h:35-38 creates ``sycl::queue q``; the line that would have taken
PyTorch's current stream, ``c10::xpu::getCurrentXPUStream().queue()``, is commented out at
:35; ``event1.wait()`` :56 and ``event2.wait()`` :75 stall the host between kernels).  The
operators below are what that commented-out line was after: each one enqueues its kernels on
PyTorch's *current* stream and returns at once -- no event, no synchronisation, nothing but
kernel launches on the stream -- so they order with the rest of a model's work and can be
recorded into a HIP graph (``torch.cuda.graph``) and replayed.

    torch.ops.fa_amd.paged_attention_loop(out, query, key_cache, value_cache, block_tables,
                                          context_lens, scale, sinks)
    torch.ops.fa_amd.paged_attention_reduce(out, exp_sums, max_logits, tmp_out, query, key_cache,
                                            value_cache, block_tables, context_lens, scale,
                                            partition_size, sinks)
    torch.ops.fa_amd.paged_attention_fp8_loop(..., scale, fp8_scale, sinks)
    torch.ops.fa_amd.paged_attention_fp8_reduce(..., scale, fp8_scale, partition_size, sinks)
    torch.ops.fa_amd.kv_cache_write(key, value, key_cache, value_cache, slot_mapping, fp8_scale)

Further optional arguments, all off by default: ``alibi_slopes`` (fp32 ``[heads]``), ``softcap``
(> 0) and ``window_left`` (>= 0) apply the score modifiers -- here a modifier that is passed is
applied, unlike ``lib.*.run``, which mirrors upstream in taking and ignoring slopes and cap; the
FP8 operators and ``kv_cache_write`` take ``k_scales`` / ``v_scales`` (fp32 ``[kv_heads]`` or
``[blocks, kv_heads]``) in place of the scalar ``fp8_scale``.  ``query`` / ``out`` may be
``[seqs, query_len, heads, head_size]``: several causal query tokens per sequence.

SCRATCH CAPACITY of the reduce operators: ``exp_sums.size(-1)`` partitions of ``partition_size`` tokens must
cover the longest context of the batch.  The kernels cannot raise an error: a longer context is attended
over its first ``partitions * partition_size`` tokens only.  Pass ``max_context_len`` (the longest
context, known on the host) and the call fails with FA_ERR_PARTITION_OVERFLOW instead.  Without it (the
default, -1) the only bound the host has is what the block table can hold, ``block_tables.size(1) *
block_size``: if the scratch arrays hold fewer tokens than that, a RuntimeWarning says so, once; an
explicit 0 checks nothing and warns of nothing.

Caches are ``[blocks, block_size, kv_heads, head_size]`` views as in ``lib.*.run``; every
output is an argument the operator mutates, nothing is allocated.  Importing this module
registers the operators; there is no CPU implementation.
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import Tensor

from .lib import (kv_cache_write as _kv_cache_write, paged_attention_fp8_loop as _fp8_loop,
                  paged_attention_fp8_reduce as _fp8_reduce, paged_attention_loop as _loop,
                  paged_attention_reduce as _reduce)

_NS = "fa_amd"


def _group(query: Tensor, key_cache: Tensor) -> int:
    return query.size(-2) // key_cache.size(2)


_warned_capacity = False


def _checked_context_len(max_context_len: int, exp_sums: Tensor, partition_size: int, query: Tensor,
                         key_cache: Tensor, block_tables: Tensor) -> int:
    """What the launcher is told the longest context is.  -1: unknown -- warn once if the block table
    could hold a context the scratch arrays cannot (nothing is read from the device for this)."""
    if max_context_len >= 0:
        return max_context_len
    global _warned_capacity
    if not _warned_capacity:
        size = partition_size if partition_size > 0 else (256 if query.size(-1) == 64 else 512)
        if exp_sums.size(-1) * size < block_tables.size(1) * key_cache.size(1):
            _warned_capacity = True
            import warnings
            warnings.warn(f"the scratch arrays hold {exp_sums.size(-1)} partitions of {size} tokens, the block table "
                          f"{block_tables.size(1)} blocks of {key_cache.size(1)}: a context beyond "
                          f"{exp_sums.size(-1) * size} tokens would be attended over its first tokens only -- pass "
                          "max_context_len to have that checked (0 to silence this warning)", RuntimeWarning, stacklevel=3)
    return 0


def _modifiers(alibi_slopes: Optional[Tensor], softcap: float, window_left: int) -> dict:
    return dict(apply_alibi=alibi_slopes is not None, apply_softcap=softcap > 0.0,
                window_left=window_left if window_left >= 0 else None)


@torch.library.custom_op(f"{_NS}::paged_attention_loop", mutates_args=("out",), device_types="cuda")
def paged_attention_loop(out: Tensor, query: Tensor, key_cache: Tensor, value_cache: Tensor,
                         block_tables: Tensor, context_lens: Tensor, scale: float,
                         sinks: Optional[Tensor] = None, alibi_slopes: Optional[Tensor] = None,
                         softcap: float = 0.0, window_left: int = -1) -> None:
    _loop.run(None, None, None, out, None, query, key_cache, value_cache, block_tables, context_lens,
              _group(query, key_cache), scale, key_cache.size(1), 0, alibi_slopes, sinks, softcap, timed=False,
              **_modifiers(alibi_slopes, softcap, window_left))


@torch.library.custom_op(f"{_NS}::paged_attention_fp8_loop", mutates_args=("out",), device_types="cuda")
def paged_attention_fp8_loop(out: Tensor, query: Tensor, key_cache: Tensor, value_cache: Tensor,
                             block_tables: Tensor, context_lens: Tensor, scale: float, fp8_scale: float,
                             sinks: Optional[Tensor] = None, alibi_slopes: Optional[Tensor] = None,
                             softcap: float = 0.0, window_left: int = -1, k_scales: Optional[Tensor] = None,
                             v_scales: Optional[Tensor] = None) -> None:
    _fp8_loop.run(None, None, None, out, None, query, key_cache, value_cache, block_tables, context_lens,
                  _group(query, key_cache), scale, fp8_scale, key_cache.size(1), 0, alibi_slopes, sinks, softcap,
                  timed=False, k_scales=k_scales, v_scales=v_scales, **_modifiers(alibi_slopes, softcap, window_left))


@torch.library.custom_op(f"{_NS}::paged_attention_reduce",
                         mutates_args=("out", "exp_sums", "max_logits", "tmp_out"), device_types="cuda")
def paged_attention_reduce(out: Tensor, exp_sums: Tensor, max_logits: Tensor, tmp_out: Tensor, query: Tensor,
                           key_cache: Tensor, value_cache: Tensor, block_tables: Tensor, context_lens: Tensor,
                           scale: float, partition_size: int = 0, sinks: Optional[Tensor] = None,
                           alibi_slopes: Optional[Tensor] = None, softcap: float = 0.0,
                           window_left: int = -1, max_context_len: int = -1) -> None:
    if tmp_out.dtype != torch.float32:
        raise RuntimeError("tmp_out must be fp32: these operators allocate nothing, not even a workspace")
    max_context_len = _checked_context_len(max_context_len, exp_sums, partition_size, query, key_cache, block_tables)
    _reduce.run(max_logits, exp_sums, tmp_out, out, None, query, key_cache, value_cache, block_tables,
                context_lens, _group(query, key_cache), scale, key_cache.size(1), max_context_len, alibi_slopes, sinks,
                softcap, partition_size=partition_size, timed=False, **_modifiers(alibi_slopes, softcap, window_left))


@torch.library.custom_op(f"{_NS}::paged_attention_fp8_reduce",
                         mutates_args=("out", "exp_sums", "max_logits", "tmp_out"), device_types="cuda")
def paged_attention_fp8_reduce(out: Tensor, exp_sums: Tensor, max_logits: Tensor, tmp_out: Tensor, query: Tensor,
                               key_cache: Tensor, value_cache: Tensor, block_tables: Tensor,
                               context_lens: Tensor, scale: float, fp8_scale: float, partition_size: int = 0,
                               sinks: Optional[Tensor] = None, alibi_slopes: Optional[Tensor] = None,
                               softcap: float = 0.0, window_left: int = -1, k_scales: Optional[Tensor] = None,
                               v_scales: Optional[Tensor] = None, max_context_len: int = -1) -> None:
    if tmp_out.dtype != torch.float32:
        raise RuntimeError("tmp_out must be fp32: these operators allocate nothing, not even a workspace")
    max_context_len = _checked_context_len(max_context_len, exp_sums, partition_size, query, key_cache, block_tables)
    _fp8_reduce.run(max_logits, exp_sums, tmp_out, out, None, query, key_cache, value_cache, block_tables,
                    context_lens, _group(query, key_cache), scale, fp8_scale, key_cache.size(1), max_context_len,
                    alibi_slopes, sinks, softcap, partition_size=partition_size, timed=False, k_scales=k_scales,
                    v_scales=v_scales, **_modifiers(alibi_slopes, softcap, window_left))


@torch.library.custom_op(f"{_NS}::kv_cache_write", mutates_args=("key_cache", "value_cache"), device_types="cuda")
def kv_cache_write(key: Tensor, value: Tensor, key_cache: Tensor, value_cache: Tensor, slot_mapping: Tensor,
                   fp8_scale: float = 1.0, k_scales: Optional[Tensor] = None,
                   v_scales: Optional[Tensor] = None) -> None:
    _kv_cache_write.run(key, value, key_cache, value_cache, slot_mapping, fp8_scale, timed=False,
                        k_scales=k_scales, v_scales=v_scales)


# Shape propagation for tracing: every operator only writes into its arguments.
for _op in (paged_attention_loop, paged_attention_fp8_loop, paged_attention_reduce, paged_attention_fp8_reduce,
            kv_cache_write):
    _op.register_fake(lambda *args, **kwargs: None)
