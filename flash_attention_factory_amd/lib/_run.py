"""Shared body of the four ``run`` functions: torch tensors -> C ABI call.

Mirrors what the upstream pybind entry does with its arguments
(paged_attention_loop/paged_attention_loop.cpp:44-79): pointers come from the tensors,
sizes from their shapes -- num_seqs, num_heads, head_size from ``query``; num_kv_heads
from ``key_cache.size(2)``; max_num_partitions from ``max_logits.size(2)``;
max_blocks_per_seq from ``block_tables.size(1)``.  Unlike upstream, cache strides are
read too, so a head-major pool passed as ``pool.permute(0, 2, 1, 3)`` works as well as
the contiguous ``[blocks, block_size, kv_heads, head_size]`` tensor.
"""
from __future__ import annotations

import ctypes
import warnings
from typing import List, Optional

import torch

from .. import _cabi

_scratch = {}
_warned_scratch = False


def _fp32_scratch(tem_output: torch.Tensor, shape) -> torch.Tensor:
    """Upstream keeps tem_output in the query dtype; the kernels here want fp32.  A
    caller that passes a 16-bit tem_output gets a cached fp32 workspace instead."""
    want = 1
    for n in shape:
        want *= n
    if tem_output.dtype == torch.float32 and tem_output.numel() == want and tem_output.is_contiguous():
        return tem_output
    global _warned_scratch
    if not _warned_scratch:
        _warned_scratch = True
        warnings.warn("tem_output is not a contiguous fp32 tensor of the scratch shape (upstream keeps it in the "
                      "query dtype): the kernels use a cached fp32 workspace of their own instead, allocated on "
                      "first use and shared by every call on this stream -- pass fp32 scratch to avoid it",
                      RuntimeWarning, stacklevel=4)
    key = (tem_output.device, torch.cuda.current_stream(tem_output.device).cuda_stream, tuple(shape))
    buf = _scratch.get(key)
    if buf is None:
        if len(_scratch) >= 8:
            _scratch.clear()
        buf = torch.empty(shape, dtype=torch.float32, device=tem_output.device)
        _scratch[key] = buf
    return buf


def run_impl(entry: str, split: bool, fp8: bool, max_logits, exp_sums, tem_output, output,
             debug_output, query, key_cache, value_cache, block_tables, context_lens,
             num_queries_per_tokens: int, sm_scale: float, fp8_scale: float, block_size: int,
             max_context_len: int, alibi_slopes, sinks: Optional[torch.Tensor], softcap: float,
             partition_size: int = 0, timed: bool = True, apply_alibi: bool = False,
             apply_softcap: bool = False, window_left: Optional[int] = None,
             k_scales: Optional[torch.Tensor] = None, v_scales: Optional[torch.Tensor] = None,
             static_scratch_partitions: int = 0, schedule: int = 0, spin_limit: int = 0,
             segment_partitions: int = 0) -> List[float]:
    """``static_scratch_partitions`` > 0 (split entries without FP8 only): the scratch arrays are the
    library's own fixed device array instead of max_logits / exp_sums / tem_output, which may then be
    None; the value is max_num_partitions."""
    L = _cabi.load()
    if not query.is_cuda:
        raise RuntimeError("paged attention runs on the GPU only: `query` is not a device tensor")
    # every pointer handed to the kernels must be a device pointer on the query's device: a host
    # tensor here would be a GPU memory fault, not an exception
    tensors = [("output", output), ("key_cache", key_cache), ("value_cache", value_cache),
               ("block_tables", block_tables), ("context_lens", context_lens), ("sinks", sinks)]
    if split and not static_scratch_partitions:
        tensors += [("max_logits", max_logits), ("exp_sums", exp_sums), ("tem_output", tem_output)]
    _cabi.require_same_device("query", query, tensors)
    for name, t in (("query", query), ("output", output), ("block_tables", block_tables),
                    ("context_lens", context_lens)):
        if not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous")
    if query.dtype not in (torch.float16, torch.bfloat16) or output.dtype != query.dtype:
        raise _cabi.PagedAttentionError(_cabi.FA_ERR_UNSUPPORTED_DTYPE,
                                        "query/output must both be fp16 or both bf16")
    if block_tables.dtype != torch.int32 or context_lens.dtype != torch.int32:
        raise _cabi.PagedAttentionError(_cabi.FA_ERR_UNSUPPORTED_DTYPE,
                                        "block_tables and context_lens must be int32")
    want_kv = (torch.float8_e5m2, torch.float8_e4m3fn, torch.uint8) if fp8 else (query.dtype,)
    if key_cache.dtype not in want_kv or value_cache.dtype != key_cache.dtype:
        raise _cabi.PagedAttentionError(_cabi.FA_ERR_UNSUPPORTED_DTYPE,
                                        f"key/value cache dtype {key_cache.dtype} not in {want_kv}")
    if key_cache.dim() != 4 or key_cache.stride(3) != 1 or value_cache.stride() != key_cache.stride():
        raise _cabi.PagedAttentionError(_cabi.FA_ERR_BAD_SHAPE,
                                        "caches must be 4-D [blocks, block_size, kv_heads, head_size] "
                                        "views with a contiguous last dimension and equal strides")
    # [S, H, D], or [S, query_len, H, D]: several query tokens per sequence (causal among themselves)
    if query.dim() == 4:
        S, QL, H, D = query.shape
    else:
        (S, H, D), QL = query.shape, 1
    if output.shape != query.shape:
        raise _cabi.PagedAttentionError(_cabi.FA_ERR_BAD_SHAPE, "output must have the shape of query")
    if block_tables.dim() != 2 or block_tables.size(0) != S or context_lens.numel() != S:
        raise _cabi.PagedAttentionError(_cabi.FA_ERR_BAD_SHAPE,
                                        f"block_tables must be [{S}, max_blocks_per_seq] and context_lens [{S}]")
    if key_cache.size(3) != D:
        raise _cabi.PagedAttentionError(_cabi.FA_ERR_UNSUPPORTED_HEAD_OR_BLOCK_SIZE,
                                        f"caches hold rows of {key_cache.size(3)} elements, query heads of {D}")
    if sinks is not None and (sinks.dtype != query.dtype or sinks.numel() != H or not sinks.is_contiguous()):
        raise _cabi.PagedAttentionError(_cabi.FA_ERR_BAD_SHAPE,
                                        f"sinks must be a contiguous [{H}] tensor of the query dtype")
    sh = _cabi.Shape()
    sh.num_seqs, sh.num_heads, sh.head_size = S, H, D
    sh.num_kv_heads = key_cache.size(2)
    sh.block_size = block_size
    sh.max_blocks_per_seq = block_tables.size(1)
    sh.max_num_partitions = (static_scratch_partitions or max_logits.size(-1)) if split else 1
    sh.partition_size = partition_size
    sh.kv_block_stride, sh.kv_token_stride, sh.kv_head_stride = (
        key_cache.stride(0), key_cache.stride(1), key_cache.stride(2))
    sh.num_pool_blocks = key_cache.size(0)
    sh.q_dtype = _cabi.FA_DTYPE_BF16 if query.dtype == torch.bfloat16 else _cabi.FA_DTYPE_F16
    if sh.num_kv_heads * num_queries_per_tokens != H:
        raise _cabi.PagedAttentionError(_cabi.FA_ERR_UNSUPPORTED_GROUP,
                                        "Unsupported number of queries per token")
    if key_cache.size(1) != block_size:
        raise _cabi.PagedAttentionError(_cabi.FA_ERR_UNSUPPORTED_HEAD_OR_BLOCK_SIZE,
                                        "Unsupported head size or block size")
    elapsed = (ctypes.c_float * 2)(0.0, 0.0)
    op = _cabi.Options()
    op.sinks = sinks.data_ptr() if sinks is not None else None
    op.alibi_slopes = alibi_slopes.data_ptr() if alibi_slopes is not None else None
    op.softcap = softcap
    op.fp8_scale = fp8_scale
    # upstream's kernels take alibi_slopes and softcap and ignore them; they act here only on request
    if apply_alibi:
        if alibi_slopes is None or alibi_slopes.dtype != torch.float32 or not alibi_slopes.is_contiguous() \
                or alibi_slopes.numel() != H or alibi_slopes.device != query.device:
            raise _cabi.PagedAttentionError(_cabi.FA_ERR_BAD_SHAPE, "apply_alibi needs contiguous fp32 alibi_slopes [num_heads] on the device")
        op.mask_flags |= _cabi.FA_MASK_ALIBI
    if apply_softcap:
        op.mask_flags |= _cabi.FA_MASK_SOFTCAP
    if window_left is not None:
        op.mask_flags |= _cabi.FA_MASK_WINDOW
        op.window_left = int(window_left)
    op.query_len = QL
    op.schedule = int(schedule)
    op.spin_limit = int(spin_limit)
    op.segment_partitions = int(segment_partitions)
    if k_scales is not None or v_scales is not None:
        if not fp8:
            raise _cabi.PagedAttentionError(_cabi.FA_ERR_UNSUPPORTED_DTYPE, "k_scales / v_scales belong to FP8 caches")
        _cabi.set_kv_scales(op, k_scales, v_scales, sh.num_kv_heads, sh.num_pool_blocks, query.device)
    # bytes are E5M2 as upstream fixes them (paged_attention_fp8_loop.cpp:43) unless the tensor says E4M3
    op.kv_fp8_format = _cabi.FA_FP8_E4M3 if key_cache.dtype == torch.float8_e4m3fn else _cabi.FA_FP8_E5M2
    op.stream = torch.cuda.current_stream(query.device).cuda_stream
    op.elapsed_us = ctypes.cast(elapsed, ctypes.POINTER(ctypes.c_float)) if timed else None
    fn = getattr(L, entry)
    args = [output.data_ptr(), query.data_ptr(), key_cache.data_ptr(), value_cache.data_ptr(),
            block_tables.data_ptr(), context_lens.data_ptr(), float(sm_scale), int(max_context_len)]
    if split and static_scratch_partitions:
        pass  # the entry point brings its own scratch
    elif split:
        tmp = _fp32_scratch(tem_output, (S * QL, H, sh.max_num_partitions, D))
        if max_logits.numel() != S * QL * H * sh.max_num_partitions or exp_sums.numel() != max_logits.numel():
            raise _cabi.PagedAttentionError(_cabi.FA_ERR_BAD_SHAPE,
                                            "max_logits/exp_sums must hold [num_seqs * query_len, num_heads, partitions]")
        if max_logits.dtype != torch.float32 or exp_sums.dtype != torch.float32 \
                or not max_logits.is_contiguous() or not exp_sums.is_contiguous():
            raise _cabi.PagedAttentionError(_cabi.FA_ERR_UNSUPPORTED_DTYPE,
                                            "max_logits/exp_sums must be contiguous fp32")
        args += [exp_sums.data_ptr(), max_logits.data_ptr(), tmp.data_ptr()]
    with torch.cuda.device(query.device):
        _cabi.check(fn(*args, ctypes.byref(sh), ctypes.byref(op)))
    if not timed:
        return []
    return [elapsed[0], elapsed[1]] if split else [elapsed[0]]
