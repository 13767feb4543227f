"""ctypes front end of the CPU oracle (TEST INFRASTRUCTURE ONLY).

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module.  It is the checker for the HIP library and
is never used to produce a result the package returns.

All tensors are CPU ``torch`` tensors; 16-bit floats travel as their raw bits.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from dataclasses import dataclass

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle_paged_attention.so")
_lib = None

Q_F16, Q_BF16 = 0, 1
KV_SAME_AS_Q, KV_E5M2, KV_E4M3 = 0, 1, 2


class _Problem(ctypes.Structure):
    _fields_ = [
        ("num_seqs", ctypes.c_int32),
        ("num_heads", ctypes.c_int32),
        ("num_kv_heads", ctypes.c_int32),
        ("head_size", ctypes.c_int32),
        ("block_size", ctypes.c_int32),
        ("max_blocks_per_seq", ctypes.c_int32),
        ("kv_block_stride", ctypes.c_int64),
        ("kv_token_stride", ctypes.c_int64),
        ("kv_head_stride", ctypes.c_int64),
        ("q_dtype", ctypes.c_int32),
        ("kv_dtype", ctypes.c_int32),
        ("scale", ctypes.c_float),
        ("fp8_scale", ctypes.c_float),
    ]


class _KvWrite(ctypes.Structure):
    _fields_ = [
        ("num_tokens", ctypes.c_int32),
        ("num_kv_heads", ctypes.c_int32),
        ("head_size", ctypes.c_int32),
        ("block_size", ctypes.c_int32),
        ("kv_block_stride", ctypes.c_int64),
        ("kv_token_stride", ctypes.c_int64),
        ("kv_head_stride", ctypes.c_int64),
        ("src_token_stride", ctypes.c_int64),
        ("src_head_stride", ctypes.c_int64),
        ("src_dtype", ctypes.c_int32),
        ("cache_dtype", ctypes.c_int32),
        ("num_pool_blocks", ctypes.c_int64),
        ("fp8_scale", ctypes.c_float),
    ]


def build(force: bool = False) -> str:
    """Compile the C restatement with the Makefile next to it."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s"], check=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        P = ctypes.c_void_p
        pp = ctypes.POINTER(_Problem)
        L.oracle_attention_ref.argtypes = [P, P, P, P, P, P, P, P, pp]
        L.oracle_attention_ref.restype = ctypes.c_int
        L.oracle_attention_ref_masked.argtypes = [P, P, P, P, P, P, P, P, P, ctypes.c_float, ctypes.c_int32,
                                                  ctypes.c_int32, pp]
        L.oracle_attention_ref_masked.restype = ctypes.c_int
        L.oracle_attention_ref_scaled.argtypes = [P, P, P, P, P, P, P, P, P, ctypes.c_float, ctypes.c_int32,
                                                  ctypes.c_int32, P, P, ctypes.c_int32, pp]
        L.oracle_attention_ref_scaled.restype = ctypes.c_int
        L.oracle_kv_cache_write_scaled.argtypes = [P, P, P, P, P, P, P, ctypes.c_int32, P]
        L.oracle_kv_cache_write_scaled.restype = ctypes.c_int
        L.oracle_kernel_loop.argtypes = [P, P, P, P, P, P, P, P, ctypes.c_int, pp]
        L.oracle_kernel_loop.restype = ctypes.c_int
        L.oracle_kernel_partition.argtypes = [P, P, P, P, P, P, P, P, P, ctypes.c_int, ctypes.c_int, pp]
        L.oracle_kernel_partition.restype = ctypes.c_int
        L.oracle_kernel_reduce.argtypes = [P, P, P, P, P, P, ctypes.c_int, ctypes.c_int, pp]
        L.oracle_kernel_reduce.restype = ctypes.c_int
        L.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_f16_to_f32.restype = ctypes.c_float
        L.oracle_f32_to_f16.argtypes = [ctypes.c_float]
        L.oracle_f32_to_f16.restype = ctypes.c_uint16
        L.oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_bf16_to_f32.restype = ctypes.c_float
        L.oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        L.oracle_f32_to_bf16.restype = ctypes.c_uint16
        L.oracle_e5m2_to_f32.argtypes = [ctypes.c_uint8]
        L.oracle_e5m2_to_f32.restype = ctypes.c_float
        L.oracle_num_threads.restype = ctypes.c_int
        L.oracle_f32_to_e5m2.argtypes = [ctypes.c_float]
        L.oracle_f32_to_e5m2.restype = ctypes.c_uint8
        L.oracle_f32_to_e4m3_array.argtypes = [P, P, ctypes.c_int64]
        L.oracle_f32_to_e4m3_array.restype = None
        L.oracle_e4m3_to_f32.argtypes = [ctypes.c_uint8]
        L.oracle_e4m3_to_f32.restype = ctypes.c_float
        L.oracle_f32_to_e5m2_array.argtypes = [P, P, ctypes.c_int64]
        L.oracle_f32_to_e5m2_array.restype = None
        L.oracle_kv_cache_write.argtypes = [P, P, P, P, P, ctypes.POINTER(_KvWrite)]
        L.oracle_kv_cache_write.restype = ctypes.c_int
        L.oracle_set_num_threads.argtypes = [ctypes.c_int]
        _lib = L
    return _lib


@dataclass
class _Args:
    problem: _Problem
    keep: list


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _problem(query, key_cache, value_cache, block_tables, context_lens, scale, block_size,
             kv_strides, fp8_scale, num_kv_heads):
    assert query.device.type == "cpu" and query.is_contiguous() and query.dim() == 3
    assert query.dtype in (torch.float16, torch.bfloat16)
    fp8 = key_cache.dtype in (torch.float8_e5m2, torch.float8_e4m3fn, torch.uint8)
    if not fp8:
        assert key_cache.dtype == query.dtype, "16-bit caches share the query dtype"
    assert value_cache.dtype == key_cache.dtype
    assert block_tables.dtype == torch.int32 and block_tables.is_contiguous()
    assert context_lens.dtype == torch.int32 and context_lens.is_contiguous()
    S, H, D = query.shape
    pr = _Problem()
    pr.num_seqs, pr.num_heads, pr.num_kv_heads, pr.head_size = S, H, num_kv_heads, D
    pr.block_size = block_size
    pr.max_blocks_per_seq = block_tables.shape[1]
    pr.kv_block_stride, pr.kv_token_stride, pr.kv_head_stride = kv_strides
    pr.q_dtype = Q_BF16 if query.dtype == torch.bfloat16 else Q_F16
    pr.kv_dtype = (KV_E4M3 if key_cache.dtype == torch.float8_e4m3fn else KV_E5M2) if fp8 else KV_SAME_AS_Q
    pr.scale = scale
    pr.fp8_scale = fp8_scale
    return pr


def _bits_out(S, H, D, dtype):
    return torch.empty((S, H, D), dtype=dtype)


def _scale_pitch(k_scales, v_scales, num_kv_heads, num_blocks) -> int:
    """0 for per-head scales [Hk], Hk for per-block scales [NB, Hk]."""
    for t in (k_scales, v_scales):
        assert t is not None and t.dtype == torch.float32 and t.is_contiguous() and t.shape == k_scales.shape
    if tuple(k_scales.shape) == (num_kv_heads,):
        return 0
    assert tuple(k_scales.shape) == (num_blocks, num_kv_heads), k_scales.shape
    return num_kv_heads


def attention_ref(query, key_cache, value_cache, block_tables, context_lens, *, scale, block_size,
                  kv_strides, num_kv_heads, sinks=None, fp8_scale=1.0, want_f32=False,
                  alibi_slopes=None, softcap=0.0, window_left=-1, k_scales=None, v_scales=None):
    """The upstream tests' PyTorch reference, restated (test_paged.py:40-168).  ``alibi_slopes``
    ([heads] fp32), ``softcap`` > 0 and ``window_left`` >= 0 switch on the score modifiers of
    test_paged.py:92-110.  ``k_scales`` / ``v_scales`` (fp32, ``[kv_heads]`` or
    ``[blocks, kv_heads]``) replace ``fp8_scale`` for an FP8 cache."""
    query_len = 1
    q3 = query
    if query.dim() == 4:  # [S, query_len, H, D]: several query tokens per sequence, causal among themselves
        query_len = query.shape[1]
        q3 = query.reshape(query.shape[0] * query_len, query.shape[2], query.shape[3])
    pr = _problem(q3, key_cache, value_cache, block_tables, context_lens, scale, block_size,
                  kv_strides, fp8_scale, num_kv_heads)
    pr.num_seqs = query.shape[0]
    S, H, D = q3.shape
    out = torch.zeros(query.shape, dtype=query.dtype)
    out32 = torch.zeros(query.shape, dtype=torch.float32)
    if k_scales is not None:
        pitch = _scale_pitch(k_scales, v_scales, num_kv_heads, key_cache.shape[0])
        rc = lib().oracle_attention_ref_scaled(_ptr(out), _ptr(out32), _ptr(query), _ptr(key_cache),
                                               _ptr(value_cache), _ptr(block_tables), _ptr(context_lens),
                                               _ptr(sinks), _ptr(alibi_slopes), float(softcap), int(window_left),
                                               int(query_len), _ptr(k_scales), _ptr(v_scales), pitch,
                                               ctypes.byref(pr))
    elif alibi_slopes is not None or softcap > 0 or window_left >= 0 or query_len > 1:
        if alibi_slopes is not None:
            assert alibi_slopes.dtype == torch.float32 and alibi_slopes.is_contiguous() and alibi_slopes.numel() == H
        rc = lib().oracle_attention_ref_masked(_ptr(out), _ptr(out32), _ptr(query), _ptr(key_cache),
                                               _ptr(value_cache), _ptr(block_tables), _ptr(context_lens),
                                               _ptr(sinks), _ptr(alibi_slopes), float(softcap), int(window_left),
                                               int(query_len), ctypes.byref(pr))
    else:
        rc = lib().oracle_attention_ref(_ptr(out), _ptr(out32), _ptr(query), _ptr(key_cache),
                                        _ptr(value_cache), _ptr(block_tables), _ptr(context_lens),
                                        _ptr(sinks), ctypes.byref(pr))
    if rc != 0:
        raise MemoryError("oracle_attention_ref")
    return (out, out32) if want_f32 else out


def kernel_loop(query, key_cache, value_cache, block_tables, context_lens, *, scale, block_size,
                kv_strides, num_kv_heads, partition_size, sinks=None, fp8_scale=1.0,
                want_f32=False):
    """Arithmetic of the upstream single-pass kernel (paged_attention_kernel_loop.hpp:610-636)."""
    pr = _problem(query, key_cache, value_cache, block_tables, context_lens, scale, block_size,
                  kv_strides, fp8_scale, num_kv_heads)
    S, H, D = query.shape
    out = torch.zeros((S, H, D), dtype=query.dtype)
    out32 = torch.zeros((S, H, D), dtype=torch.float32)
    rc = lib().oracle_kernel_loop(_ptr(out), _ptr(out32), _ptr(query), _ptr(key_cache),
                                  _ptr(value_cache), _ptr(block_tables), _ptr(context_lens),
                                  _ptr(sinks), partition_size, ctypes.byref(pr))
    if rc != 0:
        raise MemoryError("oracle_kernel_loop")
    return (out, out32) if want_f32 else out


def kernel_partition(query, key_cache, value_cache, block_tables, context_lens, *, scale,
                     block_size, kv_strides, num_kv_heads, partition_size, max_num_partitions,
                     sinks=None, fp8_scale=1.0, fill=float("nan")):
    """Arithmetic of the upstream split-context kernel (paged_attention_kernel_v2.hpp:572-587).

    Returns (exp_sums, max_logits, tmp_out) with untouched slots holding ``fill``.
    """
    pr = _problem(query, key_cache, value_cache, block_tables, context_lens, scale, block_size,
                  kv_strides, fp8_scale, num_kv_heads)
    S, H, D = query.shape
    exp_sums = torch.full((S, H, max_num_partitions), fill, dtype=torch.float32)
    max_logits = torch.full((S, H, max_num_partitions), fill, dtype=torch.float32)
    tmp_out = torch.full((S, H, max_num_partitions, D), fill, dtype=torch.float32)
    rc = lib().oracle_kernel_partition(_ptr(exp_sums), _ptr(max_logits), _ptr(tmp_out), _ptr(query),
                                       _ptr(key_cache), _ptr(value_cache), _ptr(block_tables),
                                       _ptr(context_lens), _ptr(sinks), partition_size,
                                       max_num_partitions, ctypes.byref(pr))
    if rc != 0:
        raise MemoryError("oracle_kernel_partition")
    return exp_sums, max_logits, tmp_out


def kernel_reduce(exp_sums, max_logits, tmp_out, context_lens, *, partition_size, q_dtype,
                  want_f32=False):
    """Arithmetic of the upstream reduce kernel (paged_attention_kernel_v2.hpp:957-969)."""
    S, H, NP, D = tmp_out.shape
    pr = _Problem()
    pr.num_seqs, pr.num_heads, pr.num_kv_heads, pr.head_size = S, H, H, D
    pr.q_dtype = Q_BF16 if q_dtype == torch.bfloat16 else Q_F16
    out = torch.zeros((S, H, D), dtype=q_dtype)
    out32 = torch.zeros((S, H, D), dtype=torch.float32)
    assert exp_sums.is_contiguous() and max_logits.is_contiguous() and tmp_out.is_contiguous()
    lib().oracle_kernel_reduce(_ptr(out), _ptr(out32), _ptr(exp_sums), _ptr(max_logits),
                               _ptr(tmp_out), _ptr(context_lens), partition_size, NP,
                               ctypes.byref(pr))
    return (out, out32) if want_f32 else out


def f32_to_e4m3(values: torch.Tensor) -> torch.Tensor:
    """Element-wise fp32 -> E4M3 "fn" byte (round to nearest even, beyond 448 to NaN)."""
    src = values.to(torch.float32).contiguous()
    out = torch.empty(src.shape, dtype=torch.uint8)
    lib().oracle_f32_to_e4m3_array(_ptr(src), _ptr(out), ctypes.c_int64(src.numel()))
    return out


def f32_to_e5m2(values: torch.Tensor) -> torch.Tensor:
    """Element-wise fp32 -> E5M2 byte (round to nearest even, overflow to infinity)."""
    src = values.to(torch.float32).contiguous()
    out = torch.empty(src.shape, dtype=torch.uint8)
    lib().oracle_f32_to_e5m2_array(_ptr(src), _ptr(out), ctypes.c_int64(src.numel()))
    return out


def kv_cache_write(key, value, key_cache, value_cache, slot_mapping, *, block_size, kv_strides,
                   fp8_scale=1.0, e4m3=False, k_scales=None, v_scales=None):
    """Scatter the rows of `key`/`value` ([N, Hk, D], fp16/bf16) into the paged pools in place
    (the pool build of test_paged_fp8cache.py:171-203 as a per-token scatter)."""
    assert key.device.type == "cpu" and key.dim() == 3 and key.stride(2) == 1
    assert value.shape == key.shape and value.stride() == key.stride() and value.dtype == key.dtype
    assert key.dtype in (torch.float16, torch.bfloat16)
    assert slot_mapping.dtype == torch.int64 and slot_mapping.is_contiguous()
    fp8 = key_cache.dtype in (torch.float8_e5m2, torch.float8_e4m3fn, torch.uint8) or e4m3
    if not fp8:
        assert key_cache.dtype == key.dtype
    assert value_cache.dtype == key_cache.dtype and key_cache.is_contiguous() and value_cache.is_contiguous()
    w = _KvWrite()
    w.num_tokens, w.num_kv_heads, w.head_size = key.shape
    w.block_size = block_size
    w.kv_block_stride, w.kv_token_stride, w.kv_head_stride = kv_strides
    w.src_token_stride, w.src_head_stride = key.stride(0), key.stride(1)
    w.src_dtype = Q_BF16 if key.dtype == torch.bfloat16 else Q_F16
    w.cache_dtype = (KV_E4M3 if (e4m3 or key_cache.dtype == torch.float8_e4m3fn) else KV_E5M2) if fp8 else KV_SAME_AS_Q
    w.num_pool_blocks = key_cache.shape[0]
    w.fp8_scale = fp8_scale
    if k_scales is not None:
        pitch = _scale_pitch(k_scales, v_scales, w.num_kv_heads, key_cache.shape[0])
        lib().oracle_kv_cache_write_scaled(_ptr(key), _ptr(value), _ptr(key_cache), _ptr(value_cache),
                                           _ptr(slot_mapping), _ptr(k_scales), _ptr(v_scales), pitch,
                                           ctypes.byref(w))
        return
    lib().oracle_kv_cache_write(_ptr(key), _ptr(value), _ptr(key_cache), _ptr(value_cache),
                                _ptr(slot_mapping), ctypes.byref(w))


def num_threads() -> int:
    return lib().oracle_num_threads()


def set_num_threads(n: int) -> None:
    lib().oracle_set_num_threads(n)
