"""``kv_cache_write.run``: scatter new K/V token rows into the paged pools the decode
kernels read, rounding to FP8 (E5M2, or E4M3 for ``torch.float8_e4m3fn`` pools) when the pools hold bytes.

Upstream has no extension module for this step; its tests build the pools with tensor
casts (test_paged_fp8cache.py:171-203: ``k_cache_paged.to(torch.float8_e5m2)``).  The
call below produces the same bytes on the device: ``key``/``value`` are
``[tokens, kv_heads, head_size]`` fp16 or bf16, the pools are
``[blocks, block_size, kv_heads, head_size]`` views exactly as the ``paged_attention_*``
modules take them, ``slot_mapping[n] = block * block_size + row`` (int64; a negative slot
skips the token).  Returns the kernel time in microseconds as a one-element list, or
``[]`` with ``timed=False`` (asynchronous on the current stream).  ``k_scales`` / ``v_scales``
(fp32 device tensors ``[kv_heads]`` or ``[blocks, kv_heads]``) replace the scalar
``fp8_scale``: a row is divided by the scale of its kv head, or of its destination block
and kv head, before rounding.
"""
from __future__ import annotations

import ctypes
from typing import List, Optional

import torch

from .. import _cabi


def run(key: torch.Tensor, value: torch.Tensor, key_cache: torch.Tensor, value_cache: torch.Tensor,
        slot_mapping: torch.Tensor, fp8_scale: float = 1.0, *, timed: bool = True,
        k_scales: Optional[torch.Tensor] = None, v_scales: Optional[torch.Tensor] = None) -> List[float]:
    L = _cabi.load()
    if not key.is_cuda:
        raise RuntimeError("the KV-cache writer runs on the GPU only: `key` is not a device tensor")
    _cabi.require_same_device("key", key, (("value", value), ("key_cache", key_cache), ("value_cache", value_cache),
                                           ("slot_mapping", slot_mapping)))
    if key.dtype not in (torch.float16, torch.bfloat16) or value.dtype != key.dtype:
        raise _cabi.PagedAttentionError(_cabi.FA_ERR_UNSUPPORTED_DTYPE, "key/value must both be fp16 or both bf16")
    if key.dim() != 3 or key.stride(2) != 1 or value.shape != key.shape or value.stride() != key.stride():
        raise _cabi.PagedAttentionError(_cabi.FA_ERR_BAD_SHAPE,
                                        "key and value must be [tokens, kv_heads, head_size] with equal "
                                        "strides and a contiguous last dimension")
    fp8 = key_cache.dtype in (torch.float8_e5m2, torch.float8_e4m3fn, torch.uint8)
    if (not fp8 and key_cache.dtype != key.dtype) or value_cache.dtype != key_cache.dtype:
        raise _cabi.PagedAttentionError(_cabi.FA_ERR_UNSUPPORTED_DTYPE,
                                        f"cache dtype {key_cache.dtype} is neither the source dtype nor an FP8 format")
    if key_cache.dim() != 4 or key_cache.stride(3) != 1 or value_cache.stride() != key_cache.stride() \
            or key_cache.size(2) != key.size(1) or key_cache.size(3) != key.size(2):
        raise _cabi.PagedAttentionError(_cabi.FA_ERR_BAD_SHAPE,
                                        "caches must be 4-D [blocks, block_size, kv_heads, head_size] views "
                                        "matching key/value, with equal strides")
    if slot_mapping.dtype != torch.int64 or not slot_mapping.is_contiguous() or slot_mapping.numel() != key.size(0):
        raise _cabi.PagedAttentionError(_cabi.FA_ERR_BAD_SHAPE, "slot_mapping must be contiguous int64 [tokens]")
    sh = _cabi.KvWriteShape()
    sh.num_tokens, sh.num_kv_heads, sh.head_size = key.shape
    sh.block_size = key_cache.size(1)
    sh.kv_block_stride, sh.kv_token_stride, sh.kv_head_stride = (
        key_cache.stride(0), key_cache.stride(1), key_cache.stride(2))
    sh.src_token_stride, sh.src_head_stride = key.stride(0), key.stride(1)
    sh.src_dtype = _cabi.FA_DTYPE_BF16 if key.dtype == torch.bfloat16 else _cabi.FA_DTYPE_F16
    sh.cache_dtype = _cabi.FA_KV_CACHE_16BIT if not fp8 else (
        _cabi.FA_KV_CACHE_E4M3 if key_cache.dtype == torch.float8_e4m3fn else _cabi.FA_KV_CACHE_E5M2)
    sh.num_pool_blocks = key_cache.size(0)
    elapsed = (ctypes.c_float * 2)(0.0, 0.0)
    op = _cabi.Options()
    op.fp8_scale = fp8_scale
    if k_scales is not None or v_scales is not None:
        if not fp8:
            raise _cabi.PagedAttentionError(_cabi.FA_ERR_UNSUPPORTED_DTYPE, "k_scales / v_scales belong to FP8 pools")
        _cabi.set_kv_scales(op, k_scales, v_scales, sh.num_kv_heads, sh.num_pool_blocks, key.device)
    op.stream = torch.cuda.current_stream(key.device).cuda_stream
    op.elapsed_us = ctypes.cast(elapsed, ctypes.POINTER(ctypes.c_float)) if timed else None
    with torch.cuda.device(key.device):
        _cabi.check(L.fa_kv_cache_write(key.data_ptr(), value.data_ptr(), key_cache.data_ptr(),
                                        value_cache.data_ptr(), slot_mapping.data_ptr(),
                                        ctypes.byref(sh), ctypes.byref(op)))
    return [elapsed[0]] if timed else []
