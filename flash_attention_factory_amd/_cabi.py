"""ctypes binding of libfa_paged_attention.so (declarations: include/fa_paged_attention.h,
include/fa_kv_cache.h).

There is no fallback: if the HIP library is missing or a call fails, this raises.
"""
from __future__ import annotations

import ctypes
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
# FA_PAGED_ATTENTION_LIBRARY names another build of the same sources (a debug build with the in-kernel
# timeline or a cost probe compiled in); there is no fallback to anything that is not this library
LIBRARY = os.path.abspath(os.environ.get("FA_PAGED_ATTENTION_LIBRARY") or os.path.join(_PKG, "libfa_paged_attention.so"))

FA_OK = 0
FA_ERR_NULL_POINTER = 1
FA_ERR_UNSUPPORTED_HEAD_OR_BLOCK_SIZE = 2
FA_ERR_UNSUPPORTED_GROUP = 3
FA_ERR_UNSUPPORTED_DTYPE = 4
FA_ERR_PARTITION_OVERFLOW = 5
FA_ERR_BAD_SHAPE = 6
FA_ERR_RUNTIME = 7
FA_ERR_SCRATCH_TOO_SMALL = 8

# bytes of the library-owned scratch of fa_paged_attention_reduce_static_scratch
FA_STATIC_SCRATCH_BYTES = 64 << 20

FA_DTYPE_F16 = 0
FA_DTYPE_BF16 = 1

EXPORTS = (
    "fa_paged_attention_loop",
    "fa_paged_attention_reduce",
    "fa_paged_attention_fp8_loop",
    "fa_paged_attention_fp8_reduce",
    "fa_last_error",
    "fa_paged_attention_abi_version",
    "fa_kv_cache_write",
    "fa_paged_attention_reduce_static_scratch",
    "fa_paged_attention_kernel_status",
    "fa_paged_attention_reduce_plan",
    "fa_paged_attention_init",
)

ABI_REVISION = 8

FA_KV_CACHE_16BIT = 0
FA_KV_CACHE_E5M2 = 1
FA_KV_CACHE_E4M3 = 2

FA_FP8_E5M2 = 0
FA_FP8_E4M3 = 1

FA_KV_SCALE_TENSOR = 0
FA_KV_SCALE_HEAD = 1
FA_KV_SCALE_BLOCK = 2

FA_SCHEDULE_AUTO = 0
FA_SCHEDULE_GRID = 1
FA_SCHEDULE_GRID_LDS = 2
FA_SCHEDULE_SPLIT = 3
FA_SCHEDULE_GRID_VALU = 4
FA_SCHEDULE_VALU = 5

FA_SPLIT_FORM_GRID = 0
FA_SPLIT_FORM_SEGMENT = 1
FA_SPLIT_FORM_LOOP = 2

FA_MASK_ALIBI = 1
FA_MASK_SOFTCAP = 2
FA_MASK_WINDOW = 4


class _Versioned(ctypes.Structure):
    """A struct that begins with `struct_size`: set on construction to the size declared here, which
    is how the library knows which fields the caller's revision of the header has."""

    def __init__(self, *args, **kw):
        super().__init__(*args, **kw)
        if "struct_size" not in kw:
            self.struct_size = ctypes.sizeof(type(self))


class Shape(_Versioned):
    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("num_seqs", ctypes.c_int32),
        ("num_heads", ctypes.c_int32),
        ("num_kv_heads", ctypes.c_int32),
        ("head_size", ctypes.c_int32),
        ("block_size", ctypes.c_int32),
        ("max_blocks_per_seq", ctypes.c_int32),
        ("max_num_partitions", ctypes.c_int32),
        ("partition_size", ctypes.c_int32),
        ("kv_block_stride", ctypes.c_int64),
        ("kv_token_stride", ctypes.c_int64),
        ("kv_head_stride", ctypes.c_int64),
        ("q_dtype", ctypes.c_int32),
        ("num_pool_blocks", ctypes.c_int32),
    ]


class Options(_Versioned):
    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("sinks", ctypes.c_void_p),
        ("alibi_slopes", ctypes.c_void_p),
        ("softcap", ctypes.c_float),
        ("fp8_scale", ctypes.c_float),
        ("stream", ctypes.c_void_p),
        ("elapsed_us", ctypes.POINTER(ctypes.c_float)),
        ("validate_only", ctypes.c_int32),
        ("kv_fp8_format", ctypes.c_int32),
        ("mask_flags", ctypes.c_int32),
        ("window_left", ctypes.c_int32),
        ("query_len", ctypes.c_int32),
        ("kv_scale_mode", ctypes.c_int32),
        ("k_scales", ctypes.c_void_p),
        ("v_scales", ctypes.c_void_p),
        ("schedule", ctypes.c_int32),
        ("spin_limit", ctypes.c_int32),
        ("segment_partitions", ctypes.c_int32),
    ]


class KvWriteShape(_Versioned):
    _fields_ = [
        ("struct_size", ctypes.c_uint32),
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
    ]


class SplitPlan(_Versioned):
    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("form", ctypes.c_int32),
        ("compute_units", ctypes.c_int32),
        ("work_groups", ctypes.c_int32),
        ("kv_heads_per_item", ctypes.c_int32),
    ]


def set_kv_scales(op: "Options", k_scales, v_scales, num_kv_heads: int, num_pool_blocks: int, device) -> None:
    """Fill the scale fields of `op` from two fp32 device tensors shaped [num_kv_heads]
    (per-head scales) or [num_pool_blocks, num_kv_heads] (per-block scales)."""
    import torch
    if (k_scales is None) != (v_scales is None):
        raise PagedAttentionError(FA_ERR_NULL_POINTER, "k_scales and v_scales come together")
    if k_scales is None:
        return
    for t in (k_scales, v_scales):
        if t.dtype != torch.float32 or not t.is_contiguous() or t.device != device or t.shape != k_scales.shape:
            raise PagedAttentionError(FA_ERR_BAD_SHAPE, "k_scales / v_scales must be contiguous fp32 device tensors of one shape")
    if tuple(k_scales.shape) == (num_kv_heads,):
        op.kv_scale_mode = FA_KV_SCALE_HEAD
    elif tuple(k_scales.shape) == (num_pool_blocks, num_kv_heads):
        op.kv_scale_mode = FA_KV_SCALE_BLOCK
    else:
        raise PagedAttentionError(FA_ERR_BAD_SHAPE,
                                  f"scales of shape {tuple(k_scales.shape)} are neither [{num_kv_heads}] (per kv head) "
                                  f"nor [{num_pool_blocks}, {num_kv_heads}] (per block and kv head)")
    op.k_scales = k_scales.data_ptr()
    op.v_scales = v_scales.data_ptr()


def require_same_device(anchor_name: str, anchor, named_tensors) -> None:
    """Every tensor whose pointer goes to a kernel must live on the anchor tensor's device: a host
    pointer in a kernel argument is a GPU memory fault, not an exception.  None entries are skipped."""
    for name, t in named_tensors:
        if t is not None and t.device != anchor.device:
            raise PagedAttentionError(FA_ERR_BAD_SHAPE,
                                      f"{name} is on {t.device}, {anchor_name} on {anchor.device}: every tensor "
                                      f"must live on the device of {anchor_name}")


class PagedAttentionError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"[fa_status {code}] {message}")
        self.code = code


_lib = None


def load() -> ctypes.CDLL:
    """Load the in-tree HIP library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIBRARY):
        raise RuntimeError(
            f"{LIBRARY} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "(there is no CPU or PyTorch fallback for the paged-attention kernels)")
    L = ctypes.CDLL(LIBRARY)
    P = ctypes.c_void_p
    common = [P, P, P, P, P, P, ctypes.c_float, ctypes.c_int32]
    tail = [ctypes.POINTER(Shape), ctypes.POINTER(Options)]
    for name in ("fa_paged_attention_loop", "fa_paged_attention_fp8_loop", "fa_paged_attention_reduce_static_scratch"):
        fn = getattr(L, name)
        fn.argtypes = common + tail
        fn.restype = ctypes.c_int32
    for name in ("fa_paged_attention_reduce", "fa_paged_attention_fp8_reduce"):
        fn = getattr(L, name)
        fn.argtypes = common + [P, P, P] + tail
        fn.restype = ctypes.c_int32
    L.fa_kv_cache_write.argtypes = [P, P, P, P, P, ctypes.POINTER(KvWriteShape), ctypes.POINTER(Options)]
    L.fa_kv_cache_write.restype = ctypes.c_int32
    L.fa_last_error.restype = ctypes.c_char_p
    L.fa_paged_attention_abi_version.restype = ctypes.c_int32
    L.fa_paged_attention_reduce_plan.argtypes = [ctypes.POINTER(Shape), ctypes.POINTER(Options), ctypes.c_int32,
                                                 ctypes.c_int32, ctypes.c_int32, ctypes.POINTER(SplitPlan)]
    L.fa_paged_attention_reduce_plan.restype = ctypes.c_int32
    L.fa_paged_attention_init.argtypes = []
    L.fa_paged_attention_init.restype = ctypes.c_int32
    L.fa_paged_attention_kernel_status.argtypes = [P, ctypes.c_int32]
    L.fa_paged_attention_kernel_status.restype = ctypes.c_int32
    if L.fa_paged_attention_abi_version() != ABI_REVISION:
        raise RuntimeError(f"{LIBRARY} has ABI revision {L.fa_paged_attention_abi_version()}, this binding is "
                           f"written for {ABI_REVISION}: rebuild the library")
    _lib = L
    return L


def init() -> None:
    """What the library sets up once per GPU, now, on the current device (fa_paged_attention_init): to be
    called outside a HIP graph capture before calls are recorded into one."""
    check(load().fa_paged_attention_init())


def kernel_status(stream: int = 0, clear: bool = True) -> None:
    """Raise PagedAttentionError if a persistent kernel of the current GPU gave up a wait since the
    status word was last cleared (waits for `stream`, a raw hipStream_t, first).  For callers of the
    asynchronous paths, at a synchronisation point of their own; timed calls look by themselves."""
    check(load().fa_paged_attention_kernel_status(stream or None, 1 if clear else 0))


def check(code: int) -> None:
    if code != FA_OK:
        raise PagedAttentionError(code, load().fa_last_error().decode())
