"""CPU-only checks of the C ABI: the library loads, exports every function the header
declares, and rejects bad arguments with the documented status codes (validate_only
launches nothing, so no GPU is needed)."""
import ctypes
import os
import re

import pytest

from flash_attention_factory_amd import _cabi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def L():
    if not os.path.exists(_cabi.LIBRARY):
        from flash_attention_factory_amd import _build
        _build.build()
    return _cabi.load()


def test_header_symbols_are_exported(L):
    declared = set()
    for name in ("fa_paged_attention.h", "fa_kv_cache.h"):
        header = open(os.path.join(ROOT, "include", name)).read()
        body = header[header.index('extern "C"'):]
        declared |= set(re.findall(r"\b(fa_[a-z0-9_]+)\s*\(", body))
    assert declared == set(_cabi.EXPORTS), declared ^ set(_cabi.EXPORTS)
    for name in declared:
        assert hasattr(L, name), name
    assert L.fa_paged_attention_abi_version() == 8 == _cabi.ABI_REVISION


def test_struct_layouts_match_header():
    # field order and sizes of the three structs as the headers lay them out (revision 8: every
    # struct begins with struct_size)
    assert _cabi.Shape.struct_size.offset == 0 and _cabi.Shape.num_seqs.offset == 4
    assert ctypes.sizeof(_cabi.Shape) == 4 + 8 * 4 + 4 + 3 * 8 + 2 * 4 == 72
    assert _cabi.Shape.kv_block_stride.offset == 40
    assert _cabi.Shape.num_pool_blocks.offset == 68
    assert _cabi.Options.struct_size.offset == 0 and _cabi.Options.sinks.offset == 8
    assert ctypes.sizeof(_cabi.Options) == 104
    assert _cabi.Options.schedule.offset == 88 and _cabi.Options.spin_limit.offset == 92
    assert _cabi.Options.segment_partitions.offset == 96
    assert _cabi.Options.kv_scale_mode.offset == 68
    assert _cabi.Options.k_scales.offset == 72 and _cabi.Options.v_scales.offset == 80
    assert _cabi.Options.query_len.offset == 64
    assert _cabi.Options.mask_flags.offset == 56 and _cabi.Options.window_left.offset == 60
    assert _cabi.Options.elapsed_us.offset == 40
    assert ctypes.sizeof(_cabi.SplitPlan) == 20 and _cabi.SplitPlan.kv_heads_per_item.offset == 16
    assert ctypes.sizeof(_cabi.KvWriteShape) == 4 + 4 * 4 + 4 + 5 * 8 + 2 * 4 + 8 == 80
    assert _cabi.KvWriteShape.src_dtype.offset == 64 and _cabi.KvWriteShape.num_pool_blocks.offset == 72
    # a new struct says how large it is
    assert _cabi.Shape().struct_size == 72 and _cabi.Options().struct_size == 104 and _cabi.KvWriteShape().struct_size == 80


def test_header_struct_sizes_agree_with_the_compiler(tmp_path):
    """The headers as a C compiler lays them out: sizes and the offsets the binding relies on."""
    import subprocess
    src = tmp_path / "sizes.c"
    src.write_text(
        '#include <stddef.h>\n#include <stdio.h>\n#include "fa_kv_cache.h"\n'
        'int main(void) {\n'
        '  fa_paged_attention_shape s = FA_PAGED_ATTENTION_SHAPE_INIT;\n'
        '  fa_paged_attention_options o = FA_PAGED_ATTENTION_OPTIONS_INIT;\n'
        '  fa_kv_cache_write_shape k = FA_KV_CACHE_WRITE_SHAPE_INIT;\n'
        '  printf("%u %u %u %zu %zu %zu %zu %d\\n", s.struct_size, o.struct_size, k.struct_size,\n'
        '         offsetof(fa_paged_attention_shape, num_pool_blocks), offsetof(fa_paged_attention_options, schedule),\n'
        '         offsetof(fa_paged_attention_options, spin_limit), offsetof(fa_kv_cache_write_shape, num_pool_blocks),\n'
        '         s.num_seqs + o.schedule + k.num_tokens);\n'
        '  return 0;\n}\n')
    exe = tmp_path / "sizes"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)],
                   check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()
    assert [int(x) for x in out] == [72, 104, 80, 68, 88, 92, 72, 0]


def test_shorter_and_longer_structs(L):
    """struct_size tells the library which fields the caller's header has: an options struct cut
    before `schedule` (a caller built before the field was appended) validates with the field at its
    default; sizes the library cannot make sense of are refused."""
    def call(shape_size=None, options_size=None, schedule=0, kv=False):
        op = _cabi.Options()
        op.validate_only = 1
        op.schedule = schedule
        if options_size is not None:
            op.struct_size = options_size
        p = 0x1000
        if kv:
            sh = _cabi.KvWriteShape()
            for k, v in dict(num_tokens=4, num_kv_heads=2, head_size=128, block_size=16, kv_block_stride=2 * 16 * 128,
                             kv_token_stride=128, kv_head_stride=16 * 128, src_dtype=0, cache_dtype=1, num_pool_blocks=8).items():
                setattr(sh, k, v)
            if shape_size is not None:
                sh.struct_size = shape_size
            return L.fa_kv_cache_write(p, p, p, p, p, ctypes.byref(sh), ctypes.byref(op)), L.fa_last_error().decode()
        sh = _shape()
        if shape_size is not None:
            sh.struct_size = shape_size
        return L.fa_paged_attention_loop(p, p, p, p, p, p, 0.1, 0, ctypes.byref(sh), ctypes.byref(op)), L.fa_last_error().decode()

    assert call() == (_cabi.FA_OK, "")
    assert call(schedule=9)[0] == _cabi.FA_ERR_BAD_SHAPE                      # the field is read ...
    before_schedule = _cabi.Options.schedule.offset
    assert call(options_size=before_schedule, schedule=9) == (_cabi.FA_OK, "")  # ... unless the caller's struct ends before it
    assert call(options_size=_cabi.Options.spin_limit.offset, schedule=9)[0] == _cabi.FA_ERR_BAD_SHAPE
    # the shortest struct this test may pass ends with validate_only (without it the call would launch)
    assert call(options_size=_cabi.Options.validate_only.offset + 4, schedule=9) == (_cabi.FA_OK, "")
    for bad in (0, 2, 97, 108, 1 << 20):
        rc, msg = call(options_size=bad)
        assert rc == _cabi.FA_ERR_BAD_SHAPE and "options.struct_size" in msg, (bad, msg)
    for bad in (0, 36, 68, 70, 76, 4096):  # every field of the shape is needed
        rc, msg = call(shape_size=bad)
        assert rc == _cabi.FA_ERR_BAD_SHAPE and "shape.struct_size" in msg, (bad, msg)
    assert call(kv=True) == (_cabi.FA_OK, "")
    for bad in (0, 72, 84):
        rc, msg = call(kv=True, shape_size=bad)
        assert rc == _cabi.FA_ERR_BAD_SHAPE and "shape.struct_size" in msg, (bad, msg)
    rc, msg = call(kv=True, options_size=0)
    assert rc == _cabi.FA_ERR_BAD_SHAPE and "options.struct_size" in msg


def _shape(**kw):
    s = _cabi.Shape()
    base = dict(num_seqs=2, num_heads=8, num_kv_heads=2, head_size=128, block_size=16,
                max_blocks_per_seq=4, max_num_partitions=1, partition_size=0,
                kv_block_stride=2 * 16 * 128, kv_token_stride=128, kv_head_stride=16 * 128,
                q_dtype=_cabi.FA_DTYPE_F16, num_pool_blocks=8)
    base.update(kw)
    for k, v in base.items():
        setattr(s, k, v)
    return s


def _call(L, split=False, fp8=False, shape=None, ptr=0x1000, scratch=0x1000, max_ctx=0, fp8_format=0,
          mask_flags=0, alibi=None, softcap=0.0, window_left=0, query_len=0, scale_mode=0, k_scales=None,
          v_scales=None, schedule=0):
    op = _cabi.Options()
    op.schedule = schedule
    op.kv_scale_mode, op.k_scales, op.v_scales = scale_mode, k_scales, v_scales
    op.query_len = query_len
    op.validate_only = 1
    op.kv_fp8_format = fp8_format
    op.mask_flags, op.alibi_slopes, op.softcap, op.window_left = mask_flags, alibi, softcap, window_left
    name = "fa_paged_attention_" + ("fp8_" if fp8 else "") + ("reduce" if split else "loop")
    args = [ptr, ptr, ptr, ptr, ptr, ptr, 0.1, max_ctx]
    if split:
        args += [scratch, scratch, scratch]
    sh = shape or _shape()
    return getattr(L, name)(*args, ctypes.byref(sh), ctypes.byref(op)), L.fa_last_error().decode()


@pytest.mark.parametrize("split", [False, True])
@pytest.mark.parametrize("fp8", [False, True])
def test_valid_arguments_pass(L, split, fp8):
    rc, msg = _call(L, split, fp8)
    assert rc == _cabi.FA_OK and msg == ""


def test_fp8_format_is_checked_on_fp8_entries_only(L):
    assert _call(L, fp8=True, fp8_format=_cabi.FA_FP8_E4M3)[0] == _cabi.FA_OK
    assert _call(L, fp8=True, split=True, fp8_format=_cabi.FA_FP8_E4M3)[0] == _cabi.FA_OK
    assert _call(L, fp8=True, fp8_format=7)[0] == _cabi.FA_ERR_UNSUPPORTED_DTYPE
    assert _call(L, fp8=False, fp8_format=7)[0] == _cabi.FA_OK   # 16-bit entries ignore the field


def test_score_modifier_arguments(L):
    assert _call(L, mask_flags=0, softcap=-3.0, window_left=-9)[0] == _cabi.FA_OK      # ignored, as upstream
    assert _call(L, mask_flags=_cabi.FA_MASK_ALIBI, alibi=0x1000)[0] == _cabi.FA_OK
    assert _call(L, mask_flags=_cabi.FA_MASK_ALIBI)[0] == _cabi.FA_ERR_NULL_POINTER
    assert _call(L, mask_flags=_cabi.FA_MASK_SOFTCAP, softcap=30.0)[0] == _cabi.FA_OK
    assert _call(L, mask_flags=_cabi.FA_MASK_SOFTCAP, softcap=0.0)[0] == _cabi.FA_ERR_BAD_SHAPE
    assert _call(L, split=True, mask_flags=_cabi.FA_MASK_WINDOW, window_left=0)[0] == _cabi.FA_OK
    assert _call(L, mask_flags=_cabi.FA_MASK_WINDOW, window_left=-1)[0] == _cabi.FA_ERR_BAD_SHAPE
    assert _call(L, mask_flags=8)[0] == _cabi.FA_ERR_BAD_SHAPE


def test_query_len_limits(L):
    assert _call(L, query_len=4)[0] == _cabi.FA_OK                      # group 4 x 4 tokens = 16 columns
    assert _call(L, query_len=5)[0] == _cabi.FA_OK                      # two launches: 4 tokens, then 1
    assert _call(L, query_len=64)[0] == _cabi.FA_OK
    rc, msg = _call(L, query_len=65)
    assert rc == _cabi.FA_ERR_BAD_SHAPE and "query_len" in msg
    assert _call(L, split=True, query_len=2)[0] == _cabi.FA_OK
    assert _call(L, query_len=-1)[0] == _cabi.FA_ERR_BAD_SHAPE


def test_error_codes(L):
    assert _call(L, ptr=0)[0] == _cabi.FA_ERR_NULL_POINTER
    assert _call(L, split=True, scratch=0)[0] == _cabi.FA_ERR_NULL_POINTER
    rc, msg = _call(L, shape=_shape(head_size=96))
    assert rc == _cabi.FA_ERR_UNSUPPORTED_HEAD_OR_BLOCK_SIZE and "Unsupported head size or block size" in msg
    assert _call(L, shape=_shape(block_size=24))[0] == _cabi.FA_ERR_UNSUPPORTED_HEAD_OR_BLOCK_SIZE
    assert _call(L, shape=_shape(block_size=8))[0] == _cabi.FA_ERR_UNSUPPORTED_HEAD_OR_BLOCK_SIZE
    rc, msg = _call(L, shape=_shape(num_heads=7))
    assert rc == _cabi.FA_ERR_UNSUPPORTED_GROUP and "Unsupported number of queries per token" in msg
    assert _call(L, shape=_shape(num_heads=34, num_kv_heads=2))[0] == _cabi.FA_ERR_UNSUPPORTED_GROUP
    assert _call(L, shape=_shape(q_dtype=5))[0] == _cabi.FA_ERR_UNSUPPORTED_DTYPE
    assert _call(L, shape=_shape(num_seqs=0))[0] == _cabi.FA_ERR_BAD_SHAPE
    assert _call(L, shape=_shape(kv_token_stride=100))[0] == _cabi.FA_ERR_BAD_SHAPE
    assert _call(L, ptr=0x1008)[0] == _cabi.FA_ERR_BAD_SHAPE
    # 4 blocks of 16 tokens cannot hold 100 tokens
    assert _call(L, max_ctx=100)[0] == _cabi.FA_ERR_BAD_SHAPE
    # split path: one partition of 512 tokens cannot hold 600
    rc, msg = _call(L, split=True, shape=_shape(max_blocks_per_seq=64), max_ctx=600)
    assert rc == _cabi.FA_ERR_PARTITION_OVERFLOW and "partitions" in msg
    assert _call(L, split=True, shape=_shape(partition_size=48))[0] == _cabi.FA_ERR_BAD_SHAPE
    # the same shape is fine for the loop entry, which has no partitions
    assert _call(L, shape=_shape(partition_size=48))[0] == _cabi.FA_OK
    # NULL shape / NULL options
    op = _cabi.Options(); op.validate_only = 1
    assert L.fa_paged_attention_loop(1, 1, 1, 1, 1, 1, 0.1, 0, None, ctypes.byref(op)) == _cabi.FA_ERR_NULL_POINTER


def test_run_shim_rejects_cpu_tensors():
    import torch
    from flash_attention_factory_amd import runner, workloads as W
    w = W.make_config(0)
    with pytest.raises(RuntimeError, match="GPU only"):
        runner.run_workload(w, "loop")


def test_every_tensor_must_be_on_the_anchor_device():
    # the check the run shims make before any pointer reaches a kernel, on devices a CPU box has
    import torch
    q = torch.empty(2, device="meta")
    ok = torch.empty(2, device="meta")
    host = torch.empty(2)
    _cabi.require_same_device("query", q, [("output", ok), ("sinks", None)])
    for name in ("output", "key_cache", "value_cache", "block_tables", "context_lens", "sinks", "max_logits",
                 "exp_sums", "tem_output", "slot_mapping"):
        with pytest.raises(_cabi.PagedAttentionError, match=name):
            _cabi.require_same_device("query", q, [("other", ok), (name, host)])


def test_workload_generators_are_deterministic():
    import torch
    from flash_attention_factory_amd import workloads as W
    a, b = W.make_config(0), W.make_config(0)
    assert torch.equal(a.query, b.query) and torch.equal(a.key_cache, b.key_cache)
    assert torch.equal(a.block_tables, b.block_tables) and torch.equal(a.context_lens, b.context_lens)
    # every sequence's blocks are distinct pool blocks, no block shared between sequences
    used = []
    for s in range(a.num_seqs):
        nb = (int(a.context_lens[s]) + a.block_size - 1) // a.block_size
        used += a.block_tables[s, :nb].tolist()
    assert len(used) == len(set(used)) and max(used) < a.key_cache.shape[0]
    assert a.algorithmic_bytes() == int(a.context_lens.sum()) * 8 * 64 * 2 * 2 + 2 * 4 * 8 * 64 * 2 + \
        sum((int(n) + 15) // 16 for n in a.context_lens) * 4 + 4 * 4
    g = W.make_test_shaped(batch_size=2, nheads=8, nheads_k=2, d=64, seqlen_k=339, varlen=True, has_sinks=True)
    assert g.partition_size == 256 and g.key_cache.shape == (12, 64, 2, 64)
    assert int(g.context_lens.min()) >= 319 and int(g.context_lens.max()) <= 339


def _kv_write(L, ptr=0x1000, slots=0x1000, scale_mode=0, k_scales=None, v_scales=None, **kw):
    sh = _cabi.KvWriteShape()
    base = dict(num_tokens=4, num_kv_heads=2, head_size=128, block_size=16,
                kv_block_stride=2 * 16 * 128, kv_token_stride=128, kv_head_stride=16 * 128,
                src_token_stride=0, src_head_stride=0, src_dtype=_cabi.FA_DTYPE_F16,
                cache_dtype=_cabi.FA_KV_CACHE_E5M2, num_pool_blocks=8)
    base.update(kw)
    for k, v in base.items():
        setattr(sh, k, v)
    op = _cabi.Options()
    op.validate_only = 1
    op.kv_scale_mode, op.k_scales, op.v_scales = scale_mode, k_scales, v_scales
    return L.fa_kv_cache_write(ptr, ptr, ptr, ptr, slots, ctypes.byref(sh), ctypes.byref(op)), L.fa_last_error().decode()


def test_kv_cache_write_argument_checks(L):
    assert _kv_write(L) == (_cabi.FA_OK, "")
    assert _kv_write(L, cache_dtype=_cabi.FA_KV_CACHE_16BIT, src_dtype=_cabi.FA_DTYPE_BF16)[0] == _cabi.FA_OK
    assert _kv_write(L, ptr=0)[0] == _cabi.FA_ERR_NULL_POINTER
    assert _kv_write(L, slots=0)[0] == _cabi.FA_ERR_NULL_POINTER
    assert _kv_write(L, src_dtype=5)[0] == _cabi.FA_ERR_UNSUPPORTED_DTYPE
    assert _kv_write(L, cache_dtype=_cabi.FA_KV_CACHE_E4M3)[0] == _cabi.FA_OK
    assert _kv_write(L, cache_dtype=3)[0] == _cabi.FA_ERR_UNSUPPORTED_DTYPE
    assert _kv_write(L, head_size=100)[0] == _cabi.FA_ERR_UNSUPPORTED_HEAD_OR_BLOCK_SIZE
    assert _kv_write(L, num_pool_blocks=0)[0] == _cabi.FA_ERR_BAD_SHAPE
    assert _kv_write(L, kv_token_stride=64)[0] == _cabi.FA_ERR_BAD_SHAPE       # shorter than a row
    assert _kv_write(L, kv_head_stride=16 * 128 + 4)[0] == _cabi.FA_ERR_BAD_SHAPE  # misaligned
    assert _kv_write(L, src_token_stride=100)[0] == _cabi.FA_ERR_BAD_SHAPE
    assert _kv_write(L, ptr=0x1008)[0] == _cabi.FA_ERR_BAD_SHAPE
    assert _kv_write(L, num_tokens=0)[0] == _cabi.FA_OK


def test_kv_scale_argument_checks(L):
    """Per-head / per-block scales: FP8 entries and the writer only, both arrays, a known pool size."""
    HEAD, BLOCK = _cabi.FA_KV_SCALE_HEAD, _cabi.FA_KV_SCALE_BLOCK
    for split in (False, True):
        assert _call(L, split=split, fp8=True, scale_mode=HEAD, k_scales=0x1000, v_scales=0x2000)[0] == _cabi.FA_OK
        assert _call(L, split=split, fp8=True, scale_mode=BLOCK, k_scales=0x1000, v_scales=0x2000)[0] == _cabi.FA_OK
        rc, msg = _call(L, split=split, fp8=True, scale_mode=HEAD, k_scales=0x1000)
        assert rc == _cabi.FA_ERR_NULL_POINTER and "v_scales" in msg
        assert _call(L, split=split, fp8=True, scale_mode=3, k_scales=0x1000, v_scales=0x1000)[0] == _cabi.FA_ERR_BAD_SHAPE
        assert _call(L, split=split, fp8=True, scale_mode=HEAD, k_scales=0x1002, v_scales=0x1000)[0] == _cabi.FA_ERR_BAD_SHAPE
        rc, msg = _call(L, split=split, fp8=True, scale_mode=BLOCK, k_scales=0x1000, v_scales=0x1000,
                        shape=_shape(num_pool_blocks=0))
        assert rc == _cabi.FA_ERR_BAD_SHAPE and "num_pool_blocks" in msg
        # a 16-bit cache has no scales: the fields are not read
        assert _call(L, split=split, fp8=False, scale_mode=7)[0] == _cabi.FA_OK
    assert _kv_write(L, scale_mode=HEAD, k_scales=0x1000, v_scales=0x1000)[0] == _cabi.FA_OK
    assert _kv_write(L, scale_mode=BLOCK, k_scales=0x1000, v_scales=0x1000)[0] == _cabi.FA_OK
    assert _kv_write(L, scale_mode=BLOCK, k_scales=0x1000)[0] == _cabi.FA_ERR_NULL_POINTER
    assert _kv_write(L, scale_mode=9, k_scales=0x1000, v_scales=0x1000)[0] == _cabi.FA_ERR_BAD_SHAPE
    assert _kv_write(L, scale_mode=9, cache_dtype=_cabi.FA_KV_CACHE_16BIT)[0] == _cabi.FA_OK


def test_schedule_values(L):
    for split in (False, True):
        for fp8 in (False, True):
            for schedule in (0, 1, 2, 3, 4, 5):  # the LDS and dot-product forms fall back to the grid form where they do not apply
                assert _call(L, split=split, fp8=fp8, schedule=schedule)[0] == _cabi.FA_OK
            code, text = _call(L, split=split, fp8=fp8, schedule=6)
            assert code == _cabi.FA_ERR_BAD_SHAPE and "schedule" in text


def test_static_scratch_rejects_what_does_not_fit(L):
    # the entry point that allocates nothing: a fixed array holds its scratch, so sizes have a limit
    sh = _cabi.Shape()
    for k, v in dict(num_seqs=64, num_heads=64, num_kv_heads=8, head_size=128, block_size=16, max_blocks_per_seq=2048,
                     max_num_partitions=64, partition_size=0, kv_block_stride=8 * 16 * 128, kv_token_stride=128,
                     kv_head_stride=16 * 128, q_dtype=_cabi.FA_DTYPE_F16, num_pool_blocks=1 << 16).items():
        setattr(sh, k, v)
    op = _cabi.Options()
    op.validate_only = 1
    p = 0x1000
    rc = L.fa_paged_attention_reduce_static_scratch(p, p, p, p, p, p, 0.1, 0, ctypes.byref(sh), ctypes.byref(op))
    assert rc == _cabi.FA_ERR_SCRATCH_TOO_SMALL and b"static scratch holds" in L.fa_last_error()
    sh.num_seqs = 8  # 8 * 64 * 64 slots x 130 floats = 17 MB: fits
    assert L.fa_paged_attention_reduce_static_scratch(p, p, p, p, p, p, 0.1, 0, ctypes.byref(sh), ctypes.byref(op)) == 0
    elapsed = (ctypes.c_float * 2)()
    op.elapsed_us = ctypes.cast(elapsed, ctypes.POINTER(ctypes.c_float))
    rc = L.fa_paged_attention_reduce_static_scratch(p, p, p, p, p, p, 0.1, 0, ctypes.byref(sh), ctypes.byref(op))
    assert rc == _cabi.FA_ERR_BAD_SHAPE and b"elapsed_us must be NULL" in L.fa_last_error()
