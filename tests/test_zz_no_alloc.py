"""The entry point that allocates nothing (fa_paged_attention_reduce_static_scratch, through the
C ABI) against fa_paged_attention_reduce on the same inputs: same kernels, scratch in the library's
fixed device array instead of caller-owned tensors, so `out` must be the same bits.  Two calls in
a row, the second on a smaller input, because every call on a GPU shares that GPU's array and finds
the previous call's contents in it, and the oracle."""
import pytest
import torch

from flash_attention_factory_amd import runner, workloads as W
from flash_attention_factory_amd.lib import paged_attention_reduce
from _torch_ref import call_oracle

pytestmark = pytest.mark.gpu


def _both(w_cpu, dev):
    w = w_cpu.to(dev)
    bufs = runner.alloc_buffers(w)
    runner.run_workload(w, "reduce", bufs)
    torch.cuda.synchronize()
    out = torch.full_like(bufs.out, float("nan"))
    kc, vc = runner.logical_cache_view(w, w.key_cache), runner.logical_cache_view(w, w.value_cache)
    got = paged_attention_reduce.run_static_scratch(
        out, w.query, kc, vc, w.block_tables, w.context_lens, w.num_heads // w.num_kv_heads, w.scale, w.block_size,
        int(w.block_tables.shape[1]) * w.block_size, w.max_num_partitions, w.sinks, partition_size=w.partition_size)
    assert got == []
    torch.cuda.synchronize()
    return bufs.out, out


def test_static_scratch_equals_caller_scratch_twice_in_a_row(oracle):
    assert torch.cuda.is_available(), "this test needs the GPU"
    dev = torch.device("cuda:0")
    # first a long-context GQA batch (segments of several partitions, sinks), then a smaller, ragged one
    # whose slots lie inside what the first call wrote
    big = W.make_test_shaped(batch_size=3, nheads=8, nheads_k=2, d=128, seqlen_k=5000, varlen=True, has_sinks=True)
    small = W.make_config(2, num_seqs=2, pool_blocks=1024, lens=[1500, 130])
    for w_cpu in (big, small):
        want, got = _both(w_cpu, dev)
        assert torch.isfinite(got.float()).all()
        assert torch.equal(got, want), f"{w_cpu.name}: static-scratch output differs from fa_paged_attention_reduce"
        _, ref32 = call_oracle(oracle.attention_ref, w_cpu, want_f32=True)
        torch.testing.assert_close(got.float().cpu(), ref32, atol=1e-2, rtol=1e-2)
