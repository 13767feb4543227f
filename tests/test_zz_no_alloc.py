"""The entry point that allocates nothing (fa_paged_attention_reduce_static_scratch, through the
C ABI) against fa_paged_attention_reduce on the same inputs: same kernels, scratch in the library's
fixed device array instead of caller-owned tensors, so `out` must be the same bits.  Two calls in
a row, the second on a smaller input, because every call on a GPU shares that GPU's array and finds
the previous call's contents in it, and the oracle."""
import pytest
import torch

from flash_attention_factory_amd import _cabi, runner, workloads as W
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


def test_static_scratch_in_a_hip_graph(oracle):
    """What the entry point is for: recorded into a HIP graph (after fa_paged_attention_init and one eager
    call of the shape), replayed several times with eager work, synchronisations and new inputs in
    between; every replay equals the eager result on the same inputs."""
    dev = torch.device("cuda:0")
    w_cpu = W.make_test_shaped(batch_size=3, nheads=8, nheads_k=2, d=128, seqlen_k=5000, varlen=True, has_sinks=True)
    w = w_cpu.to(dev)
    kc, vc = runner.logical_cache_view(w, w.key_cache), runner.logical_cache_view(w, w.value_cache)
    query = w.query.clone()
    out = torch.zeros_like(query)
    partitions = w_cpu.max_num_partitions  # (read from the host copy: nothing may synchronise under capture)

    def call(o, q):
        return paged_attention_reduce.run_static_scratch(
            o, q, kc, vc, w.block_tables, w.context_lens, w.num_heads // w.num_kv_heads, w.scale, w.block_size,
            int(w.block_tables.shape[1]) * w.block_size, partitions, w.sinks, partition_size=w.partition_size)

    _cabi.init()
    call(out, query)  # the eager call of this shape
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(out, query)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(out, query)
    gen = torch.Generator(device=dev).manual_seed(3)
    for replay in range(4):
        query.copy_(torch.randn(query.shape, generator=gen, device=dev).to(query.dtype))  # the graph reads this tensor
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        eager = torch.zeros_like(out)
        call(eager, query)                                       # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {replay} differs from the eager call"
    w_cpu.query = query.cpu()
    _, ref32 = call_oracle(oracle.attention_ref, w_cpu, want_f32=True)
    torch.testing.assert_close(out.float().cpu(), ref32, atol=1e-2, rtol=1e-2)


def test_static_scratch_refuses_what_does_not_fit():
    """A call that needs more than FA_STATIC_SCRATCH_BYTES: FA_ERR_SCRATCH_TOO_SMALL on the GPU as without
    one, nothing launched, `out` untouched -- and the next call that fits works."""
    dev = torch.device("cuda:0")
    w = W.make_test_shaped(batch_size=4, nheads=64, nheads_k=8, d=128, seqlen_k=600, varlen=False, has_sinks=False).to(dev)
    kc, vc = runner.logical_cache_view(w, w.key_cache), runner.logical_cache_view(w, w.value_cache)
    out = torch.full_like(w.query, 7.0)
    args = (out, w.query, kc, vc, w.block_tables, w.context_lens, 8, w.scale, w.block_size, 640)
    too_many = _cabi.FA_STATIC_SCRATCH_BYTES // (4 * 64 * 130 * 4) + 1   # slots x (head_size + 2) floats
    with pytest.raises(_cabi.PagedAttentionError, match="static scratch holds") as e:
        paged_attention_reduce.run_static_scratch(*args, too_many, None, partition_size=512)
    assert e.value.code == _cabi.FA_ERR_SCRATCH_TOO_SMALL
    torch.cuda.synchronize()
    assert (out == 7.0).all()
    paged_attention_reduce.run_static_scratch(*args, 2, None, partition_size=512)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all() and not (out == 7.0).all()
