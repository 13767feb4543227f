"""On the GPU: the segment length the attention kernels choose equals the host restatement of the rule
(tests/_segment_policy.py) on batches the recorded fixture does not hold; a call of the split path
whose rows are provably short runs as the single-pass kernel and gives the bits that kernel gives;
and a fixed segment length (options->segment_partitions) changes the partials, not the result."""
import importlib.util
import os

import pytest
import torch

from flash_attention_factory_amd import _cabi, runner, workloads as W
from _torch_ref import call_oracle

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
spec = importlib.util.spec_from_file_location("make_segment_policy_cases",
                                              os.path.join(HERE, "golden", "make_segment_policy_cases.py"))
mk = importlib.util.module_from_spec(spec)
spec.loader.exec_module(mk)


def test_device_choice_equals_the_host_restatement():
    """The segment length the attention kernels choose and the slots in which they leave partials,
    against the host restatement, on batches the fixture does not hold; and the same batches cut into
    even shares on request."""
    dev = torch.device("cuda:0")
    checked = 0
    for case in mk.batches(seed=7, per_shape=6):
        m, plan, slots = mk.device_choice(case, dev)
        if plan["form"] != _cabi.FA_SPLIT_FORM_SEGMENT:
            continue
        want = mk.replay(case, plan)
        if m is not None:  # some piece covers two partitions, so the marks tell the cut
            assert m == want, (case, plan, m, want)
        assert slots == mk.replay_slots(case, plan, want), (case, plan, want)
        m, plan, slots = mk.device_choice(case, dev, segment_partitions=-1)
        assert m in (0, None) and slots == mk.replay_slots(case, plan, 0), (case, plan)
        checked += 1
    assert checked >= 25, checked


def test_even_shares_on_request(oracle):
    """options->segment_partitions = -1 cuts any batch into even shares: the rows' partitions laid end
    to end, one contiguous run per work-group.  A small ragged batch (more work-groups than
    partitions: shares of one partition or none), against the oracle and the restated cuts."""
    dev = torch.device("cuda:0")
    case = dict(head_size=128, num_kv_heads=4, group=2, fp8=False, token_major=False, block_size=16, partition_size=512,
                lens=[5000, 0, 513, 1, 2100, 30000])
    m, plan, slots = mk.device_choice(case, dev, segment_partitions=-1)
    assert m in (0, None) and slots == mk.replay_slots(case, plan, 0)
    w_cpu = W.make_config(2, num_seqs=6, pool_blocks=4096, lens=case["lens"])
    _, ref32 = call_oracle(oracle.attention_ref, w_cpu, want_f32=True)
    w = w_cpu.to(dev)
    for kernel_kw in (dict(segment_partitions=-1), dict()):
        bufs = runner.alloc_buffers(w)
        runner.run_workload(w, "reduce", bufs, **kernel_kw)
        torch.cuda.synchronize()
        live = w_cpu.context_lens > 0
        torch.testing.assert_close(bufs.out.float().cpu()[live], ref32[live], atol=1e-2, rtol=1e-2)
        assert (bufs.out.cpu()[~live] == 0).all()


def test_even_shares_full_serving_mix(oracle):
    """A serving mix cut into even shares (128 sequences, log-normal lengths, E5M2 pools, bf16 queries,
    8 query heads per kv head, sinks): every output row against the oracle."""
    dev = torch.device("cuda:0")
    gen = torch.Generator().manual_seed(5)
    lens = torch.exp(torch.randn(128, generator=gen) * 0.75 + 8.3).long().clamp(64, 32768)
    lens[3] = 0
    w_cpu = W.make_config(4, num_seqs=128, pool_blocks=int(sum(-(-int(n) // 16) for n in lens)) + 8, lens=lens.tolist())
    w_cpu.sinks = torch.linspace(-1, 3, w_cpu.num_heads).to(w_cpu.query.dtype)
    w = w_cpu.to(dev)
    bufs = runner.alloc_buffers(w)
    runner.run_workload(w, "fp8_reduce", bufs, segment_partitions=-1)
    torch.cuda.synchronize()
    bits = bufs.max_logits.view(torch.int32).cpu()
    marks = bits[(bits & mk.MARK_MASK) == mk.MARK_BITS]
    assert marks.numel() and set((marks & 0xFF).tolist()) == {0}, "this batch is meant to be cut into even shares"
    _, ref32 = call_oracle(oracle.attention_ref, w_cpu, want_f32=True)
    live = w_cpu.context_lens > 0
    torch.testing.assert_close(bufs.out.float().cpu()[live], ref32[live], atol=1e-2, rtol=1e-2)
    assert (bufs.out.cpu()[~live] == 0).all()


@pytest.mark.parametrize("fp8", [False, True], ids=["fp16", "e5m2"])
def test_short_rows_run_as_the_single_pass_kernel(oracle, fp8):
    """Upstream's perf shape cut down in head count only (64 sequences of 1500 keys, 8 kv heads, head
    size 64, block 64, sinks, token-major pools): the split entry returns {t, 0}, leaves the scratch
    arrays alone and gives the loop entry's bits; the same call under schedule = grid, and with a
    fixed segment length, runs the split kernels and agrees within the tolerance."""
    dev = torch.device("cuda:0")
    w_cpu = W.make_test_shaped(batch_size=64, nheads=16, nheads_k=8, d=64, seqlen_k=1500, varlen=True, has_sinks=True, fp8=fp8)
    w = w_cpu.to(dev)
    pre = "fp8_" if fp8 else ""
    loop = runner.alloc_buffers(w)
    runner.run_workload(w, pre + "loop", loop)
    split = runner.alloc_buffers(w)
    times = runner.run_workload(w, pre + "reduce", split, max_context_len=1500)
    torch.cuda.synchronize()
    assert len(times) == 2 and times[0] > 0 and times[1] == 0.0
    assert torch.equal(split.out, loop.out)
    assert torch.isnan(split.max_logits).all() and torch.isnan(split.exp_sums).all() and torch.isnan(split.tmp_out).all()
    _, ref32 = call_oracle(oracle.attention_ref, w_cpu, want_f32=True)
    torch.testing.assert_close(split.out.float().cpu(), ref32, atol=1e-2, rtol=1e-2)
    for kw in (dict(schedule=1), dict(segment_partitions=2), dict(segment_partitions=64)):
        other = runner.alloc_buffers(w)
        times = runner.run_workload(w, pre + "reduce", other, max_context_len=1500, **kw)
        torch.cuda.synchronize()
        assert times[1] > 0 and not torch.isnan(other.max_logits[:, :, 0]).any()
        torch.testing.assert_close(other.out.float().cpu(), ref32, atol=1e-2, rtol=1e-2)


def test_fixed_segment_length(oracle):
    """options->segment_partitions = n: partials in slots 0, n, 2n, ... and the mark in slot 1."""
    dev = torch.device("cuda:0")
    w_cpu = W.make_config(2, num_seqs=3, pool_blocks=2048, lens=[5000, 2100, 700])
    w = w_cpu.to(dev)
    _, ref32 = call_oracle(oracle.attention_ref, w_cpu, want_f32=True)
    for n in (1, 2, 3, 7, 64):
        bufs = runner.alloc_buffers(w)
        runner.run_workload(w, "reduce", bufs, segment_partitions=n)
        torch.cuda.synchronize()
        torch.testing.assert_close(bufs.out.float().cpu(), ref32, atol=1e-2, rtol=1e-2)
        ml = bufs.max_logits.cpu()
        parts = [10, 5, 2]
        for s in range(3):
            slots = set(range(0, parts[s], n))
            written = {j for j in range(parts[s]) if not torch.isnan(ml[s, 0, j])}
            if n > 1:
                bits = int(ml[s, 0, 1].view(torch.int32)) & 0xFFFFFFFF
                assert bits == (mk.MARK_BITS | n), (n, s, hex(bits))
                written.discard(1)
            assert written == slots, (n, s, written)
