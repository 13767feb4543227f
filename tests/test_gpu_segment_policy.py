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
    dev = torch.device("cuda:0")
    checked = 0
    for case in mk.batches(seed=7, per_shape=6):
        m, plan = mk.device_choice(case, dev)
        if m is None:
            continue
        assert mk.replay(case, plan) == m, (case, plan, m)
        checked += 1
    assert checked >= 25


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
