"""Committed fixtures (tests/golden/paged_attention_small.npz, written by
tests/golden/make_fixtures.py with this repository's own oracle; upstream has none).

CPU: the generators still produce the same input bits and the oracle still gives the
same answers.  GPU: the HIP kernels match the frozen answers."""
import importlib.util
import os

import numpy as np
import pytest
import torch

from _torch_ref import assert_close_to_reference

HERE = os.path.dirname(os.path.abspath(__file__))
spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(HERE, "golden", "make_fixtures.py"))
mk = importlib.util.module_from_spec(spec)
spec.loader.exec_module(mk)


@pytest.fixture(scope="module")
def golden():
    return np.load(os.path.join(HERE, "golden", "paged_attention_small.npz"), allow_pickle=False)


@pytest.mark.parametrize("name", list(mk.CASES))
def test_oracle_reproduces_fixtures(oracle, golden, name):
    w = mk.build(name)
    for key, t in (("query", w.query), ("key_cache", w.key_cache), ("value_cache", w.value_cache),
                   ("sinks", w.sinks)):
        assert np.array_equal(mk.bits(t), golden[f"{name}/{key}"]), key
    assert np.array_equal(w.block_tables.numpy(), golden[f"{name}/block_tables"])
    assert np.array_equal(w.context_lens.numpy(), golden[f"{name}/context_lens"])
    common = dict(scale=w.scale, block_size=w.block_size, kv_strides=w.kv_strides(),
                  num_kv_heads=w.num_kv_heads, sinks=w.sinks, fp8_scale=w.fp8_scale)
    args = (w.query, w.key_cache, w.value_cache, w.block_tables, w.context_lens)
    _, ref32 = oracle.attention_ref(*args, want_f32=True, **common)
    np.testing.assert_allclose(ref32.numpy(), golden[f"{name}/out_f32"], rtol=2e-6, atol=1e-7)
    es, ml, tmp = oracle.kernel_partition(*args, partition_size=w.partition_size,
                                          max_num_partitions=w.max_num_partitions, **common)
    for got, key in ((es, "exp_sums"), (ml, "max_logits"), (tmp, "tmp_out")):
        np.testing.assert_allclose(got.numpy(), golden[f"{name}/{key}"], rtol=2e-6, atol=1e-7, equal_nan=True)


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(mk.CASES))
def test_kernels_match_fixtures(golden, name):
    from flash_attention_factory_amd import runner
    w = mk.build(name).to(torch.device("cuda:0"))
    want = torch.from_numpy(golden[f"{name}/out_f32"])
    for kernel in (("fp8_loop", "fp8_reduce") if w.is_fp8 else ("loop", "reduce")):
        bufs = runner.alloc_buffers(w)
        runner.run_workload(w, kernel, bufs)
        torch.cuda.synchronize()
        assert_close_to_reference(bufs.out, want, f"{name}/{kernel}")
        if "reduce" in kernel:
            # rows this short run as the single-pass kernel unless the call fixes the partials: one
            # per partition, as the fixtures hold them
            bufs = runner.alloc_buffers(w)
            runner.run_workload(w, kernel, bufs, segment_partitions=1)
            torch.cuda.synchronize()
            assert_close_to_reference(bufs.out, want, f"{name}/{kernel}/one partial per partition")
            live = ~np.isnan(golden[f"{name}/exp_sums"])
            np.testing.assert_allclose(bufs.max_logits.cpu().numpy()[live], golden[f"{name}/max_logits"][live],
                                       rtol=1e-5, atol=1e-4)
            np.testing.assert_allclose(bufs.exp_sums.cpu().numpy()[live], golden[f"{name}/exp_sums"][live],
                                       rtol=1e-4, atol=1e-4)
            # a row of a single partial has it in `out` (as the row's result), not in tmp_out
            several = live & (live.sum(axis=2, keepdims=True) >= 2)
            np.testing.assert_allclose(bufs.tmp_out.cpu().numpy()[several], golden[f"{name}/tmp_out"][several],
                                       rtol=1e-2, atol=1e-2)
            assert np.isnan(bufs.exp_sums.cpu().numpy()[~live]).all()
