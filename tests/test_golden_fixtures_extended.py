"""Committed fixtures of what goes beyond upstream's kernels (tests/golden/paged_attention_extended.npz,
written by tests/golden/make_fixtures_extended.py with this repository's own oracle).

CPU: the generators still produce the same input bits and the oracle still gives the same
answers.  GPU: the HIP kernels match the frozen answers; the writer's pools bit for bit."""
import importlib.util
import os

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
spec = importlib.util.spec_from_file_location("make_fixtures_extended",
                                              os.path.join(HERE, "golden", "make_fixtures_extended.py"))
mk = importlib.util.module_from_spec(spec)
spec.loader.exec_module(mk)


@pytest.fixture(scope="module")
def golden():
    return np.load(os.path.join(HERE, "golden", "paged_attention_extended.npz"), allow_pickle=False)


@pytest.mark.parametrize("name", list(mk.CASES))
def test_oracle_reproduces_fixtures(oracle, golden, name):
    w, query, okw = mk.build(name)
    for key, t in (("query", query), ("key_cache", w.key_cache), ("value_cache", w.value_cache), ("sinks", w.sinks)):
        assert np.array_equal(mk.bits(t), golden[f"{name}/{key}"]), key
    assert np.array_equal(w.block_tables.numpy(), golden[f"{name}/block_tables"])
    assert np.array_equal(w.context_lens.numpy(), golden[f"{name}/context_lens"])
    for k in ("alibi_slopes", "k_scales", "v_scales"):
        if k in okw:
            assert np.array_equal(okw[k].numpy(), golden[f"{name}/{k}"]), k
    np.testing.assert_allclose(mk.reference(w, query, okw).numpy(), golden[f"{name}/out_f32"], rtol=2e-6, atol=1e-7)


def test_writer_oracle_reproduces_fixture(oracle, golden):
    key, value, slots, ks, vs, shape = mk.writer_case()
    assert np.array_equal(mk.bits(key), golden["writer/key"]) and np.array_equal(slots.numpy(), golden["writer/slots"])
    kc, vc = mk.written_pools(key, value, slots, ks, vs, shape)
    assert np.array_equal(kc.numpy(), golden["writer/key_cache"])
    assert np.array_equal(vc.numpy(), golden["writer/value_cache"])


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(mk.CASES))
def test_kernels_match_fixtures(golden, name):
    from flash_attention_factory_amd import lib
    dev = torch.device("cuda:0")
    w, query, okw = mk.build(name)
    want = torch.from_numpy(golden[f"{name}/out_f32"])
    unit = want.abs().max()
    wd = w.to(dev)
    q = query.to(dev)
    rows = q.shape[0] * (q.shape[1] if q.dim() == 4 else 1)
    H, D = q.shape[-2], q.shape[-1]
    NP = -(-int(w.context_lens.max()) // 64)
    alibi = okw["alibi_slopes"].to(dev) if "alibi_slopes" in okw else None
    kw = dict(apply_alibi=alibi is not None, apply_softcap="softcap" in okw, window_left=okw.get("window_left"))
    if "k_scales" in okw:
        kw.update(k_scales=okw["k_scales"].to(dev), v_scales=okw["v_scales"].to(dev))
    kv, vv = (wd.key_cache.permute(0, 2, 1, 3), wd.value_cache.permute(0, 2, 1, 3)) if w.layout == "head_major" \
        else (wd.key_cache, wd.value_cache)
    for kernel in (("fp8_loop", "fp8_reduce") if w.is_fp8 else ("loop", "reduce")):
        ml = torch.full((rows, H, NP), float("nan"), dtype=torch.float32, device=dev)
        es, tmp = torch.full_like(ml, float("nan")), torch.full((rows, H, NP, D), float("nan"), dtype=torch.float32, device=dev)
        out = torch.zeros_like(q)
        head = [ml, es, tmp, out, None, q, kv, vv, wd.block_tables, wd.context_lens, H // w.num_kv_heads, w.scale]
        if w.is_fp8:
            head.append(w.fp8_scale)
        extra = dict(partition_size=64) if "reduce" in kernel else {}
        getattr(lib, "paged_attention_" + kernel).run(*head, w.block_size, int(w.context_lens.max()), alibi, wd.sinks,
                                                      okw.get("softcap", 0.0), **extra, **kw)
        torch.cuda.synchronize()
        torch.testing.assert_close(out.float().cpu() / unit, want / unit, atol=1e-2, rtol=1e-2,
                                   msg=lambda m: f"{name} {kernel}: {m}")


@pytest.mark.gpu
def test_writer_matches_fixture(golden):
    from flash_attention_factory_amd.lib import kv_cache_write
    dev = torch.device("cuda:0")
    key, value, slots, ks, vs, shape = mk.writer_case()
    kc = torch.full(shape, 9, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    vc = torch.full(shape, 9, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    kv_cache_write.run(key.to(dev), value.to(dev), kc, vc, slots.to(dev), k_scales=ks.to(dev), v_scales=vs.to(dev))
    torch.cuda.synchronize()
    assert np.array_equal(kc.view(torch.uint8).cpu().numpy(), golden["writer/key_cache"])
    assert np.array_equal(vc.view(torch.uint8).cpu().numpy(), golden["writer/value_cache"])
