"""GPU parity of the opt-in score modifiers (soft-capping, local window, ALiBi) with the oracle,
through all four entry points; and the default stays upstream's: slopes and cap are ignored."""
import pytest
import torch

from flash_attention_factory_amd import lib, runner, workloads as W
from _torch_ref import call_oracle

pytestmark = pytest.mark.gpu
ATOL = RTOL = 1e-2

CASES = [
    dict(window_left=100),
    dict(window_left=0),
    dict(window_left=700),
    dict(alibi=True),
    dict(softcap=5.0),
    dict(softcap=0.7, alibi=True, window_left=64),
    dict(softcap=30.0, alibi=True, window_left=1300),
]


def _dev():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch.device("cuda:0")


def _call(w, kernel, **mods):
    """One call of lib.<kernel>.run with upstream's positional arguments plus the opt-in keywords."""
    mod = getattr(lib, "paged_attention_" + kernel)
    bufs = runner.alloc_buffers(w)
    H, Hk = w.query.shape[1], w.num_kv_heads
    kv, vv = (w.key_cache.permute(0, 2, 1, 3), w.value_cache.permute(0, 2, 1, 3)) if w.layout == W.HEAD_MAJOR \
        else (w.key_cache, w.value_cache)
    head = [bufs.max_logits, bufs.exp_sums, bufs.tmp_out, bufs.out, None, w.query, kv, vv, w.block_tables,
            w.context_lens, H // Hk, w.scale]
    if kernel.startswith("fp8"):
        head.append(w.fp8_scale)
    alibi, softcap = mods.pop("alibi_slopes", None), mods.pop("softcap", 0.0)
    extra = dict(partition_size=w.partition_size) if "reduce" in kernel else {}
    mod.run(*head, w.block_size, int(w.context_lens.max()), alibi, w.sinks, softcap, **extra, **mods)
    torch.cuda.synchronize()
    return bufs.out


@pytest.mark.parametrize("mk", CASES, ids=lambda m: "_".join(f"{k}{v}" for k, v in m.items()))
@pytest.mark.parametrize("fp8", [False, True])
def test_modifiers_match_oracle(oracle, mk, fp8):
    w = W.make_test_shaped(batch_size=4, nheads=8, nheads_k=2, d=128, seqlen_k=1500, varlen=True, has_sinks=True,
                           fp8=fp8, seed=5)
    w.context_lens[0] = 1
    w.context_lens[1] = 513          # one token into the second partition
    H = w.query.shape[1]
    alibi = torch.rand(H, generator=torch.Generator().manual_seed(2)) * 0.05 if mk.get("alibi") else None
    okw = dict(alibi_slopes=alibi, softcap=mk.get("softcap", 0.0), window_left=mk.get("window_left", -1))
    ref = call_oracle(oracle.attention_ref, w, want_f32=True, **okw)[1]
    wd = w.to(_dev())
    mods = dict(alibi_slopes=None if alibi is None else alibi.to(_dev()), softcap=okw["softcap"],
                apply_alibi=alibi is not None, apply_softcap=okw["softcap"] > 0,
                window_left=mk.get("window_left"))
    for kernel in (("fp8_loop", "fp8_reduce") if fp8 else ("loop", "reduce")):
        got = _call(wd, kernel, **dict(mods)).float().cpu()
        assert torch.isfinite(got).all()
        torch.testing.assert_close(got, ref, atol=ATOL, rtol=RTOL, msg=lambda m: f"{kernel} {mk}: {m}")


def test_modifiers_on_a_measured_shape(oracle):
    """bf16 queries, E5M2 pools, G = 8, block 16, head-major, window across many partitions."""
    w = W.make_config(4, num_seqs=3, pool_blocks=1200, lens=[5000, 64, 2049])
    H = w.query.shape[1]
    alibi = torch.linspace(0.001, 0.02, H)
    ref = call_oracle(oracle.attention_ref, w, want_f32=True, alibi_slopes=alibi, softcap=20.0, window_left=1500)[1]
    wd = w.to(_dev())
    for kernel in ("fp8_loop", "fp8_reduce"):
        got = _call(wd, kernel, alibi_slopes=alibi.to(_dev()), softcap=20.0, apply_alibi=True, apply_softcap=True,
                    window_left=1500).float().cpu()
        torch.testing.assert_close(got, ref, atol=ATOL, rtol=RTOL)


def test_default_ignores_slopes_and_cap(oracle):
    """Upstream's tests hand the kernels alibi_slopes = ones and expect plain attention
    (test_paged.py:456,480): without the opt-in keywords that is what comes out."""
    w = W.make_test_shaped(batch_size=2, nheads=8, nheads_k=2, d=64, seqlen_k=400, varlen=True, has_sinks=False)
    ref = call_oracle(oracle.attention_ref, w, want_f32=True)[1]
    wd = w.to(_dev())
    ones = torch.ones(8, dtype=torch.float32, device=_dev())
    for kernel in ("loop", "reduce"):
        got = _call(wd, kernel, alibi_slopes=ones, softcap=3.0).float().cpu()
        torch.testing.assert_close(got, ref, atol=ATOL, rtol=RTOL)
