"""GPU parity of the KV-cache writer (lib.kv_cache_write.run -> fa_kv_cache_write) with its
CPU oracle: bit-exact, as the work is byte and integer placement plus one rounding."""
import pytest
import torch

from flash_attention_factory_amd import workloads as W
from flash_attention_factory_amd.lib import kv_cache_write

pytestmark = pytest.mark.gpu


def _dev():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch.device("cuda:0")


def _all_16bit(dtype):
    return torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype)


def _pool(layout, NB, B, Hk, D, dtype, fill=9):
    shape = (NB, B, Hk, D) if layout == W.TOKEN_MAJOR else (NB, Hk, B, D)
    if dtype == torch.float8_e5m2:
        return torch.full(shape, fill, dtype=torch.uint8)
    return torch.full(shape, float(fill), dtype=dtype)


def _view(pool, layout):
    return pool if layout == W.TOKEN_MAJOR else pool.permute(0, 2, 1, 3)


def _bits(t):
    return t if t.dtype == torch.uint8 else t.view(torch.int16)


def _both(oracle, key, value, kc, vc, slots, layout, B, scale=1.0):
    """Run the oracle on CPU copies and the kernel on device copies; return both pool pairs."""
    dev = _dev()
    kc_d, vc_d = kc.to(dev), vc.to(dev)
    v = _view(kc, layout)
    oracle.kv_cache_write(key, value, kc, vc, slots, block_size=B,
                          kv_strides=(v.stride(0), v.stride(1), v.stride(2)), fp8_scale=scale)
    kv = _view(kc_d, layout), _view(vc_d, layout)
    kv = tuple(t.view(torch.float8_e5m2) if t.dtype == torch.uint8 else t for t in kv)
    us = kv_cache_write.run(key.to(dev), value.to(dev), kv[0], kv[1], slots.to(dev), scale)
    torch.cuda.synchronize()
    assert len(us) == 1 and us[0] > 0
    return (kc, vc), (kc_d.cpu(), vc_d.cpu())


@pytest.mark.parametrize("src", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("scale", [1.0, 0.5, 3.0])
def test_every_16bit_pattern(oracle, src, scale):
    x = _all_16bit(src).view(512, 1, 128)
    kc, vc = _pool(W.TOKEN_MAJOR, 512, 1, 1, 128, torch.float8_e5m2), _pool(W.TOKEN_MAJOR, 512, 1, 1, 128, torch.float8_e5m2)
    slots = torch.arange(512, dtype=torch.int64)
    (wk, wv), (gk, gv) = _both(oracle, x, x.flip(0).contiguous(), kc, vc, slots, W.TOKEN_MAJOR, 1, scale)
    assert torch.equal(gk, wk) and torch.equal(gv, wv)
    if scale == 1.0:  # and the oracle's bytes are torch's
        assert torch.equal(wk.view(-1), x.to(torch.float8_e5m2).view(torch.uint8).view(-1))


@pytest.mark.parametrize("src", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("scale", [1.0, 0.5, 3.0])
def test_every_16bit_pattern_e4m3(oracle, src, scale):
    dev = _dev()
    x = _all_16bit(src).view(512, 1, 128)
    y = x.flip(0).contiguous()
    slots = torch.arange(512, dtype=torch.int64)
    wk, wv = torch.zeros((512, 1, 1, 128), dtype=torch.uint8), torch.zeros((512, 1, 1, 128), dtype=torch.uint8)
    oracle.kv_cache_write(x, y, wk, wv, slots, block_size=1, kv_strides=(128, 128, 128), fp8_scale=scale, e4m3=True)
    gk = torch.zeros((512, 1, 1, 128), dtype=torch.float8_e4m3fn, device=dev)
    gv = torch.zeros_like(gk)
    kv_cache_write.run(x.to(dev), y.to(dev), gk, gv, slots.to(dev), scale)
    torch.cuda.synchronize()
    assert torch.equal(gk.view(torch.uint8).cpu(), wk) and torch.equal(gv.view(torch.uint8).cpu(), wv)
    if scale == 1.0:  # and the oracle's bytes are torch's
        assert torch.equal(wk.view(-1), x.to(torch.float8_e4m3fn).view(torch.uint8).view(-1))


@pytest.mark.parametrize("layout", [W.TOKEN_MAJOR, W.HEAD_MAJOR])
@pytest.mark.parametrize("src", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("D", [64, 128])
def test_scatter_matches_oracle(oracle, layout, src, fp8, D):
    g = torch.Generator().manual_seed(11)
    N, Hk, B, NB = 333, 5, 16, 40
    key = (torch.randn(N, Hk, D, generator=g) * 8).to(src)
    value = (torch.randn(N, Hk, D, generator=g) * 8).to(src)
    slots = torch.randperm(NB * B, generator=g)[:N].to(torch.int64)
    slots[::17] = -1
    slots[3] = NB * B
    slots[4] = 1 << 40
    cdt = torch.float8_e5m2 if fp8 else src
    (wk, wv), (gk, gv) = _both(oracle, key, value, _pool(layout, NB, B, Hk, D, cdt), _pool(layout, NB, B, Hk, D, cdt),
                               slots, layout, B)
    assert torch.equal(_bits(gk), _bits(wk)) and torch.equal(_bits(gv), _bits(wv))
    assert (_bits(gk) == _bits(_pool(layout, NB, B, Hk, D, cdt))).any()  # skipped slots kept their fill


def test_strided_source_and_empty_batch(oracle):
    g = torch.Generator().manual_seed(5)
    N, Hk, D, B, NB = 50, 2, 128, 16, 8
    fused = (torch.randn(N, 3, Hk, D, generator=g)).to(torch.float16)   # a [q, k, v] projection output
    key, value = fused[:, 1], fused[:, 2]
    slots = torch.randperm(NB * B, generator=g)[:N].to(torch.int64)
    (wk, wv), (gk, gv) = _both(oracle, key, value, _pool(W.HEAD_MAJOR, NB, B, Hk, D, torch.float8_e5m2),
                               _pool(W.HEAD_MAJOR, NB, B, Hk, D, torch.float8_e5m2), slots, W.HEAD_MAJOR, B)
    assert torch.equal(gk, wk) and torch.equal(gv, wv)
    dev = _dev()
    pool = torch.zeros((2, 16, 2, 128), dtype=torch.float16, device=dev)
    empty = torch.zeros((0, 2, 128), dtype=torch.float16, device=dev)
    assert kv_cache_write.run(empty, empty, pool, pool.clone(), torch.zeros(0, dtype=torch.int64, device=dev)) == [0.0]


def test_written_pool_feeds_the_decode_kernels(oracle):
    """Prefill through the writer, decode through the FP8 kernels: the same answer as the
    decode kernels give on a pool quantised by the tensor cast upstream's tests use."""
    from flash_attention_factory_amd import runner
    dev = _dev()
    w = W.make_config(3, num_seqs=4, pool_blocks=600, lens=[100, 2048, 777, 1])   # FP8 pools, fp16 queries
    B, Hk, D = w.block_size, w.num_kv_heads, w.query.shape[2]
    g = torch.Generator().manual_seed(2)
    toks = int(w.context_lens.sum())
    key = torch.randn(toks, Hk, D, generator=g).to(torch.float16)
    value = torch.randn(toks, Hk, D, generator=g).to(torch.float16)
    slots, n = torch.empty(toks, dtype=torch.int64), 0
    for s, L in enumerate(w.context_lens.tolist()):
        t = torch.arange(L)
        slots[n:n + L] = w.block_tables[s, t // B].long() * B + t % B
        n += L
    # reference pools: tensor cast + indexing, as upstream's tests build them
    view_k = w.key_cache.view(torch.uint8).permute(0, 2, 1, 3) if w.layout == W.HEAD_MAJOR else w.key_cache.view(torch.uint8)
    view_v = w.value_cache.view(torch.uint8).permute(0, 2, 1, 3) if w.layout == W.HEAD_MAJOR else w.value_cache.view(torch.uint8)
    view_k[slots // B, slots % B] = key.to(torch.float8_e5m2).view(torch.uint8)
    view_v[slots // B, slots % B] = value.to(torch.float8_e5m2).view(torch.uint8)
    wd = w.to(dev)
    kc = torch.zeros_like(wd.key_cache.view(torch.uint8))
    vc = torch.zeros_like(kc)
    kv = (kc if w.layout == W.TOKEN_MAJOR else kc.permute(0, 2, 1, 3)).view(torch.float8_e5m2)
    vv = (vc if w.layout == W.TOKEN_MAJOR else vc.permute(0, 2, 1, 3)).view(torch.float8_e5m2)
    kv_cache_write.run(key.to(dev), value.to(dev), kv, vv, slots.to(dev))
    written = kc.cpu() != 0
    assert torch.equal(kc.cpu()[written], w.key_cache.view(torch.uint8)[written])
    bufs_ref = runner.alloc_buffers(wd)
    runner.run_workload(wd, "fp8_loop", bufs_ref)
    bufs = runner.alloc_buffers(wd)
    runner.run_workload(wd, "fp8_loop", bufs, key_cache=kc.view(wd.key_cache.dtype), value_cache=vc.view(wd.value_cache.dtype))
    torch.cuda.synchronize()
    assert torch.equal(bufs.out, bufs_ref.out)


def test_prefill_sized_batch_against_torch_cast():
    """32768 tokens x 8 kv heads x 128: every written row equals torch's own cast of its
    source row (a second, independent implementation), and nothing else was touched."""
    dev = _dev()
    N, Hk, D, B = 32768, 8, 128, 16
    NB = N // B + 64
    g = torch.Generator(device=dev).manual_seed(0)
    key = torch.randn(N, Hk, D, generator=g, device=dev, dtype=torch.float16) * 3
    value = torch.randn(N, Hk, D, generator=g, device=dev, dtype=torch.float16) * 3
    slots = torch.randperm(NB * B, generator=g, device=dev)[:N].to(torch.int64)
    kc = torch.full((NB, Hk, B, D), 7, dtype=torch.uint8, device=dev)
    vc = torch.full((NB, Hk, B, D), 7, dtype=torch.uint8, device=dev)
    kv_cache_write.run(key, value, kc.permute(0, 2, 1, 3).view(torch.float8_e5m2),
                       vc.permute(0, 2, 1, 3).view(torch.float8_e5m2), slots)
    torch.cuda.synchronize()
    got_k = kc.permute(0, 2, 1, 3)[slots // B, slots % B]
    got_v = vc.permute(0, 2, 1, 3)[slots // B, slots % B]
    assert torch.equal(got_k, key.to(torch.float8_e5m2).view(torch.uint8))
    assert torch.equal(got_v, value.to(torch.float8_e5m2).view(torch.uint8))
    untouched = torch.ones(NB * B, dtype=torch.bool, device=dev)
    untouched[slots] = False
    assert (kc.permute(0, 2, 1, 3).reshape(NB * B, Hk, D)[untouched] == 7).all()
