#!/usr/bin/env python3
"""Writes tests/golden/paged_attention_extended.npz: small cases of what goes beyond upstream's
kernels -- score modifiers, several query tokens per sequence, E4M3 pools, per-head and per-block
FP8 scales, and the KV-cache writer with scales -- with the outputs of this repository's CPU
oracle.  Upstream holds no vectors for any of it (its kernels do not implement it); the oracle
functions involved are pinned against library routines in tests/test_oracle_masks.py,
tests/test_oracle_kv_scales.py and tests/test_oracle_kv_cache.py, and these files freeze their
answers.

Run from the repository root:  python tests/golden/make_fixtures_extended.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from flash_attention_factory_amd import workloads as W  # noqa: E402
from oracle import oracle as O  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "paged_attention_extended.npz")

# name: (make_test_shaped kwargs, query tokens per sequence, modifiers, scale mode)
CASES = {
    "f16_window_alibi_cap": (dict(batch_size=2, nheads=4, nheads_k=2, d=64, seqlen_k=120, varlen=True, has_sinks=True,
                                  block_size=16, seed=51), 1, dict(window_left=50, alibi=True, softcap=8.0), None),
    "f16_three_query_tokens": (dict(batch_size=2, nheads=4, nheads_k=2, d=64, seqlen_k=70, varlen=True, has_sinks=False,
                                    block_size=16, layout=W.HEAD_MAJOR, seed=52), 3, dict(), None),
    "bf16_e4m3_block_scales": (dict(batch_size=2, nheads=8, nheads_k=2, d=128, seqlen_k=90, varlen=True, has_sinks=True,
                                    fp8=True, dtype=torch.bfloat16, block_size=16, fp8_dtype=torch.float8_e4m3fn,
                                    seed=53), 1, dict(), "block"),
    "f16_e5m2_head_scales_two_tokens_window": (dict(batch_size=2, nheads=4, nheads_k=2, d=64, seqlen_k=100, varlen=True,
                                                    has_sinks=False, fp8=True, block_size=16, seed=54), 2,
                                               dict(window_left=40), "head"),
}


def bits(t):
    if t is None:
        return np.zeros(0, dtype=np.uint16)
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.contiguous().view(torch.int16).numpy().view(np.uint16)
    if t.dtype in (torch.float8_e5m2, torch.float8_e4m3fn):
        return t.contiguous().view(torch.uint8).numpy()
    return t.contiguous().numpy()


def build(name):
    """(workload, query [S, QL, H, D] or [S, H, D], oracle keywords) of a case; seeded."""
    kw, ql, mods, scale_mode = CASES[name]
    w = W.make_test_shaped(**kw)
    g = torch.Generator().manual_seed(kw["seed"] + 1000)
    H, Hk = w.num_heads, w.num_kv_heads
    query = w.query if ql == 1 else torch.randn(w.num_seqs, ql, H, w.head_size, generator=g).to(w.query.dtype)
    okw = {}
    if mods.get("alibi"):
        okw["alibi_slopes"] = (torch.rand(H, generator=g) * 0.1 + 0.01).float()
    if "softcap" in mods:
        okw["softcap"] = mods["softcap"]
    if "window_left" in mods:
        okw["window_left"] = mods["window_left"]
    if scale_mode is not None:
        shape = (w.key_cache.shape[0], Hk) if scale_mode == "block" else (Hk,)
        okw["k_scales"] = (torch.rand(shape, generator=g) * 1.5 + 0.25).float()
        okw["v_scales"] = (torch.rand(shape, generator=g) * 1.5 + 0.25).float()
    return w, query, okw


def reference(w, query, okw):
    return O.attention_ref(query, w.key_cache, w.value_cache, w.block_tables, w.context_lens, scale=w.scale,
                           block_size=w.block_size, kv_strides=w.kv_strides(), num_kv_heads=w.num_kv_heads,
                           sinks=w.sinks, fp8_scale=w.fp8_scale, want_f32=True, **okw)[1]


def writer_case():
    """Inputs of a KV-cache write with per-block E4M3 scales, and the pools the oracle produces."""
    g = torch.Generator().manual_seed(77)
    N, Hk, D, B, NB = 23, 2, 64, 16, 3
    key = (torch.randn(N, Hk, D, generator=g) * 3).to(torch.float16)
    value = (torch.randn(N, Hk, D, generator=g) * 3).to(torch.float16)
    slots = torch.randperm(NB * B, generator=g)[:N].to(torch.int64)
    slots[4] = -1
    ks = (torch.rand(NB, Hk, generator=g) * 0.05 + 0.005).float()
    vs = (torch.rand(NB, Hk, generator=g) * 0.05 + 0.005).float()
    return key, value, slots, ks, vs, (NB, B, Hk, D)


def written_pools(key, value, slots, ks, vs, shape):
    NB, B, Hk, D = shape
    kc = torch.full(shape, 9, dtype=torch.uint8)
    vc = torch.full(shape, 9, dtype=torch.uint8)
    O.kv_cache_write(key, value, kc, vc, slots, block_size=B, kv_strides=(B * Hk * D, Hk * D, D), e4m3=True,
                     k_scales=ks, v_scales=vs)
    return kc, vc


def main():
    out = {}
    for name in CASES:
        w, query, okw = build(name)
        out[f"{name}/query"] = bits(query)
        out[f"{name}/key_cache"] = bits(w.key_cache)
        out[f"{name}/value_cache"] = bits(w.value_cache)
        out[f"{name}/block_tables"] = w.block_tables.numpy()
        out[f"{name}/context_lens"] = w.context_lens.numpy()
        out[f"{name}/sinks"] = bits(w.sinks)
        for k in ("alibi_slopes", "k_scales", "v_scales"):
            if k in okw:
                out[f"{name}/{k}"] = okw[k].numpy()
        out[f"{name}/out_f32"] = reference(w, query, okw).numpy()
    key, value, slots, ks, vs, shape = writer_case()
    kc, vc = written_pools(key, value, slots, ks, vs, shape)
    out["writer/key"], out["writer/value"], out["writer/slots"] = bits(key), bits(value), slots.numpy()
    out["writer/k_scales"], out["writer/v_scales"] = ks.numpy(), vs.numpy()
    out["writer/key_cache"], out["writer/value_cache"] = kc.numpy(), vc.numpy()
    np.savez_compressed(OUT, **out)
    print(f"wrote {OUT}: {os.path.getsize(OUT) / 1024:.1f} KiB, {len(out)} arrays")


if __name__ == "__main__":
    main()
