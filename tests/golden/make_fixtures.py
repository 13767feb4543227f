#!/usr/bin/env python3
"""Writes tests/golden/paged_attention_small.npz: small paged-attention cases with the
outputs of this repository's CPU oracle.

The upstream repository holds no golden vectors for this path (its tests only compare two
computations on an Intel GPU), so the fixtures pin this build's own oracle instead: the
oracle itself is pinned against library routines and closed forms in
tests/test_oracle_*.py; these files freeze its answers so that a later change to the
oracle, the generators or the kernels shows up as a diff against committed data.

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from flash_attention_factory_amd import workloads as W  # noqa: E402
from oracle import oracle as O  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "paged_attention_small.npz")

CASES = {
    # name: (builder kwargs, partition size for the split-path expectations)
    "f16_d64_b16_g1": (dict(batch_size=3, nheads=2, nheads_k=2, d=64, seqlen_k=40, varlen=False,
                            has_sinks=False, block_size=16, layout=W.HEAD_MAJOR, seed=1), 64, [1, 17, 40]),
    "f16_d128_b64_g4_sink": (dict(batch_size=2, nheads=8, nheads_k=2, d=128, seqlen_k=150, varlen=True,
                                  has_sinks=True, seed=2), 64, None),
    "bf16_fp8_d128_g8": (dict(batch_size=2, nheads=8, nheads_k=1, d=128, seqlen_k=100, varlen=True,
                              has_sinks=False, fp8=True, dtype=torch.bfloat16, block_size=16,
                              layout=W.HEAD_MAJOR, seed=3), 64, None),
    "f16_fp8_d64_g3_sink": (dict(batch_size=2, nheads=6, nheads_k=2, d=64, seqlen_k=90, varlen=True,
                                 has_sinks=True, fp8=True, seed=4), 64, None),
}


def bits(t):
    if t is None:
        return np.zeros(0, dtype=np.uint16)
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.contiguous().view(torch.int16).numpy().view(np.uint16)
    if t.dtype == torch.float8_e5m2:
        return t.contiguous().view(torch.uint8).numpy()
    return t.contiguous().numpy()


def build(name):
    kw, psize, lens = CASES[name]
    w = W.make_test_shaped(**kw)
    if lens is not None:
        w.context_lens = torch.tensor(lens, dtype=torch.int32)
    w.partition_size = psize
    return w


def main():
    out = {}
    for name in CASES:
        w = build(name)
        common = dict(scale=w.scale, block_size=w.block_size, kv_strides=w.kv_strides(),
                      num_kv_heads=w.num_kv_heads, sinks=w.sinks, fp8_scale=w.fp8_scale)
        args = (w.query, w.key_cache, w.value_cache, w.block_tables, w.context_lens)
        ref16, ref32 = O.attention_ref(*args, want_f32=True, **common)
        NP = w.max_num_partitions
        es, ml, tmp = O.kernel_partition(*args, partition_size=w.partition_size, max_num_partitions=NP, **common)
        out[f"{name}/query"] = bits(w.query)
        out[f"{name}/key_cache"] = bits(w.key_cache)
        out[f"{name}/value_cache"] = bits(w.value_cache)
        out[f"{name}/block_tables"] = w.block_tables.numpy()
        out[f"{name}/context_lens"] = w.context_lens.numpy()
        out[f"{name}/sinks"] = bits(w.sinks)
        out[f"{name}/out_f32"] = ref32.numpy()
        out[f"{name}/out_bits"] = bits(ref16)
        out[f"{name}/exp_sums"] = es.numpy()
        out[f"{name}/max_logits"] = ml.numpy()
        out[f"{name}/tmp_out"] = tmp.numpy()
    np.savez_compressed(OUT, **out)
    print(f"wrote {OUT}: {os.path.getsize(OUT) / 1024:.1f} KiB, {len(out)} arrays")


if __name__ == "__main__":
    main()
