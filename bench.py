#!/usr/bin/env python3
"""Throughput of the paged-attention decode path on one MI355X.

A "step" is one call of the hot path (`lib.paged_attention_loop.run`) over the
Llama-2-7B-shaped decode batch (configuration 1: 32 sequences, 32 heads, head size
128, block size 16, context lengths uniform in [512, 2048], fp16).  KV pools are
resident in HBM before timing starts; three pool clones are rotated so that no call
finds its blocks in the 256 MB Infinity Cache (the upstream perf loop rotates 50
clones for the same reason, test_paged.py:488-496).

value        algorithmic bytes per step / wall time per step over K asynchronous steps
roofline     the dominant kernel against the HBM peak.  Loop path: one kernel per step, so its
             average duration is the time between two HIP events around the K steps, on the launch
             stream, over K (for a batch so small that the host cannot launch as fast as the kernel
             runs: the kernel's own pair of events).  Split path: the attention kernel between a pair of events of its own
             (blocking calls, the library's elapsed_us path; the pair's cost counts in);
             "hbm_frac" there is the whole call -- both kernels and the gap -- by the region's events
cpu_baseline the CPU oracle (C + OpenMP restatement of the upstream tests' PyTorch
             reference) on the same workload on this box's host cores; under "torch_reference"
             that reference itself, restated in PyTorch (oracle/torch_reference.py), on a bounded
             sample of every configuration: one sequence and kv head at a time, and for
             configurations 0, 1 and 3 also in its literal padded form
configs      the other four configurations, each timed the same way, each with a roofline block
             of its own; the split configurations also say how many partitions one partial
             covers, how many scratch bytes were really written, and carry a "strict_partitions"
             leg: upstream's decomposition, one partial per 512-token partition
lds_staging  the FP8 configurations in the grid form, K/V through registers against K/V staged
             through LDS by direct-to-LDS loads
single_head_groups  the two configurations with one query head per kv head (1 and 3) by lane dot
             products and fp32 multiply-adds in the VALU (schedules FA_SCHEDULE_GRID_VALU, FA_SCHEDULE_VALU)
             against the matrix cores (15 of 16 MFMA columns idle): the grid form of both, and the
             resident form beside the configurations' own figures above
reference_perf_recipe  the shape upstream's own perf loop runs (test_paged.py:607-631 and the FP8
             twin: 64 sequences of 1500 tokens, 64 or 40 query heads over 8 kv heads, head size 64,
             block size 64, sinks, its token-major pools) through the loop and the split kernels,
             with upstream's bandwidth figure (bytes of the whole pool, test_paged.py:524-526)
             beside the algorithmic one
score_modifiers  configuration 1 with soft-capping, ALiBi and a local window switched on
query_tokens  configuration 1 with four query tokens per sequence (speculative-decoding step);
             query_tokens_two_tiles: with 32, which fill two tiles of MFMA columns;
             query_tokens_split_two_tiles: the same in the split path (configurations 2 and 4
             with 8 and 4 tokens)
token_major_layout  configurations 1-4 with pools laid out as the reference's tests build them
kv_block_scales  the FP8 loop configuration with E4M3 pools and per-block K and V scales
stream_ordered  host cost of a small decode step: blocking `run` calls (upstream's behaviour),
             the asynchronous torch.library operators, and a HIP-graph replay of them
kv_cache_write  the step before the path (scatter of new K/V rows into the pools with E5M2
             rounding): kernel time by the same events, read + written bytes against the
             HBM peak, and its CPU oracle on a bounded sample; random slots, and under
             kv_cache_write_prefill the slots a prefill writes (consecutive per sequence)
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0

# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script
# (summaries under profiles/); None where not yet measured.
# 512-sequence variants of the configurations (--large-batches): blocks per pool
LARGE_BATCH_POOL_BLOCKS = {1: 49152, 3: 49152, 4: 220000}

def kernel_sources_digest():
    """sha256 over the kernel sources (csrc/*.h, csrc/*.hip, names and contents in sorted order): what
    ties a counter measurement to the code it was made on."""
    import hashlib
    h = hashlib.sha256()
    folder = os.path.join(ROOT, "flash_attention_factory_amd", "csrc")
    for name in sorted(os.listdir(folder)):
        if name.endswith((".h", ".hip")):
            h.update(name.encode())
            h.update(open(os.path.join(folder, name), "rb").read())
    return h.hexdigest()[:16]


def _measured_traffic():
    """HBM bytes per launch of each configuration's dominant kernel, from the rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE runs summarised in profiles/hbm_traffic.txt (lines: name fetch_MB
    write_MB).  The file names the digest of the kernel sources it was measured on ("# csrc:"); if
    the sources have changed since, nothing is reported (None), and None for a configuration the
    file does not list."""
    table = {}
    path = os.path.join(ROOT, "profiles", "hbm_traffic.txt")
    if os.path.exists(path):
        measured_on = None
        for line in open(path):
            parts = line.split()
            if line.startswith("# csrc:") and len(parts) >= 3:
                measured_on = parts[2]
            elif len(parts) >= 3 and not line.startswith("#"):
                table[parts[0]] = (float(parts[1]) + float(parts[2])) * 1e6
        if measured_on != kernel_sources_digest():
            return {}
    return table


KERNEL_NAMES = {
    0: "paged_attn_loop_persistent_kernel<64, F16, kv16, 4 waves>",
    1: "paged_attn_loop_persistent_kernel<128, F16, kv16, 4 waves>",
    2: "paged_attn_segment_kernel<128, F16, kv16, 4 waves>",
    3: "paged_attn_loop_persistent_kernel<128, F16, e5m2, 4 waves>",
    4: "paged_attn_segment_kernel<128, BF16, e5m2, 4 waves>",
}


def _clones(w, torch):
    pool_bytes = w.key_cache.numel() * w.key_cache.element_size()
    n = max(2, min(8, math.ceil((1 << 30) / pool_bytes) + 1))
    ks = [w.key_cache] + [w.key_cache.clone() for _ in range(n - 1)]
    vs = [w.value_cache] + [w.value_cache.clone() for _ in range(n - 1)]
    return ks, vs


def _build_config(index, torch, W, runner, dev, **kw):
    w = W.make_config(index, device=dev, pools_on_device=True, **kw)
    ks, vs = _clones(w, torch)
    return w, ks, vs


# The legs beside the headline warm up for at least this long, whatever --warmup says: after the
# host-side pause between two legs the first 10 to 15 ms of launches run 3 % slower than the rest
# (268 us against 278 us per call on the serving mix), and these legs are short.
SIDE_LEG_WARM_MS = 30.0


def _time_config(built, steps, warmup, torch, W, runner, dev, schedule=0, traffic_key=None, min_warm_ms=SIDE_LEG_WARM_MS):
    w, ks, vs = built
    kernel = W.CONFIG_KERNEL[w.meta["config"]] if "config" in w.meta else w.meta["kernel"]
    bufs = runner.alloc_buffers(w)
    n = len(ks)
    warmed = 0
    t_warm = time.perf_counter()
    while warmed < warmup or ((time.perf_counter() - t_warm) * 1e3 < min_warm_ms and warmed < warmup + 1000):
        runner.run_workload(w, kernel, bufs, key_cache=ks[warmed % n], value_cache=vs[warmed % n], timed=False, schedule=schedule)
        warmed += 1
        if warmed >= warmup and warmed % 8 == 0:
            torch.cuda.synchronize()  # so that the host's clock sees the GPU's time
    torch.cuda.synchronize()
    # the timed region: K asynchronous calls, between two HIP events on the stream the kernels are
    # launched on (torch's current one) and the host's clock
    first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    first.record()
    for it in range(steps):
        runner.run_workload(w, kernel, bufs, key_cache=ks[it % n], value_cache=vs[it % n], timed=False, schedule=schedule)
    last.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    region_us = first.elapsed_time(last) * 1e3 / steps
    # every kernel by itself: blocking calls, a pair of HIP events around each launch (the
    # library's elapsed_us path).  The pair costs one to three microseconds that it counts in.
    ev = []
    for it in range(steps):
        ev.append(runner.run_workload(w, kernel, bufs, key_cache=ks[it % n], value_cache=vs[it % n], schedule=schedule))
    ev_t = torch.tensor(ev, dtype=torch.float64)
    res = dict(
        workload=w.name, kernel=kernel, steps=steps, warmup_steps=warmed,
        ms_per_step=wall / steps * 1e3,
        algorithmic_bytes=w.algorithmic_bytes(),
        kernel_us_mean=[float(x) for x in ev_t.mean(0)],
        kernel_us_median=[float(x) for x in ev_t.median(0).values],
        # time of the call's kernels: both figures bound it from above (the region's by the launch
        # gaps and, for batches of a few microseconds, the host's launch rate; the blocking calls'
        # by their event pairs), so the smaller one
        us_per_call=min(region_us, float(ev_t.sum(1).mean())),
        us_per_call_region=region_us,
        us_per_call_blocking=float(ev_t.sum(1).mean()),
        pool_clones=n,
    )
    res["gbps_wall"] = res["algorithmic_bytes"] / (wall / steps) / 1e9
    res["gbps_kernels"] = res["algorithmic_bytes"] / (res["us_per_call"] * 1e-6) / 1e9
    res["hbm_frac"] = res["gbps_kernels"] / HBM_PEAK_GBPS
    # The dominant kernel alone.  Loop path: the only kernel of a call, so its average duration is
    # the region's events over the launches -- unless the host launches more slowly than the
    # kernel runs (a batch of a few microseconds), where the kernel's own pair of events is the
    # closer bound; both bound the duration from above.  Split path: the attention kernel by its
    # own pair of events (the reduce kernel is reported beside it).
    kernel_us = res["kernel_us_mean"][0]
    if len(res["kernel_us_mean"]) == 1:
        kernel_us = min(kernel_us, region_us)
    achieved = res["algorithmic_bytes"] / (kernel_us * 1e-6) / 1e9
    res["gbps_attention_kernel"] = achieved
    res["roofline"] = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                       "frac": achieved / HBM_PEAK_GBPS, "traffic": _measured_traffic().get(traffic_key),
                       "kernel": KERNEL_NAMES.get(w.meta.get("config")) if schedule == 0 else "paged_attn_kernel (grid form)",
                       "kernel_us": kernel_us}
    if "reduce" in kernel:
        # What the attention kernel really leaves in the scratch arrays: one call into NaN-filled
        # buffers, then count.  A partial is (head_size + 2) floats per query head.
        probe = runner.alloc_buffers(w)
        runner.run_workload(w, kernel, probe, timed=False, schedule=schedule)
        torch.cuda.synchronize()
        written = ~torch.isnan(probe.max_logits)
        S, H, D = w.query.shape
        longest = int(torch.argmax(w.context_lens))
        slots = torch.nonzero(written[longest, 0]).flatten().tolist()
        res["scratch_bytes_allocated"] = w.scratch_bytes()
        # a row's only partial goes into `out` as its result: two scalars in the scratch arrays, no row
        rows = ~torch.isnan(probe.tmp_out[..., 0])
        res["scratch_bytes_written"] = int(written.sum()) * 2 * 4 + int(rows.sum()) * D * 4
        res["partials"] = int(written.sum()) // H * w.num_kv_heads
        res["partials_stored_into_out"] = (int(written.sum()) - int(rows.sum())) // H * w.num_kv_heads
        res["partitions_per_segment"] = (slots[1] - slots[0]) if len(slots) > 1 else None
        res["partition_size"] = w.partition_size
    return w, res


def _cpu_baseline(index, torch, W, budget_s=10.0):
    from oracle import oracle as O
    w = W.make_config(index)  # CPU generator, seeded
    def call():
        return O.attention_ref(w.query, w.key_cache, w.value_cache, w.block_tables, w.context_lens,
                               scale=w.scale, block_size=w.block_size, kv_strides=w.kv_strides(),
                               num_kv_heads=w.num_kv_heads, sinks=w.sinks, fp8_scale=w.fp8_scale)
    call()  # warm-up
    reps, t0 = 0, time.perf_counter()
    while True:
        call()
        reps += 1
        dt = time.perf_counter() - t0
        if dt > budget_s or reps >= 200:
            break
    per = dt / reps
    return dict(value=w.algorithmic_bytes() / per / 1e9, unit="GB/s", cores=O.num_threads(), kind="port",
                ms_per_call=per * 1e3,
                sample=f"full {w.name} workload (seed 0), {reps} repetitions of the C/OpenMP oracle "
                       f"oracle_attention_ref, {dt:.1f} s")


# Bounded samples of the configurations for the PyTorch reference on the host cores: the same
# shapes and length distributions with fewer sequences (and pools just large enough for them),
# so that the whole leg stays within seconds.
_TORCH_SAMPLES = {0: dict(), 1: dict(), 2: dict(num_seqs=2, pool_blocks=4096), 3: dict(),
                  4: dict(num_seqs=16, pool_blocks=12288)}


def _torch_reference_baseline(torch, W, budget_s=2.5):
    """The upstream tests' PyTorch reference (oracle/torch_reference.py) timed on this box's host
    cores with torch's own threading: per configuration the per-sequence form, and for
    configurations 0, 1 and 3 also the literal padded form (dense K/V gathered and repeated over
    the query group, as test_paged.py builds them)."""
    from oracle import torch_reference as T
    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    out = []
    for index, kw in _TORCH_SAMPLES.items():
        w = W.make_config(index, **kw)
        forms = [("per_sequence", False)] + ([("padded", True)] if index in (0, 1, 3) else [])
        for form, padded in forms:
            T.run_workload(w, padded=padded)  # warm-up
            reps, t0 = 0, time.perf_counter()
            while True:
                T.run_workload(w, padded=padded)
                reps += 1
                dt = time.perf_counter() - t0
                if dt > budget_s or reps >= 50:
                    break
            per = dt / reps
            full = W._CONFIGS[index]["S"]
            out.append(dict(config=index, form=form, value=w.algorithmic_bytes() / per / 1e9, unit="GB/s",
                            ms_per_call=per * 1e3, cores=threads, torch_threads=torch.get_num_threads(), kind="port",
                            sample=f"{w.num_seqs} of the {full} sequences of {w.name} "
                                   f"({w.algorithmic_bytes() / 1e6:.1f} MB of K/V), {reps} repetitions, {dt:.1f} s"
                                   + (f", dense K/V of {T.padded_bytes(w) / 1e6:.0f} MB" if padded else "")))
    return out


def _reference_perf_recipe(steps, torch, W, runner, dev):
    """Upstream's own perf shape and loop (test_paged.py:607-631, 485-560; FP8 twin
    test_paged_fp8cache.py:612-636): batch 64, 64 (FP8: 40) query heads over 8 kv heads, 1500 keys,
    head size 64, block size 64, sinks, pools in upstream's token-major layout with every block
    referenced by exactly one sequence, several pool clones rotated, 5 warm-up calls, kernel-event
    time.  Upstream counts the bytes of the whole pool (:524-526); the algorithmic figure (keys
    inside the contexts only) is given beside it."""
    legs = []
    for fp8, heads in ((False, 64), (True, 40)):
        w = W.make_test_shaped(batch_size=64, nheads=heads, nheads_k=8, d=64, seqlen_k=1500, varlen=False,
                               has_sinks=True, fp8=fp8, device=dev)
        w.meta["kernel"] = "fp8_loop" if fp8 else "loop"
        pool_bytes = w.key_cache.numel() * w.key_cache.element_size() * 2
        ks, vs = _clones(w, torch)
        pre = "fp8_" if fp8 else ""
        # loop entry; split entry as upstream calls it; split entry made to run its two kernels (whole rows
        # as one segment each, and upstream's one partial per partition)
        for kernel, forced in ((pre + "loop", {}), (pre + "reduce", {}), (pre + "reduce", dict(segment_partitions=64)),
                               (pre + "reduce", dict(schedule=1))):
            bufs = runner.alloc_buffers(w)
            ts = []
            for it in range(5 + steps):
                # upstream passes seqlen_k as max_context_len (test_paged.py:478-480)
                t = runner.run_workload(w, kernel, bufs, key_cache=ks[it % len(ks)], value_cache=vs[it % len(ks)],
                                        max_context_len=1500, **forced)
                if it >= 5:
                    ts.append(sum(t))
            us = float(torch.tensor(ts, dtype=torch.float64).mean())
            form = None
            if "reduce" in kernel:  # which kernels the split entry ran
                form = "single-pass kernel" if t[1] == 0.0 else "split kernels"
                if forced:
                    form += " (forced: " + ", ".join(f"{k}={v}" for k, v in forced.items()) + ")"
            legs.append(dict(workload=f"upstream perf recipe: S64 H{heads} Hk8 D64 B64 ctx1500 sinks, token-major, "
                                      f"{'E5M2' if fp8 else 'fp16'} pools", kernel=kernel, steps=steps,
                             us_per_call=us, form=form, pool_clones=len(ks), whole_pool_bytes=pool_bytes,
                             gbps_whole_pool=pool_bytes / us / 1e3,
                             algorithmic_bytes=w.algorithmic_bytes(), gbps_kernels=w.algorithmic_bytes() / us / 1e3,
                             hbm_frac=w.algorithmic_bytes() / us / 1e3 / HBM_PEAK_GBPS))
        del ks, vs, w
    return legs


def _time_kv_cache_write(steps, torch, dev, cpu_leg, prefill_shaped=False):
    """Prefill-sized batch of the KV-cache writer: 32768 new tokens x 8 kv heads x 128, fp16
    rows into E5M2 head-major pools of 65536 16-token blocks.  Slots: random free ones (the worst
    case: every 128-byte row of a kv head lands somewhere else), or, prefill_shaped, what a prefill
    writes: 16 sequences of 2048 new tokens each, a sequence's tokens in consecutive slots of blocks
    that lie anywhere in the pool.  Six source/pool sets rotate (1.6 GB between two uses of the same
    bytes)."""
    from flash_attention_factory_amd.lib import kv_cache_write
    N, Hk, D, B, NB, R = 32768, 8, 128, 16, 65536, 6
    g = torch.Generator(device=dev).manual_seed(0)
    keys = [torch.randn(N, Hk, D, generator=g, device=dev, dtype=torch.float16) for _ in range(R)]
    vals = [torch.randn(N, Hk, D, generator=g, device=dev, dtype=torch.float16) for _ in range(R)]
    pools = [(torch.zeros((NB, Hk, B, D), dtype=torch.uint8, device=dev),
              torch.zeros((NB, Hk, B, D), dtype=torch.uint8, device=dev)) for _ in range(R)]
    if prefill_shaped:
        within = torch.arange(N, device=dev) % B
        slots = [torch.randperm(NB, generator=g, device=dev)[:N // B].repeat_interleave(B).to(torch.int64) * B + within
                 for _ in range(R)]
    else:
        slots = [torch.randperm(NB * B, generator=g, device=dev)[:N].to(torch.int64) for _ in range(R)]
    view = lambda t: t.permute(0, 2, 1, 3).view(torch.float8_e5m2)
    ts = []
    for it in range(5 + steps):
        k = it % R
        t = kv_cache_write.run(keys[k], vals[k], view(pools[k][0]), view(pools[k][1]), slots[k])
        if it >= 5:
            ts.append(t[0])
    us = float(torch.tensor(ts, dtype=torch.float64).mean())
    read_b, write_b = 2 * N * Hk * D * 2 + 8 * N, 2 * N * Hk * D
    res = dict(workload=f"kv_cache_write: {N} tokens x {Hk} kv heads x {D}, fp16 -> E5M2, head-major pool of "
                        f"{NB} blocks of {B}, " + ("consecutive slots per sequence (16 sequences of 2048 tokens, blocks "
                                                   "anywhere)" if prefill_shaped else "random slots"),
               kernel="kv_cache_write_kernel<F16, e5m2>", steps=steps, us_per_call=us,
               read_bytes=read_b, write_bytes=write_b, gbps_kernels=(read_b + write_b) / us / 1e3,
               hbm_frac=(read_b + write_b) / us / 1e3 / HBM_PEAK_GBPS)
    if cpu_leg:
        from oracle import oracle as O
        n = 2048
        kc = torch.zeros((n // B, Hk, B, D), dtype=torch.uint8)
        vc = torch.zeros_like(kc)
        kh, vh = keys[0][:n].cpu(), vals[0][:n].cpu()
        sl = torch.randperm(n, dtype=torch.int64)
        t0 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t0 < 3.0:
            O.kv_cache_write(kh, vh, kc, vc, sl, block_size=B, kv_strides=(Hk * B * D, D, B * D))
            reps += 1
        per = (time.perf_counter() - t0) / reps
        res["cpu_baseline"] = dict(value=(read_b + write_b) * (n / N) / per / 1e9, unit="GB/s", cores=1, kind="port",
                                   sample=f"{n} of the {N} tokens, {reps} repetitions of oracle_kv_cache_write")
    return res


def _time_score_modifiers(built, steps, torch, W, runner, dev):
    """Configuration 1 with the opt-in score modifiers: soft-capping 30, ALiBi, and a local window
    of 1024 keys (the window shortens what has to be read; bytes are counted for visible keys)."""
    from flash_attention_factory_amd.lib import paged_attention_loop
    w, ks, vs = built
    S, H, D = w.query.shape
    Hk, B = w.num_kv_heads, w.block_size
    window_left = 1023
    alibi = torch.linspace(0.002, 0.05, H, device=dev, dtype=torch.float32)
    bufs = runner.alloc_buffers(w)
    view = (lambda t: t.permute(0, 2, 1, 3)) if w.layout == W.HEAD_MAJOR else (lambda t: t)
    ts = []
    for it in range(5 + steps):
        k = it % len(ks)
        t = paged_attention_loop.run(None, None, None, bufs.out, None, w.query, view(ks[k]), view(vs[k]),
                                     w.block_tables, w.context_lens, H // Hk, w.scale, B, 0, alibi, w.sinks, 30.0,
                                     apply_alibi=True, apply_softcap=True, window_left=window_left)
        if it >= 5:
            ts.append(t[0])
    us = float(torch.tensor(ts, dtype=torch.float64).mean())
    visible = torch.clamp(w.context_lens, max=window_left + 1).sum().item()
    nbytes = visible * Hk * D * 2 * w.key_cache.element_size() + 2 * S * H * D * 2 + 4 * S + 4 * H \
        + sum(-(-min(int(c), window_left + 1) // B) for c in w.context_lens.tolist()) * 4
    return dict(workload="config1 + soft-capping 30 + ALiBi + local window of 1024 keys",
                kernel="paged_attn_loop_persistent_kernel<128, F16, kv16, extended>", steps=steps, us_per_call=us,
                algorithmic_bytes=nbytes, gbps_kernels=nbytes / us / 1e3, hbm_frac=nbytes / us / 1e3 / HBM_PEAK_GBPS)


def _time_query_tokens(built, steps, torch, W, runner, dev, query_len=4):
    """Configuration 1 with several query tokens per sequence (a speculative-decoding
    verification step): the K/V bytes are read once for all of them."""
    from flash_attention_factory_amd.lib import paged_attention_loop
    w, ks, vs = built
    S, H, D = w.query.shape
    Hk, B = w.num_kv_heads, w.block_size
    query4 = torch.randn((S, query_len, H, D), device=dev).to(w.query.dtype)
    out4 = torch.zeros_like(query4)
    view = (lambda t: t.permute(0, 2, 1, 3)) if w.layout == W.HEAD_MAJOR else (lambda t: t)
    ts = []
    for it in range(5 + steps):
        k = it % len(ks)
        t = paged_attention_loop.run(None, None, None, out4, None, query4, view(ks[k]), view(vs[k]), w.block_tables,
                                     w.context_lens, H // Hk, w.scale, B, 0, None, w.sinks, 0.0)
        if it >= 5:
            ts.append(t[0])
    us = float(torch.tensor(ts, dtype=torch.float64).mean())
    nbytes = w.algorithmic_bytes() + 2 * S * (query_len - 1) * H * D * 2
    two_tiles = query_len * (H // Hk) > 16  # more (query token, head) pairs than one tile of MFMA columns holds
    res = dict(workload=f"config1 with {query_len} query tokens per sequence, causal",
               kernel="paged_attn_loop_two_tile_kernel<128, F16, kv16>" if two_tiles
               else "paged_attn_loop_persistent_kernel<128, F16, kv16, extended>", steps=steps, us_per_call=us,
               algorithmic_bytes=nbytes, gbps_kernels=nbytes / us / 1e3, hbm_frac=nbytes / us / 1e3 / HBM_PEAK_GBPS)
    if two_tiles:  # K and V are meant to cross HBM once for both tiles: say what the counters saw
        res["traffic"] = _measured_traffic().get("query_tokens_two_tiles")
    return res


def _time_query_tokens_split(built, steps, torch, W, runner, dev, query_len):
    """A split-path configuration with several query tokens per sequence, enough to fill two tiles
    of MFMA columns (query_len x group > 16): both tiles are held by every wavefront, K and V are
    read once."""
    from flash_attention_factory_amd import lib
    w, ks, vs = built
    S, H, D = w.query.shape
    Hk, B = w.num_kv_heads, w.block_size
    mod = lib.paged_attention_fp8_reduce if w.is_fp8 else lib.paged_attention_reduce
    query4 = torch.randn((S, query_len, H, D), device=dev).to(w.query.dtype)
    out4 = torch.zeros_like(query4)
    NP = max(1, math.ceil(int(w.context_lens.max()) / w.partition_size))
    ml = torch.zeros((S * query_len, H, NP), dtype=torch.float32, device=dev)
    es = torch.zeros_like(ml)
    tmp = torch.zeros((S * query_len, H, NP, D), dtype=torch.float32, device=dev)
    view = (lambda t: t.permute(0, 2, 1, 3)) if w.layout == W.HEAD_MAJOR else (lambda t: t)
    ts = []
    for it in range(5 + steps):
        k = it % len(ks)
        head = [ml, es, tmp, out4, None, query4, view(ks[k]), view(vs[k]), w.block_tables, w.context_lens, H // Hk, w.scale]
        if w.is_fp8:
            head.append(1.0)
        t = mod.run(*head, B, 0, None, w.sinks, 0.0, partition_size=w.partition_size)
        if it >= 5:
            ts.append(t)
    mean = torch.tensor(ts, dtype=torch.float64).mean(0)
    us = float(mean.sum())
    nbytes = w.algorithmic_bytes() + 2 * S * (query_len - 1) * H * D * 2
    return dict(workload=f"{w.name} with {query_len} query tokens per sequence, causal",
                kernel="paged_attn_loop_two_tile_kernel<split path> + paged_attn_reduce_kernel",
                steps=steps, kernel_us_mean=[float(x) for x in mean], us_per_call=us, algorithmic_bytes=nbytes,
                gbps_kernels=nbytes / us / 1e3, hbm_frac=nbytes / us / 1e3 / HBM_PEAK_GBPS)


def _time_block_scales(built, steps, torch, W, runner, dev):
    """The FP8 loop configuration with E4M3 pools and one K and one V scale per physical block
    and kv head (two more fp32 per 16-token tile of 4 KiB)."""
    from flash_attention_factory_amd.lib import paged_attention_fp8_loop
    w, ks, vs = built
    S, H, D = w.query.shape
    Hk, B = w.num_kv_heads, w.block_size
    NB = w.key_cache.shape[0]
    k_scales = torch.rand((NB, Hk), device=dev) * 0.02 + 0.005
    v_scales = torch.rand((NB, Hk), device=dev) * 0.02 + 0.005
    bufs = runner.alloc_buffers(w)
    view = (lambda t: t.permute(0, 2, 1, 3)) if w.layout == W.HEAD_MAJOR else (lambda t: t)
    ts = []
    for it in range(5 + steps):
        k = it % len(ks)
        t = paged_attention_fp8_loop.run(None, None, None, bufs.out, None, w.query, view(ks[k]), view(vs[k]),
                                         w.block_tables, w.context_lens, H // Hk, w.scale, 1.0, B, 0, None, w.sinks,
                                         0.0, k_scales=k_scales, v_scales=v_scales)
        if it >= 5:
            ts.append(t[0])
    us = float(torch.tensor(ts, dtype=torch.float64).mean())
    blocks = sum(-(-int(c) // B) for c in w.context_lens.tolist())
    nbytes = w.algorithmic_bytes() + blocks * Hk * 2 * 4
    return dict(workload="config3 (E4M3 pools) with per-block K and V scales",
                kernel="paged_attn_loop_persistent_kernel<128, F16, e4m3, extended>", steps=steps, us_per_call=us,
                algorithmic_bytes=nbytes, gbps_kernels=nbytes / us / 1e3, hbm_frac=nbytes / us / 1e3 / HBM_PEAK_GBPS)


def _time_stream_ordered(steps, torch, W, runner, dev):
    """Host cost of one small decode step (configuration 0: KV-cache append of one token per
    sequence, then the loop kernel) three ways: the timed `run` calls, which block on every
    kernel as upstream's launchers do; the torch.library operators, asynchronous on the
    current stream; and the same two operators replayed from a HIP graph."""
    from flash_attention_factory_amd import torch_ops  # noqa: F401
    from flash_attention_factory_amd.lib import kv_cache_write, paged_attention_loop
    ops = torch.ops.fa_amd
    w = W.make_config(0, device=dev, pools_on_device=True)
    S, H, D = w.query.shape
    Hk, B = w.num_kv_heads, w.block_size
    kv, vv = (w.key_cache.permute(0, 2, 1, 3), w.value_cache.permute(0, 2, 1, 3)) if w.layout == W.HEAD_MAJOR \
        else (w.key_cache, w.value_cache)
    bufs = runner.alloc_buffers(w)
    key = torch.randn((S, Hk, D), device=dev).to(w.query.dtype)
    value = torch.randn((S, Hk, D), device=dev).to(w.query.dtype)
    last = (w.context_lens - 1).long()
    slots = w.block_tables.gather(1, (last // B)[:, None]).squeeze(1).long() * B + last % B

    def blocking():
        kv_cache_write.run(key, value, kv, vv, slots)
        paged_attention_loop.run(None, None, None, bufs.out, None, w.query, kv, vv, w.block_tables, w.context_lens,
                                 H // Hk, w.scale, B, 0, None, w.sinks, 0.0)

    def asynchronous():
        ops.kv_cache_write(key, value, kv, vv, slots, 1.0)
        ops.paged_attention_loop(bufs.out, w.query, kv, vv, w.block_tables, w.context_lens, w.scale, w.sinks)

    def wall(fn, n):
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n * 1e6

    res = dict(workload="config0 decode step: kv_cache_write of 1 token per sequence + loop kernel (S4 H8 D64)",
               us_per_step_blocking=wall(blocking, steps), us_per_step_async_ops=wall(asynchronous, steps))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        asynchronous()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        asynchronous()
    res["us_per_step_graph_replay"] = wall(graph.replay, steps)
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--configs", type=str, default="0,2,3,4",
                    help="other configurations to time besides configuration 1 ('' for none)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kv-cache-write", action="store_true")
    ap.add_argument("--no-token-major", action="store_true",
                    help="skip the token-major legs (they run the same kernels as configurations 1 and 3, "
                         "which blurs a per-kernel profile)")
    ap.add_argument("--layout", choices=["head_major", "token_major"], default="head_major",
                    help="pool layout of the main configurations (token_major = the reference's own "
                         "[blocks, block_size, kv_heads, head_size]); for profiling one layout alone")
    ap.add_argument("--no-extras", action="store_true",
                    help="time the configurations only: no modifier, query-token, E4M3, scale or stream-ordered legs")
    ap.add_argument("--large-batches", action="store_true",
                    help="also time configurations 4, 3 and 1 with 512 sequences (up to 26 GB of pools), "
                         "each in a process of its own")
    ap.add_argument("--large-batch-only", type=int, default=-1, help=argparse.SUPPRESS)
    ap.add_argument("--calibrate-counters", action="store_true",
                    help="run nothing but three plain device-to-device copies of 1 GiB (read 1 GiB, write 1 GiB "
                         "each): under rocprofv3 --pmc FETCH_SIZE or WRITE_SIZE their readings give the scale of "
                         "the counter")
    ap.add_argument("--sources-digest", action="store_true", help="print the digest of the kernel sources and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this path has no multi-GPU form in this build "
              f"(--gpus {args.gpus} refused)", file=sys.stderr)
        return 2

    if args.sources_digest:
        print(kernel_sources_digest())
        return 0
    import torch
    from flash_attention_factory_amd import _cabi, runner, workloads as W
    if args.calibrate_counters:
        src = torch.full((1 << 30,), 0x5a, dtype=torch.uint8, device="cuda:0")
        dst = torch.zeros_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "3 device-to-device copies", "read_bytes_each": 1 << 30, "written_bytes_each": 1 << 30}))
        return 0
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    _cabi.load()  # raises if the HIP library was not built: there is no fallback
    dev = torch.device("cuda:0")
    if args.large_batch_only >= 0:
        # a batch beyond what one persistent launch lists: sub-batches (split path, 16-bit loop
        # path) or the grid form (FP8 loop path)
        idx = args.large_batch_only
        big = _build_config(idx, torch, W, runner, dev, num_seqs=512, pool_blocks=LARGE_BATCH_POOL_BLOCKS[idx])
        _, r = _time_config(big, 20, 3, torch, W, runner, dev)
        r["workload"] += "_512_sequences"
        # what the library runs for such a batch (launch_kernels_loop.h, launch_kernels_reduce.h)
        r["roofline"]["kernel"] = {1: "paged_attn_valu_kernel<kv16, 8 waves> (grid form, lane dot products)",
                                   3: "paged_attn_kernel<128, F16, e5m2, 8 waves> (grid form)",
                                   4: "paged_attn_segment_kernel<128, BF16, e5m2, 4 waves>, two sub-batches"}[idx]
        print(json.dumps(r), flush=True)
        return 0

    # All pools are allocated before anything is timed, largest first: memory handed out
    # after other pools were freed is fragmented into small pages, and the randomly
    # addressed KV blocks then pay TLB misses that have nothing to do with the kernels.
    indices = [1] + [int(x) for x in args.configs.split(",") if x.strip() != ""]
    order = sorted(set(indices), key=lambda i: -W._CONFIGS[i]["NB"] * W._CONFIGS[i]["Hk"])
    built = {i: _build_config(i, torch, W, runner, dev, layout=args.layout) for i in order}
    torch.cuda.synchronize()

    # the headline: exactly --warmup untimed steps, then exactly --steps timed ones
    _, main_res = _time_config(built[1], args.steps, args.warmup, torch, W, runner, dev, min_warm_ms=0.0,
                               traffic_key="config1" + ("" if args.layout == "head_major" else "_token_major"))
    others = []
    sub_steps = max(20, args.steps // 2)
    suffix = "" if args.layout == "head_major" else "_token_major"
    for idx in indices[1:]:
        _, r = _time_config(built[idx], sub_steps, args.warmup, torch, W, runner, dev, traffic_key=f"config{idx}{suffix}")
        if "reduce" in r["kernel"] and not args.no_extras:
            # upstream's own decomposition: one work-group and one partial per 512-token partition
            _, strict = _time_config(built[idx], sub_steps, args.warmup, torch, W, runner, dev, schedule=1)
            r["strict_partitions"] = {k: strict[k] for k in ("kernel_us_mean", "us_per_call", "gbps_kernels", "hbm_frac",
                                                            "scratch_bytes_written", "partials", "partitions_per_segment")}
        others.append(r)
    line = {
        "metric": "achieved HBM GB/s, fp16 paged decode (loop kernel)",
        "value": main_res["gbps_wall"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": main_res["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp16",
        "data": "synthetic",
        "config": {"workload": "config1: fp16 loop kernel, S32 H32 Hk32 D128 B16 ctx U[512,2048], "
                               "4096-block head-major pool, shuffled block tables",
                   "layout": args.layout,
                   "us_per_call": main_res["us_per_call"],
                   "algorithmic_bytes": main_res["algorithmic_bytes"],
                   "hbm_frac_of_8TBps": main_res["hbm_frac"]},
        "roofline": main_res.pop("roofline"),
        "configs": others,
    }
    if not args.no_extras:
        line["score_modifiers"] = _time_score_modifiers(built[1], max(20, args.steps // 2), torch, W, runner, dev)
        line["query_tokens"] = _time_query_tokens(built[1], max(20, args.steps // 2), torch, W, runner, dev)
        # 32 tokens of one head are two column tiles, both held by every wavefront
        line["query_tokens_two_tiles"] = _time_query_tokens(built[1], max(20, args.steps // 2), torch, W, runner, dev,
                                                            query_len=32)
        # the split path with two tiles: 8 tokens x 4 heads of config 2, 4 tokens x 8 heads of config 4
        line["query_tokens_split_two_tiles"] = [
            _time_query_tokens_split(built[idx], sub_steps, torch, W, runner, dev, ql)
            for idx, ql in ((2, 8), (4, 4)) if idx in built]
        # the FP8 loop configuration once more with E4M3 bytes in the pools (same shape, same bytes moved)
        e4m3 = _build_config(3, torch, W, runner, dev, fp8_dtype=torch.float8_e4m3fn)
        _, r = _time_config(e4m3, max(20, args.steps // 2), args.warmup, torch, W, runner, dev)
        r["workload"] += "_e4m3"
        others.append(r)
        line["kv_block_scales"] = _time_block_scales(e4m3, max(20, args.steps // 2), torch, W, runner, dev)
        del e4m3
        # configurations 1 and 3 once more with pools in the reference's own layout
        # [blocks, block_size, kv_heads, head_size]: a token's row of one kv head is then the only
        # contiguous piece (256 or 128 bytes), successive tokens lie kv_heads rows apart
        line["token_major_layout"] = []
        for idx in (() if args.no_token_major else (4, 2, 1, 3)):
            tm = _build_config(idx, torch, W, runner, dev, layout=W.TOKEN_MAJOR)
            _, r = _time_config(tm, max(20, args.steps // 2), args.warmup, torch, W, runner, dev,
                                traffic_key=f"config{idx}_token_major")
            r["workload"] += "_token_major"
            line["token_major_layout"].append(r)
            del tm
        line["token_major_layout"].sort(key=lambda r: r["workload"])
        # the grid form of the FP8 configurations with K/V through registers (schedule 1) and staged
        # through LDS by direct-to-LDS loads (schedule 2), beside the persistent forms timed above
        line["lds_staging"] = []
        for idx in (3, 4):
            if idx not in built:
                continue
            for schedule, name in ((1, "grid form, K/V through registers"), (2, "grid form, K/V staged through LDS")):
                _, r = _time_config(built[idx], sub_steps, args.warmup, torch, W, runner, dev, schedule=schedule)
                line["lds_staging"].append(dict(workload=r["workload"], schedule=name, kernel_us_mean=r["kernel_us_mean"],
                                                us_per_call=r["us_per_call"], hbm_frac=r["hbm_frac"]))
        # query groups of one head: the grid form by the matrix cores (schedule 1) against the grid
        # form by dot products in the VALU (schedule 4), beside the persistent forms timed above
        line["single_head_groups"] = []
        for idx in (1, 3):
            if idx not in built:
                continue
            for schedule, name in ((1, "grid form, matrix cores"), (4, "grid form, VALU dot products"),
                                   (5, "resident work-groups, VALU dot products")):
                _, r = _time_config(built[idx], sub_steps, args.warmup, torch, W, runner, dev, schedule=schedule)
                line["single_head_groups"].append(dict(workload=r["workload"], schedule=name, kernel_us_mean=r["kernel_us_mean"],
                                                       us_per_call=r["us_per_call"], hbm_frac=r["hbm_frac"]))
        line["reference_perf_recipe"] = _reference_perf_recipe(max(20, args.steps // 2), torch, W, runner, dev)
        line["stream_ordered"] = _time_stream_ordered(max(200, args.steps), torch, W, runner, dev)
    if not args.no_kv_cache_write:
        del built
        torch.cuda.empty_cache()
        line["kv_cache_write"] = _time_kv_cache_write(max(20, args.steps // 2), torch, dev, not args.no_cpu_baseline)
        line["kv_cache_write_prefill"] = _time_kv_cache_write(max(20, args.steps // 2), torch, dev, False, prefill_shaped=True)
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = _cpu_baseline(1, torch, W)
        line["cpu_baseline"]["torch_reference"] = _torch_reference_baseline(torch, W)
    if args.large_batches:
        # Pools of tens of GB want an allocator nobody has fragmented (see above): one child
        # process per configuration, after this process has given its own pools back.
        import subprocess
        built = None
        torch.cuda.empty_cache()
        line["large_batches"] = []
        for idx in sorted(LARGE_BATCH_POOL_BLOCKS):
            child = subprocess.run([sys.executable, os.path.abspath(__file__), "--large-batch-only", str(idx)],
                                   capture_output=True, text=True)
            if child.returncode != 0:
                print(child.stderr, file=sys.stderr)
                return child.returncode
            line["large_batches"].append(json.loads(child.stdout.strip().splitlines()[-1]))
    # Every configuration's figures once more, compact and LAST in the line (and inside `config`), so
    # that whoever keeps only the head or the tail of it keeps them: microseconds per call, the dominant
    # kernel's duration and fraction of the HBM peak, measured traffic.
    summary = [_summary_of("config1: " + args.layout, main_res["us_per_call"], line["roofline"])]
    for r in others:
        summary.append(_summary_of(r["workload"], r["us_per_call"], r["roofline"], r.get("kernel_us_mean")))
    for key in ("kv_cache_write", "kv_cache_write_prefill"):
        if key in line:
            summary.append(dict(w=key, us=round(line[key]["us_per_call"], 2), frac=round(line[key]["hbm_frac"], 4)))
    for r in line.get("reference_perf_recipe", []):
        if r.get("form") is None or "forced" not in r["form"]:
            summary.append(dict(w=("recipe_e5m2_" if "E5M2" in r["workload"] else "recipe_fp16_") + r["kernel"],
                                us=round(r["us_per_call"], 2), frac=round(r["hbm_frac"], 4), form=r.get("form")))
    line["config"]["configs_summary"] = summary
    line["configs_summary"] = summary
    print(json.dumps(line), flush=True)
    return 0


def _summary_of(name, us_per_call, roofline, kernel_us_mean=None):
    out = dict(w=name, us=round(us_per_call, 2), kernel_us=round(roofline["kernel_us"], 2),
               GBps=round(roofline["achieved"], 1), frac=round(roofline["frac"], 4),
               traffic_MB=None if roofline["traffic"] is None else round(roofline["traffic"] / 1e6, 2))
    if kernel_us_mean and len(kernel_us_mean) > 1:
        out["reduce_us"] = round(kernel_us_mean[1], 2)
    return out


if __name__ == "__main__":
    sys.exit(main())
