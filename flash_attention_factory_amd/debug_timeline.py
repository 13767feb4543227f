"""Where the time of a persistent launch goes: the in-kernel timeline of a debug build, as a table.

A library compiled with -DFA_TIMELINE has every wavefront of the persistent kernels (loop, segment)
leave wall-clock stamps of the 100 MHz counter in a device array (csrc/paged_attention_utils.h:
timeline_stamp) and exports fa_debug_timeline to fetch them.  The product library carries neither.

    python -m flash_attention_factory_amd._build --output flash_attention_factory_amd/libfa_timeline.so -DFA_TIMELINE
    FA_PAGED_ATTENTION_LIBRARY=flash_attention_factory_amd/libfa_timeline.so \
        python -m flash_attention_factory_amd.debug_timeline 3 1 4        # benchmark configurations, on the GPU

Per configuration it prints, in microseconds from the first wavefront's entry and as percentiles over
wavefronts (or work-groups, or compute units): kernel entry, context lengths in and items listed,
first K tile in registers, last chunk done, last merge stored; the chunks a compute unit was dealt
(the static imbalance of the deal) and when each unit's last work-group ended, by XCC.
"""
from __future__ import annotations

import argparse
import ctypes
import json

import numpy as np

WAVES, SLOTS = 8192, 8
QS = (0, 10, 50, 90, 100)


def _pct(x, qs=QS):
    x = np.asarray(x, dtype=np.float64)
    x = x[~np.isnan(x)]
    return [round(float(np.percentile(x, q)), 2) for q in qs] if x.size else [float("nan")] * len(qs)


def read_timeline(lib, clear: bool) -> np.ndarray:
    buf = np.zeros(WAVES * SLOTS, dtype=np.uint64)
    status = lib.fa_debug_timeline(buf.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(buf.nbytes), int(clear))
    if status != 0:
        raise RuntimeError(f"fa_debug_timeline failed with {status}")
    return buf.reshape(WAVES, SLOTS).astype(np.int64)


def timeline_of(idx: int, launches: int, warm: int, segment_partitions=None, schedule=0):
    import torch
    from . import _cabi, runner, workloads as W
    lib = _cabi.load()
    if not hasattr(lib, "fa_debug_timeline"):
        raise RuntimeError(f"{_cabi.LIBRARY} was not compiled with -DFA_TIMELINE")
    lib.fa_debug_timeline.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int32]
    dev = torch.device("cuda:0")
    w = W.make_config(idx, device=dev, pools_on_device=True)
    kernel = W.CONFIG_KERNEL[idx]
    # three copies of the pools in turn, so that no launch finds the previous one's lines in a cache
    pools = [(w.key_cache, w.value_cache)] + [(w.key_cache.clone(), w.value_cache.clone()) for _ in range(2)]
    bufs = runner.alloc_buffers(w)
    extra = {}
    if "reduce" in kernel:
        extra["schedule"] = schedule
        if segment_partitions is not None:
            extra["segment_partitions"] = segment_partitions
    launches_out = []
    for it in range(warm + launches):
        key, value = pools[it % 3]
        if it >= warm:
            read_timeline(lib, clear=True)
        event_us = runner.run_workload(w, kernel, bufs, key_cache=key, value_cache=value, **extra)
        if it < warm:
            continue
        t = read_timeline(lib, clear=False)
        t = t[t[:, 0] > 0]
        waves_per_group = 4
        # (a wavefront that found no work leaves the later slots at zero: not a time)
        us = lambda col: np.where(t[:, col] > 0, (t[:, col] - t[:, 0].min()) / 100.0, np.nan)
        ran = t[:, 5] > 0
        group_end = np.nan_to_num(us(4), nan=0.0).reshape(-1, waves_per_group).max(axis=1)
        group_chunks = t[:, 5].reshape(-1, waves_per_group).sum(axis=1)
        hw = t[:, 6].reshape(-1, waves_per_group)[:, 0]
        xcc = t[:, 7].reshape(-1, waves_per_group)[:, 0] & 0xF
        unit = xcc * 1024 + ((hw >> 13) & 0x7) * 16 + ((hw >> 8) & 0xF)  # (XCC, shader engine, CU)
        units = np.unique(unit)
        unit_end = np.array([group_end[unit == u].max() for u in units])
        unit_chunks = np.array([group_chunks[unit == u].sum() for u in units])
        unit_end = np.where(unit_chunks > 0, unit_end, np.nan)  # units without work do not count
        launches_out.append(dict(
            event_us=[round(float(x), 2) for x in event_us], wavefronts=int(t.shape[0]), work_groups=int(group_end.shape[0]),
            compute_units=int(units.shape[0]),
            entry=_pct(us(0)), lengths_in=_pct(us(1)), first_k_tile=_pct(us(2)[ran]), last_chunk_done=_pct(us(3)[ran]),
            last_store=_pct(us(4)), lengths_minus_entry=_pct(us(1) - us(0)), first_k_minus_lengths=_pct((us(2) - us(1))[ran]),
            store_minus_last_chunk=_pct((us(4) - us(3))[ran]),
            us_per_chunk=_pct(((us(3) - us(2))[ran]) / np.maximum(t[:, 5][ran], 1)),
            unit_end=_pct(unit_end, (0, 5, 25, 50, 75, 95, 100)),
            unit_chunks_over_mean=_pct(unit_chunks / unit_chunks.mean(), (0, 50, 100)),
            unit_end_by_xcc=[round(float(np.nanmean(unit_end[(units // 1024) == x])), 2) for x in range(8)]))
    return dict(config=idx, kernel=kernel, launches=launches_out)


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("configs", nargs="+", type=int, help="benchmark configurations (0-4)")
    ap.add_argument("--launches", type=int, default=5)
    ap.add_argument("--warm", type=int, default=6)
    ap.add_argument("--segment-partitions", type=int, default=None)
    ap.add_argument("--schedule", type=int, default=0)
    ap.add_argument("--json", action="store_true", help="one JSON object per configuration instead of the table")
    args = ap.parse_args()
    for idx in args.configs:
        res = timeline_of(idx, args.launches, args.warm, args.segment_partitions, args.schedule)
        if args.json:
            print(json.dumps(res), flush=True)
            continue
        first = res["launches"][0]
        print(f"config {idx} ({res['kernel']}): {first['work_groups']} work-groups, {first['wavefronts']} wavefronts on "
              f"{first['compute_units']} compute units; kernel time by HIP events, us: "
              f"{[l['event_us'] for l in res['launches']]}")
        med = lambda key: [round(float(np.median([l[key][i] for l in res["launches"]])), 2) for i in range(len(first[key]))]
        print(f"  {'us from the first entry; median over ' + str(len(res['launches'])) + ' launches of':58s} "
              f"{'min':>8s} {'p10':>8s} {'p50':>8s} {'p90':>8s} {'max':>8s}")
        for key, label in (("entry", "kernel entry (wavefronts)"), ("lengths_in", "context lengths in, items listed"),
                           ("first_k_tile", "first K tile in registers"), ("last_chunk_done", "last chunk done"),
                           ("last_store", "last merge stored"), ("lengths_minus_entry", "  listing: lengths in - entry"),
                           ("first_k_minus_lengths", "  first tile - lengths in"),
                           ("store_minus_last_chunk", "  last store - last chunk"),
                           ("us_per_chunk", "  us per chunk of a wavefront (32 keys of a head)")):
            print(f"  {label:58s} " + " ".join(f"{v:8.2f}" for v in med(key)))
        print(f"  {'when a compute unit finished: min p5 p25 p50 p75 p95 max':58s} " + " ".join(f"{v:8.2f}" for v in med("unit_end")))
        print(f"  {'chunks dealt to a unit / mean: min p50 max':58s} " + " ".join(f"{v:8.3f}" for v in med("unit_chunks_over_mean")))
        print(f"  {'mean finish of a unit by XCC 0-7':58s} " + " ".join(f"{v:8.2f}" for v in med("unit_end_by_xcc")), flush=True)


if __name__ == "__main__":
    main()
