// Split-context attention kernel, persistent form with multi-wavefront work-groups.
//
// Same role as the other split kernels (upstream paged_attention_kernel_v2.hpp:572-587):
// partial softmax states go to exp_sums / max_logits / tmp_out and the reduce kernel merges
// them.  What differs is how much of a sequence one partial covers.  With one partial per
// 512-token partition a large ragged batch writes thousands of 512-byte rows scattered over
// the scratch arrays, and a few percent of scattered writes mixed into a saturated read
// stream cost far more than their bytes.  Here a work-group of NW wavefronts takes a SEGMENT
// of m consecutive partitions of one (sequence, kv head): its wavefronts interleave the
// segment's chunks, merge their states in LDS (no barrier: the deferred merge of the
// persistent loop kernel) and write ONE partial into the slot of the segment's first
// partition.  The other m - 1 slots of max_logits get a mark (segment_mark) by which the reduce
// kernel tells them from slots that hold partials.
// A sequence that fits one segment has one partial, which is its result: that one is rounded to
// the query type and stored into the call's `out` (PagedAttnParams::final_out), its scalars into
// exp_sums and max_logits as ever, and the reduce kernel leaves the row alone -- in a batch of
// many sequences that is most rows, and spares them the trip through tmp_out.
//
// m is chosen on the device from the batch itself -- every wavefront evaluates
// partitions_per_segment() on the same context lengths -- so that a segment is about what a
// compute unit, or a work-group of it, should stream: a batch of few long sequences gets one
// segment per unit or per work-group.  Segments are dealt to the work-groups longest first in
// snake order (see below).  On request (options->segment_partitions = -1) a batch is cut differently,
// into even shares: the rows laid end to end, one contiguous share per work-group, so that a
// work-group's pieces are the end of one row, whole rows and the beginning of another
// (paged_attention_segment_policy.h).
// Built for up to 256 sequences; larger batches use the grid form.
//
// EXT: the extended instance (score modifiers, several query tokens per sequence, per-head or
// per-block FP8 scales; see WaveAttn).  Rows of the scratch arrays are then (sequence, query
// token) pairs.  A segment starts at its first chunk inside the local window; one that lies
// wholly before the window publishes empty states and stores an empty partial (max -inf,
// sum 0, zeros), which the reduce kernel weighs with 0.
#pragma once

#include "paged_attention_items.h"
#include "paged_attention_kernel.h"
#include "paged_attention_loop_persistent_kernel.h"
#include "paged_attention_segment_policy.h"

// Builds that time what the stores of the partials cost (profiles/): 1 leaves out the rows of tmp_out,
// 2 the scalars as well.  Their results are wrong; the product is built with 0.
#ifndef FA_COST_PROBE
#define FA_COST_PROBE 0
#endif

namespace fa {

//
template <int D, typename QT, int KVF, int NWG, int OCC, int TPC, bool EXT = false, int HPW = 1>
__global__ void __launch_bounds__(NWG * 64) __attribute__((amdgpu_waves_per_eu(OCC)))
paged_attn_segment_kernel(const PagedAttnParams p) {
  constexpr int NW = NWG;       // wavefronts of the work-group
  constexpr int NT = NW / HPW;  // of which a team of NT shares a segment's chunks of one kv head and merges
  using W = WaveAttn<D, QT, KVF, TPC, SegmentSplit<(KVF != 0)>::stream_loads, EXT>;
  using Chunk = typename W::Chunk;
  using Ids = typename W::Ids;
  using ItemExt = typename W::ItemExt;
  using TileScales = typename W::TileScales;
  constexpr int CT = W::CT;
  constexpr int NR = W::NR;
  constexpr int NDT = W::NDT;
  constexpr int SL = NR / NT;
  static_assert(NT >= 1 && NW % HPW == 0 && NR % NT == 0 && SL >= 4 && SL % 4 == 0,
                "each wavefront stores whole 16-byte pieces");
  // NT == 1: every wavefront has a kv head of its own and the whole of each item's chunks, so an item's
  // state never leaves its registers: no LDS, no waiting for the others.

  FA_TIMELINE_STAMP(0);
  FA_TIMELINE_WHERE();
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int team = HPW == 1 ? 0 : wave / NT;   // which of the item's HPW adjacent kv heads
  const int tw = HPW == 1 ? wave : wave % NT;  // wavefront within the team
  const int G = gridDim.x;
  [[maybe_unused]] int timeline_chunks = 0;
  [[maybe_unused]] bool timeline_first = true;
  const int col_max = p.max_blocks_per_seq - 1;

  // The segment list (SegmentItems): all full segments, then the sequences' last, shorter segments
  // in order of length, dealt to the work-groups in snake order, so that the work-groups' totals
  // come out even although a work-group only gets a handful of segments.
  using Item = WorkItem;  // c_lo .. c_end: the segment's chunks; ctx: the sequence's length (EXT)
  SegmentItems items;
  items.build(p, lane, G, HPW, W::ROWB * HPW);
  // n-th item of this work-group; with HPW > 1 an item is HPW adjacent kv heads of one segment, of
  // which this wavefront's team takes one (kvh is then the team's own head)
  auto item_at = [&](int nth, Item &it) {
    const bool there = items.at(nth, G, (int)blockIdx.x, CT, it);
    if constexpr (HPW > 1) it.kvh = it.kvh * HPW + team;
    return there;
  };

  // Partial states of two items in flight: the n-th item of this work-group goes to buffer n & 1.
  __shared__ float sm_m[2][NW][16];
  __shared__ float sm_l[2][NW][16];
  __shared__ float sm_acc[2][NW][NR][64];
  __shared__ int sm_arrived[2];  // wavefronts that have published into the buffer, ever

  Item cur;
  if (!item_at(0, cur)) return;  // the same for every wavefront of the work-group
  FA_TIMELINE_STAMP(1);
  if (threadIdx.x < 2) sm_arrived[threadIdx.x] = 0;
  __syncthreads();  // the only barrier: wavefronts meet through the counters from here on

  W wa(p, lane);
  const int r = wa.r, i = wa.i;
  Chunk R;
  // EXT: a segment is read from its first chunk inside the local window
  auto clip = [&](Item &it) {
    if constexpr (EXT) it.c_lo = wa.first_visible_chunk(it.ctx, it.c_lo);
  };

  auto publish = [&](int n) {
    const int b = n & 1;
    wa.settle();
    wa.l = rows_sum(wa.l);
    if (r == 0) {
      sm_m[b][wave][i] = wa.m;
      sm_l[b][wave][i] = wa.l;
    }
#pragma unroll
    for (int e = 0; e < NR; ++e) sm_acc[b][wave][e][lane] = wa.acc_at(e);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    if (lane == 0)
      __hip_atomic_fetch_add(&sm_arrived[b], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  };
  // Store this wavefront's slice o[SL] of an item's merged, un-normalised output (maximum M in base-2
  // units, sum L) as the item's partial -- or, where the item is its row's only piece, as the row's result.
  auto store_slice = [&](const Item &it, float M, float L, const float (&o)[SL], float out_mul) {
    if (wa.col_valid && wa.keeps_output()) {
      const int head = it.kvh * p.group + wa.col_g;
      int64_t row = it.seq;
      float inv = p.out_scale / L;
      if constexpr (EXT) {
        row = (int64_t)it.seq * p.query_len + wa.col_q;
        inv = L > 0.f ? out_mul / L : 0.f;  // L = 0: the query token sees no key of the segment
      }
      const int64_t slot = (row * p.num_heads + head) * p.max_num_partitions + it.part0;
      const int d0 = wa.out_elem(4 * r * NDT + tw * SL);
      // the row's only partial is its result (PagedAttnParams::final_out); it.ctx is the length as
      // far as the scratch arrays hold it
      if (p.final_out != nullptr && it.part0 == 0 && it.tok_end >= it.ctx)
        W::template store_q<SL>(
            reinterpret_cast<char *>(p.final_out) + ((row * p.num_heads + head) * wa.out_row_elems() + d0) * 2, o, inv);
      else if (FA_COST_PROBE < 1)  // (cost probes: 1 = no rows of partials, 2 = no scalars either)
        W::template store_f32<SL>(reinterpret_cast<float *>(p.out) + slot * wa.out_row_elems() + d0, o, inv);
      if ((wa.paired() ? (r & 1) == 0 : r == 0) && tw == 0 && FA_COST_PROBE < 2) {  // one lane per column, see merge_and_store
        p.max_logits[slot] = M * kLn2;  // natural-log units, as upstream stores them
        p.exp_sums[slot] = L;
      }
    }
    // the slots that the piece covers beyond its first tell the reduce kernel that they hold no partial
    if (tw == 0 && it.parts > 1) {
      const int rows = EXT ? p.query_count : 1;  // query tokens of the launch
      for (int q = 0; q < rows; ++q) {
        const int64_t row = EXT ? (int64_t)it.seq * p.query_len + p.query_first + q : it.seq;
        mark_covered_slots(p.max_logits, (row * p.num_heads + (int64_t)it.kvh * p.group) * p.max_num_partitions + it.part0,
                           p.group, p.max_num_partitions, it.parts, lane, items.m);
      }
    }
  };
  // NT == 1: the item at hand straight from the registers.  (A lane holds NR consecutive floats of its
  // head's row, so a store instruction puts 16 bytes into each of 32 lines.  Exchanging pieces through
  // LDS first, so that eight lanes write a whole line, was built and timed: 317 -> 310 us on the serving
  // mix with one partial per partition, 120 -> 140 us on the long-context batch; not kept.)
  auto store_own = [&](const Item &it, float out_mul) {
    wa.settle();
    const float L = rows_sum(wa.l);
    float o[SL];
#pragma unroll
    for (int e = 0; e < SL; ++e) o[e] = wa.acc_at(e);
    store_slice(it, wa.m, L, o, out_mul);
  };
  // Merge the NW published states of the work-group's n-th item, normalise, store this
  // wavefront's slice of the partial (see the persistent loop kernel for why the wait
  // always ends and why a buffer is never overwritten while it is read).
  auto finish = [&](int n, const Item &it, float out_mul) {
    if constexpr (NT > 1) {  // (NT == 1: stored when the item ended, store_own)
    const int b = n & 1;
    const int target = NW * ((n >> 1) + 1);
    bool arrived = false;
    for (int spin = 0; spin < p.spin_limit; ++spin) {
      const int seen = __hip_atomic_load(&sm_arrived[b], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      if (__builtin_amdgcn_readfirstlane(seen) >= target) {
        arrived = true;
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    // Gave up: what follows merges states that are not all there, so the result is wrong; say so in
    // the status word (one lane, a plain vector store) and carry on, so that the grid still drains.
    if (!arrived && lane == 0) __hip_atomic_store(p.status, kStatusSpinLimit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    const int w0 = team * NT;  // the team's wavefronts: w0 .. w0 + NT - 1
    float M = -INFINITY;
#pragma unroll
    for (int u = 0; u < NT; ++u) M = fmaxf(M, sm_m[b][w0 + u][i]);
    float f[NT];
    float L = 0.f;
#pragma unroll
    for (int u = 0; u < NT; ++u) {
      const float mw = sm_m[b][w0 + u][i];
      f[u] = (mw == -INFINITY) ? 0.f : fast_exp2(mw - M);  // a wavefront without chunks
      L += f[u] * sm_l[b][w0 + u][i];
    }
    float o[SL];
#pragma unroll
    for (int e = 0; e < SL; ++e) {
      float a = 0.f;
#pragma unroll
      for (int u = 0; u < NT; ++u) a += f[u] * sm_acc[b][w0 + u][tw * SL + e][lane];
      o[e] = a;
    }
    store_slice(it, M, L, o, out_mul);
    }
  };

  int n = 0;
  clip(cur);
  // first chunk of the first item
  bool armed = cur.c_lo + tw < cur.c_end;  // loads of this wavefront's first chunk of `cur` in flight
  ItemExt cur_ext = {}, nxt_ext = {};            // extended instances only
  TileScales ts = {}, nts = {}, nxt_ts = {};
  if constexpr (EXT) cur_ext = wa.fetch_item_ext(cur.kvh, p.block_tables + (int64_t)cur.seq * p.max_blocks_per_seq);
  if (armed) {
    const Ids ids = wa.fetch_ids(p.block_tables + (int64_t)cur.seq * p.max_blocks_per_seq, cur.c_lo + tw, col_max);
    wa.load_q(cur.seq, cur.kvh);
    wa.issue_k(R, cur.kvh, cur.c_lo + tw, ids);
    wa.issue_v(R, cur.kvh, cur.c_lo + tw, ids);
    if constexpr (EXT) ts = wa.fetch_scales(ids, cur.kvh, cur_ext);
  }
  uint32_t sink_raw = wa.load_sink(cur.kvh, tw == 0 && cur.part0 == 0);
  Item prev = cur;  // the item whose merge is still owed (from the second item on)
  float prev_out_mul = 1.f;

  while (true) {
    Item nxt = cur;
    const bool has_next = item_at(n + 1, nxt);
    if (has_next) {
      clip(nxt);
      if constexpr (EXT)
        nxt_ext = wa.fetch_item_ext(nxt.kvh, p.block_tables + (int64_t)nxt.seq * p.max_blocks_per_seq);
    }
    const bool next_armed = has_next && nxt.c_lo + tw < nxt.c_end;
    Ids nxt_ids = {};
    if (next_armed)
      nxt_ids = wa.fetch_ids(p.block_tables + (int64_t)nxt.seq * p.max_blocks_per_seq, nxt.c_lo + tw, col_max);

    wa.reset(sink_raw);
    if constexpr (EXT) wa.set_item(cur_ext, cur.ctx);
    uint32_t next_sink = W::kNoSink;
    if constexpr (EXT) {
      // a segment before the local window arms no wavefront, yet its partial carries the sink
      if (has_next && !next_armed) next_sink = wa.load_sink(nxt.kvh, tw == 0 && nxt.part0 == 0);
    }
    bool owed = n > 0;
    if (armed) {
      const int32_t *table = p.block_tables + (int64_t)cur.seq * p.max_blocks_per_seq;
      int ci = cur.c_lo + tw;
      Ids nids = wa.fetch_ids(table, ci + NT, col_max);
      if (ci + NT < cur.c_end) {
        {  // first chunk of the item, then the merge owed to the previous item
          const int cn = ci + NT;
          const auto s = wa.qk(R);
          FA_TIMELINE_QK();
          wa.issue_k(R, cur.kvh, cn, nids);
          if constexpr (EXT) nts = wa.fetch_scales(nids, cur.kvh, cur_ext);
          const auto pb = wa.template soft<false, EXT>(R, s, ci, cur.tok_end, &ts);
          wa.pv(R, pb);
          wa.issue_v(R, cur.kvh, cn, nids);
          nids = wa.fetch_ids(table, cn + NT, col_max);
          ts = nts;
          ci = cn;
        }
        if (owed) {
          finish(n - 1, prev, prev_out_mul);
          owed = false;
        }
        while (ci + NT < cur.c_end) {  // steady state: the next chunk belongs to the same item
          const int cn = ci + NT;
          const auto s = wa.qk(R);
          FA_TIMELINE_QK();
          wa.issue_k(R, cur.kvh, cn, nids);
          if constexpr (EXT) nts = wa.fetch_scales(nids, cur.kvh, cur_ext);
          const auto pb = wa.template soft<false, EXT>(R, s, ci, cur.tok_end, &ts);
          wa.pv(R, pb);
          wa.issue_v(R, cur.kvh, cn, nids);
          nids = wa.fetch_ids(table, cn + NT, col_max);
          ts = nts;
          ci = cn;
        }
      }
      // last chunk of this wavefront in `cur`: what goes out next belongs to `nxt`
      const auto s = wa.qk(R);
      FA_TIMELINE_QK();
      if (next_armed) {
        wa.load_q(nxt.seq, nxt.kvh);  // Q registers are free once the last scores are out
        next_sink = wa.load_sink(nxt.kvh, tw == 0 && nxt.part0 == 0);
        wa.issue_k(R, nxt.kvh, nxt.c_lo + tw, nxt_ids);
        if constexpr (EXT) nxt_ts = wa.fetch_scales(nxt_ids, nxt.kvh, nxt_ext);
      }
      const auto pb = wa.template soft<true, EXT>(R, s, ci, cur.tok_end, &ts);
      wa.pv(R, pb);
      if (next_armed) wa.issue_v(R, nxt.kvh, nxt.c_lo + tw, nxt_ids);
    } else if (next_armed) {  // nothing to do in `cur`, but the next item starts here
      wa.load_q(nxt.seq, nxt.kvh);
      next_sink = wa.load_sink(nxt.kvh, tw == 0 && nxt.part0 == 0);
      wa.issue_k(R, nxt.kvh, nxt.c_lo + tw, nxt_ids);
      wa.issue_v(R, nxt.kvh, nxt.c_lo + tw, nxt_ids);
      if constexpr (EXT) nxt_ts = wa.fetch_scales(nxt_ids, nxt.kvh, nxt_ext);
    }
    if (!has_next) FA_TIMELINE_STAMP(3);
    if (owed) finish(n - 1, prev, prev_out_mul);
    if constexpr (NT == 1) store_own(cur, EXT ? cur_ext.out_mul : 1.f);
    else publish(n);

    if (!has_next) break;
    prev = cur;
    cur = nxt;
    armed = next_armed;
    sink_raw = next_sink;
    if constexpr (EXT) {
      prev_out_mul = cur_ext.out_mul;
      cur_ext = nxt_ext;
      ts = nxt_ts;
    }
    ++n;
  }
  finish(n, cur, EXT ? cur_ext.out_mul : 1.f);
  FA_TIMELINE_STAMP(4);
  FA_TIMELINE_PUT(5, timeline_chunks);
}

}  // namespace fa
