// Single-pass ("loop") attention kernel, persistent form.
//
// Same results as the grid form (paged_attention_kernel.h with PART = false; upstream
// paged_attention_kernel_loop.hpp:610-636).  The grid form launches one work-group per
// (sequence, kv head); a decode batch of a few hundred such items of very different
// lengths then runs as a handful of waves of work-groups, each of which pays its own
// start-up (length -> block ids -> first K/V) and its own merge with nothing in flight.
// Here the launch holds only as many work-groups as stay resident, and each of them walks
// a list of items:
//   * items are ordered longest first (every wavefront ranks context_lens in registers)
//     and dealt to the work-groups in snake order, so the work-groups' totals are even;
//   * a wavefront that is through with its chunks of an item has already requested the
//     query rows and the first K/V chunk of the next item; it parks its softmax state in
//     LDS and goes on.  The states of an item are merged one chunk later, when all
//     wavefronts have as a rule long delivered theirs: there is no barrier between items
//     and the stream never drains.
// Built for up to 128 sequences of fewer than 2^24 tokens; anything else uses the grid form.
//
// EXT: the extended instance (score modifiers, several query tokens per sequence, per-head or
// per-block FP8 scales; see WaveAttn).  An item then also brings its ALiBi slope and scales,
// requested one item ahead like the query rows; chunks wholly before a local window are
// skipped, so an item starts at its first visible chunk.
#pragma once

#include "paged_attention_items.h"
#include "paged_attention_kernel.h"

// (debug builds with -DFA_TIMELINE) after a score pass: count it, and stamp the first one of the wavefront
#ifdef FA_TIMELINE
#define FA_TIMELINE_QK()              \
  do {                                \
    ++timeline_chunks;                \
    if (timeline_first) {             \
      timeline_first = false;         \
      FA_TIMELINE_STAMP(2);           \
    }                                 \
  } while (0)
#else
#define FA_TIMELINE_QK() ((void)0)
#endif

namespace fa {

constexpr int kLoopPersistentMaxSeqs = 128;
constexpr int kLoopPersistentMaxContext = 1 << 24;  // lengths are packed into 24 bits of a sort key
// Upper bound on the polls of one wait for the other wavefronts of a work-group (each poll
// sleeps ~64 cycles).  Never reached in a correct run -- every wavefront publishes every
// item -- it only turns a would-be hang into a wrong answer plus a flag in the launch's status
// word, which a timed call reports as FA_ERR_RUNTIME.
constexpr int kLoopPersistentSpinLimit = 1 << 24;
// What a kernel leaves in the status word (PagedAttnParams::status) when it gave up such a wait.
constexpr int32_t kStatusSpinLimit = 1;

//
template <int D, typename QT, int KVF, int NWG, int OCC, int TPC, bool EXT = false, bool KROW = true, int HPW = 1>
__global__ void __launch_bounds__(NWG * 64) __attribute__((amdgpu_waves_per_eu(OCC)))
paged_attn_loop_persistent_kernel(const PagedAttnParams p) {
  constexpr int NW = NWG;       // wavefronts of the work-group
  constexpr int NT = NW / HPW;  // of which a team of NT shares the chunks of one kv head of an item and merges
  using W = WaveAttn<D, QT, KVF, TPC, Pipeline<(KVF != 0)>::stream_loads_loop, EXT, KROW>;
  using Chunk = typename W::Chunk;
  using Ids = typename W::Ids;
  using ItemExt = typename W::ItemExt;
  using TileScales = typename W::TileScales;
  constexpr int CT = W::CT;
  constexpr int NR = W::NR;
  constexpr int NDT = W::NDT;
  constexpr int SL = NR / NT;
  static_assert(NT > 1 && NW % HPW == 0 && NR % NT == 0 && SL >= 2, "merge slices the output across wavefronts");

  FA_TIMELINE_STAMP(0);
  FA_TIMELINE_WHERE();
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int team = HPW == 1 ? 0 : wave / NT;   // which of the item's HPW adjacent kv heads
  const int tw = HPW == 1 ? wave : wave % NT;  // wavefront within the team
  const int G = gridDim.x;
  const int wg = blockIdx.x;
  [[maybe_unused]] int timeline_chunks = 0;
  [[maybe_unused]] bool timeline_first = true;
  const int col_max = p.max_blocks_per_seq - 1;

  // The items, (sequence, kv head) pairs with the longest sequences first, dealt in snake order;
  // c_lo: first chunk to read (0 unless EXT)
  using Item = WorkItem;
  LoopItems<TPC> items;
  items.build(p, lane, tw, G, CT, HPW);
  // with HPW > 1 an item is HPW adjacent kv heads of a sequence, of which this wavefront's team
  // takes one (kvh is then the team's own head)
  auto item_at = [&](int n, Item &it) -> bool {
    const bool there = items.at(n, G, wg, CT, it);
    if constexpr (HPW > 1) it.kvh = it.kvh * HPW + team;
    return there;
  };

  // Partial states of two items in flight: item n goes to buffer n & 1.
  __shared__ float sm_m[2][NW][16];
  __shared__ float sm_l[2][NW][16];
  __shared__ float sm_acc[2][NW][NR][64];
  __shared__ int sm_arrived[2];  // wavefronts that have published into the buffer, ever

  W wa(p, lane);
  const int r = wa.r, i = wa.i;
  Chunk R;

  int n = 0;
  Item cur;
  if (!item_at(0, cur)) return;  // the same for every wavefront of the work-group
  FA_TIMELINE_STAMP(1);
  if constexpr (EXT) cur.c_lo = wa.first_visible_chunk(cur.ctx, 0);
  if (threadIdx.x < 2) sm_arrived[threadIdx.x] = 0;
  __syncthreads();  // the only barrier: wavefronts meet through the counters from here on

  // A wavefront's state of item n goes to LDS and the wavefront moves on; nobody waits here.
  auto publish = [&](int item) {
    const int b = item & 1;
    wa.settle();
    wa.l = rows_sum(wa.l);
    if (r == 0) {
      sm_m[b][wave][i] = wa.m;
      sm_l[b][wave][i] = wa.l;
    }
#pragma unroll
    for (int k = 0; k < NR; ++k) sm_acc[b][wave][k][lane] = wa.acc_at(k);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    if (lane == 0)
      __hip_atomic_fetch_add(&sm_arrived[b], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  };
  // Merge the NW published states of an item, normalise, store this wavefront's slice.
  // Called one chunk into the following item (or after the last item), when the other
  // wavefronts have as a rule long published: the wait below is then a single read.
  // Every wavefront publishes every item in order, so the count is always reached; a
  // wavefront calls finish(item) before it publishes item + 1, and finish(item) returns
  // only after all have published `item`, hence after all have finished item - 1: a
  // buffer is never overwritten while somebody still reads it.
  auto finish = [&](int item, int seq, int kvh, float out_mul) {
    const int b = item & 1;
    const int target = NW * ((item >> 1) + 1);
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
    for (int k = 0; k < SL; ++k) {
      float a = 0.f;
#pragma unroll
      for (int u = 0; u < NT; ++u) a += f[u] * sm_acc[b][w0 + u][tw * SL + k][lane];
      o[k] = a;
    }
    if (wa.col_valid && wa.keeps_output()) {
      const int head = kvh * p.group + wa.col_g;
      const int d0 = wa.out_elem(4 * r * NDT + tw * SL);
      int64_t row = seq;
      float inv = p.out_scale / L;
      if constexpr (EXT) {
        row = (int64_t)seq * p.query_len + wa.col_q;
        inv = L > 0.f ? out_mul / L : 0.f;  // L = 0: the query token sees no key
      }
      W::template store_q<SL>(
          reinterpret_cast<char *>(p.out) + ((row * p.num_heads + head) * wa.out_row_elems() + d0) * 2, o, inv);
    }
  };

  // first chunk of the first item
  bool armed = cur.c_lo + tw < cur.c_end;  // loads of this wavefront's first chunk of `cur` in flight
  ItemExt cur_ext = {}, nxt_ext = {};         // extended instances only
  TileScales ts = {}, nts = {}, nxt_ts = {};
  if constexpr (EXT) cur_ext = wa.fetch_item_ext(cur.kvh, p.block_tables + (int64_t)cur.seq * p.max_blocks_per_seq);
  if (armed) {
    Ids ids;
#pragma unroll
    for (int t = 0; t < TPC; ++t) {
      ids.v[t] = min((uint32_t)items.first_id(t, cur.seq), (uint32_t)p.max_block_id);
    }
    if constexpr (EXT) {
      if (cur.c_lo != 0)  // the ids requested with the lengths are those of chunk `tw`
        ids = wa.fetch_ids(p.block_tables + (int64_t)cur.seq * p.max_blocks_per_seq, cur.c_lo + tw, col_max);
    }
    wa.load_q(cur.seq, cur.kvh);
    wa.issue_k(R, cur.kvh, cur.c_lo + tw, ids);
    wa.issue_v(R, cur.kvh, cur.c_lo + tw, ids);
    if constexpr (EXT) ts = wa.fetch_scales(ids, cur.kvh, cur_ext);
  }
  uint32_t sink_raw = wa.load_sink(cur.kvh, tw == 0);
  Item prev = cur;  // the item whose merge is still owed (from the second item on)
  float prev_out_mul = 1.f;

  while (true) {
    Item nxt;
    const bool has_next = item_at(n + 1, nxt);
    if constexpr (EXT) {
      if (has_next) {
        nxt.c_lo = wa.first_visible_chunk(nxt.ctx, 0);
        nxt_ext = wa.fetch_item_ext(nxt.kvh, p.block_tables + (int64_t)nxt.seq * p.max_blocks_per_seq);
      }
    }
    const bool next_armed = has_next && nxt.c_lo + tw < nxt.c_end;
    Ids nxt_ids = {};
    if (next_armed)
      nxt_ids = wa.fetch_ids(p.block_tables + (int64_t)nxt.seq * p.max_blocks_per_seq, nxt.c_lo + tw, col_max);

    wa.reset(sink_raw);
    if constexpr (EXT) wa.set_item(cur_ext, cur.ctx);
    uint32_t next_sink = W::kNoSink;
    if constexpr (EXT) {  // the sink goes with the item whether or not wavefront 0 has a chunk of it
      if (has_next && !next_armed) next_sink = wa.load_sink(nxt.kvh, tw == 0);
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
          const auto pb = wa.template soft<false, EXT>(R, s, ci, cur.ctx, &ts);
          wa.pv(R, pb);
          wa.issue_v(R, cur.kvh, cn, nids);
          nids = wa.fetch_ids(table, cn + NT, col_max);
          ts = nts;
          ci = cn;
        }
        if (owed) {
          finish(n - 1, prev.seq, prev.kvh, prev_out_mul);
          owed = false;
        }
        while (ci + NT < cur.c_end) {  // steady state: the next chunk belongs to the same item
          const int cn = ci + NT;
          const auto s = wa.qk(R);
          FA_TIMELINE_QK();
          wa.issue_k(R, cur.kvh, cn, nids);
          if constexpr (EXT) nts = wa.fetch_scales(nids, cur.kvh, cur_ext);
          const auto pb = wa.template soft<false, EXT>(R, s, ci, cur.ctx, &ts);
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
        next_sink = wa.load_sink(nxt.kvh, tw == 0);
        wa.issue_k(R, nxt.kvh, nxt.c_lo + tw, nxt_ids);
        if constexpr (EXT) nxt_ts = wa.fetch_scales(nxt_ids, nxt.kvh, nxt_ext);
      }
      const auto pb = wa.template soft<true, EXT>(R, s, ci, cur.ctx, &ts);
      wa.pv(R, pb);
      if (next_armed) wa.issue_v(R, nxt.kvh, nxt.c_lo + tw, nxt_ids);
    } else if (next_armed) {  // nothing to do in `cur`, but the next item starts here
      wa.load_q(nxt.seq, nxt.kvh);
      next_sink = wa.load_sink(nxt.kvh, tw == 0);
      wa.issue_k(R, nxt.kvh, nxt.c_lo + tw, nxt_ids);
      wa.issue_v(R, nxt.kvh, nxt.c_lo + tw, nxt_ids);
      if constexpr (EXT) nxt_ts = wa.fetch_scales(nxt_ids, nxt.kvh, nxt_ext);
    }
    if (!has_next) FA_TIMELINE_STAMP(3);
    if (owed) finish(n - 1, prev.seq, prev.kvh, prev_out_mul);
    publish(n);

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
  finish(n, cur.seq, cur.kvh, EXT ? cur_ext.out_mul : 1.f);
  FA_TIMELINE_STAMP(4);
  FA_TIMELINE_PUT(5, timeline_chunks);
}

}  // namespace fa
