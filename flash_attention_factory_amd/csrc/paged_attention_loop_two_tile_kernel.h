// Single-pass ("loop") attention kernel, persistent form, for query blocks of two column tiles.
//
// The extended persistent loop kernel (paged_attention_loop_persistent_kernel.h) fills the 16
// MFMA columns of a kv head with (query token, head) pairs.  A launch of up to 32 such pairs --
// a speculative-decoding step of 4 tokens over a group of 8 heads, 32 tokens of one head -- needs
// two column tiles.  Here BOTH tiles live in the registers of the same wavefront: one chunk of K
// and V is loaded once, every operand is built once and feeds the MFMAs of both tiles
// (WaveAttn::qk_two, pv_two), each tile keeps its own queries, softmax state and accumulators,
// masks by its own columns' positions and is merged and stored for itself.  K and V cross HBM
// and the caches exactly once per launch.  The price is registers (two sets of queries and
// accumulators): one wavefront per SIMD, so nothing else hides a wavefront's waits for memory.
//
// That is why a wavefront keeps TWO chunks in registers (R0, R1: chunk j of an item sits in
// R(j & 1)): while chunk j is computed, chunk j+1 is on its way, and as soon as the scores (the
// values) of chunk j are out, K (V) of chunk j+2 is requested into the registers just freed.
// Every load has a chunk and a half of compute to arrive.  Across items: the first chunk of the
// next item is requested into R0 by the last step of the current item that uses R0, together
// with what the item needs beyond K and V (queries, sinks, per-item multipliers).
//
// The wait counts in front of the MFMAs are fixed when the kernel is compiled, for the worst of
// all paths that lead there; a path on which a load was skipped is one on which the registers
// about to be used hold the newest load, and the count would be zero.  So the loop that runs
// for most of an item (`steady`) requests its loads unconditionally, is entered only from code
// that has requested both register sets; the one to three chunks that end an item (or make up a
// short one) go through steps with conditions.
//
// Item order (longest first, dealt in a snake over the work-groups) and the merge through LDS
// without barriers (publish / finish, one arrival counter per buffer): as in the one-tile kernel,
// except that the merge owed to item n-1 is done one chunk into a long item n (its stores add
// operations to one path into the loop's waits and cannot lower a count), else at its end.
#pragma once

#include "paged_attention_items.h"
#include "paged_attention_loop_persistent_kernel.h"

namespace fa {

// PART: the split path.  Items are segments of partitions (SegmentItems), what is stored per item
// and column is a partial -- max, sum and normalised values in exp_sums / max_logits / tmp_out at
// the slot of the segment's first partition -- and the reduce kernel follows.
template <int D, typename QT, int KVF, int NWG, int TPC, bool KROW = true, bool PART = false, int HPW = 1>
__global__ void __launch_bounds__(NWG * 64) __attribute__((amdgpu_waves_per_eu(1)))
paged_attn_loop_two_tile_kernel(const PagedAttnParams p) {
  constexpr int NW = NWG;       // wavefronts of the work-group
  constexpr int NT = NW / HPW;  // of which a team of NT shares the chunks of one kv head of an item and merges
  using W = WaveAttn<D, QT, KVF, TPC, PART ? SegmentSplit<(KVF != 0)>::stream_loads : Pipeline<(KVF != 0)>::stream_loads_loop, true, KROW>;
  using Chunk = typename W::Chunk;
  using Ids = typename W::Ids;
  using ItemExt = typename W::ItemExt;
  using TileScales = typename W::TileScales;
  using Scores = typename W::Scores;
  constexpr int CT = W::CT;
  constexpr int NR = W::NR;
  constexpr int NDT = W::NDT;
  constexpr int SL = NR / NT;
  static_assert(NT > 1 && NW % HPW == 0 && NR % NT == 0 && SL >= 2, "merge slices the output across wavefronts");

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int team = HPW == 1 ? 0 : wave / NT;   // which of the item's HPW adjacent kv heads
  const int tw = HPW == 1 ? wave : wave % NT;  // wavefront within the team
  const int G = gridDim.x;
  const int wg = blockIdx.x;
  const int col_max = p.max_blocks_per_seq - 1;

  W wa(p, lane, 0), wb(p, lane, 1);  // the two column tiles
  const int r = wa.r, i = wa.i;
  using Item = WorkItem;
  std::conditional_t<PART, SegmentItems, LoopItems<TPC>> items;
  if constexpr (PART) items.build(p, lane, G, HPW, W::ROWB * HPW);
  else items.build(p, lane, tw, G, CT, HPW);
  // n-th item of this work-group, read from its first chunk that some query token of the launch
  // sees (local window; the launch's earliest query token decides: the same for both tiles)
  auto item_at = [&](int n, Item &it) __attribute__((always_inline)) -> bool {
    if (!items.at(n, G, wg, CT, it)) return false;
    // with HPW > 1 an item is HPW adjacent kv heads, of which this wavefront's team takes one
    if constexpr (HPW > 1) it.kvh = it.kvh * HPW + team;
    it.c_lo = wa.first_visible_chunk(it.ctx, it.c_lo);
    return true;
  };

  // Partial states of two items in flight, per column tile: item n goes to buffer n & 1.
  __shared__ float sm_m[2][2][NW][16];
  __shared__ float sm_l[2][2][NW][16];
  __shared__ float sm_mt[PART ? 2 : 1][2][NW][16];  // true maxima (split path: max_logits)
  __shared__ float sm_acc[2][2][NW][NR][64];
  __shared__ int sm_arrived[2];  // wavefronts that have published (both tiles) into the buffer, ever

  Item first;
  if (!item_at(0, first)) return;  // the same for every wavefront of the work-group
  if (threadIdx.x < 2) sm_arrived[threadIdx.x] = 0;
  __syncthreads();  // the only barrier: wavefronts meet through the counters from here on

  // A wavefront's states of item n go to LDS and the wavefront moves on; nobody waits here.
  // The states go out as they are, sums and accumulators against the reference maximum m, which may
  // lag the true one (mt): a pass over 64 accumulators in AGPRs to bring them up (WaveAttn::settle)
  // would cost more than everything else here, and the merge is indifferent to the reference.
  auto publish_tile = [&](W &w, int tile, int b) __attribute__((always_inline)) {
    w.l = rows_sum(w.l);
    if (r == 0) {
      sm_m[tile][b][wave][i] = w.m;
      sm_l[tile][b][wave][i] = w.l;
      if constexpr (PART) sm_mt[tile][b][wave][i] = w.mt;
    }
#pragma unroll
    for (int k = 0; k < NR; ++k) sm_acc[tile][b][wave][k][lane] = w.acc_at(k);
  };
  auto publish = [&](int item) __attribute__((always_inline)) {
    const int b = item & 1;
    publish_tile(wa, 0, b);
    publish_tile(wb, 1, b);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    if (lane == 0) __hip_atomic_fetch_add(&sm_arrived[b], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  };
  // Merge the NW published states of one tile of an item, normalise, store this wavefront's slice.
  // whole: the item is the row's only partial, which goes to the call's `out` as its result
  // (PagedAttnParams::final_out)
  auto finish_tile = [&](W &w, int tile, int b, int seq, int kvh, int part0, bool whole, float out_mul) __attribute__((always_inline)) {
    const int w0 = team * NT;  // the team's wavefronts: w0 .. w0 + NT - 1
    float M = -INFINITY;
#pragma unroll
    for (int u = 0; u < NT; ++u) M = fmaxf(M, sm_m[tile][b][w0 + u][i]);
    float f[NT];
    float L = 0.f;
#pragma unroll
    for (int u = 0; u < NT; ++u) {
      const float mv = sm_m[tile][b][w0 + u][i];
      f[u] = (mv == -INFINITY) ? 0.f : fast_exp2(mv - M);  // a wavefront without chunks
      L += f[u] * sm_l[tile][b][w0 + u][i];
    }
    float o[SL];
#pragma unroll
    for (int k = 0; k < SL; ++k) {
      float a = 0.f;
#pragma unroll
      for (int u = 0; u < NT; ++u) a += f[u] * sm_acc[tile][b][w0 + u][tw * SL + k][lane];
      o[k] = a;
    }
    if (w.col_valid) {
      const int head = kvh * p.group + w.col_g;
      const int d0 = 4 * r * NDT + tw * SL;
      const int64_t row = (int64_t)seq * p.query_len + w.col_q;
      const float inv = L > 0.f ? out_mul / L : 0.f;  // L = 0: the query token sees no key (of the segment)
      if constexpr (PART) {
        const int64_t slot = (row * p.num_heads + head) * p.max_num_partitions + part0;
        if (whole)
          W::template store_q<SL>(reinterpret_cast<char *>(p.final_out) + ((row * p.num_heads + head) * D + d0) * 2, o, inv);
        else
          W::template store_f32<SL>(reinterpret_cast<float *>(p.out) + slot * D + d0, o, inv);
        if (r == 0 && tw == 0) {  // one lane per column: the true maximum, and the sum against it
          float MT = -INFINITY;
#pragma unroll
          for (int u = 0; u < NT; ++u) MT = fmaxf(MT, sm_mt[tile][b][w0 + u][i]);
          p.max_logits[slot] = MT * kLn2;  // natural-log units, as upstream stores them
          p.exp_sums[slot] = MT == -INFINITY ? 0.f : L * fast_exp2(M - MT);
        }
      } else {
        W::template store_q<SL>(reinterpret_cast<char *>(p.out) + ((row * p.num_heads + head) * D + d0) * 2, o, inv);
      }
    }
  };
  // Every wavefront runs  ... finish(n-2), publish(n-1), finish(n-1), publish(n) ...  in this order.
  // finish(n-1) waits for the publish(n-1) of all wavefronts, none of which waits for anything
  // later than finish(n-2): the wait ends.  And publish(n) overwrites the buffer of item n-2 only
  // after finish(n-1) has seen every wavefront's publish(n-1), which each of them issues after
  // its finish(n-2).
  auto finish = [&](int item, const Item &it, float out_mul) __attribute__((always_inline)) {
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
    if (!arrived && lane == 0) __hip_atomic_store(p.status, kStatusSpinLimit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    bool whole = false;
    if constexpr (PART) whole = p.final_out != nullptr && it.part0 == 0 && it.tok_end >= it.ctx;
    finish_tile(wa, 0, b, it.seq, it.kvh, it.part0, whole, out_mul);
    finish_tile(wb, 1, b, it.seq, it.kvh, it.part0, whole, out_mul);
    if constexpr (PART) {
      // the slots that the piece covers beyond its first tell the reduce kernel that they hold no partial
      if (tw == 0 && it.parts > 1) {
        for (int q = 0; q < p.query_count; ++q) {
          const int64_t row = (int64_t)it.seq * p.query_len + p.query_first + q;
          mark_covered_slots(p.max_logits, (row * p.num_heads + (int64_t)it.kvh * p.group) * p.max_num_partitions + it.part0,
                             p.group, p.max_num_partitions, it.parts, lane, items.m);
        }
      }
    }
  };
  auto table_of = [&](int seq) __attribute__((always_inline)) { return p.block_tables + (int64_t)seq * p.max_blocks_per_seq; };
  // this wavefront's chunks of an item: c_lo + tw, + NW, ... below c_end
  auto count_of = [&](const Item &it) __attribute__((always_inline)) { return max(0, (it.c_end - it.c_lo - tw + NT - 1) / NT); };

  Chunk R0, R1;
  TileScales ts0 = {}, ts1 = {};  // multipliers of the chunks in R0, R1
  bool k1_ready = false;          // K of the item's second chunk has been requested into R1 already
  constexpr int kWaitVmcnt0 = 0x0F70;  // s_waitcnt vmcnt(0), no wait on the other counters

  int n = 0;
  Item cur = first;
  int m = count_of(cur);  // chunks of `cur` this wavefront computes; the first is in flight in R0 if there is one
  ItemExt cur_a = wa.fetch_item_ext(cur.kvh, table_of(cur.seq)), cur_b = wb.fetch_item_ext(cur.kvh, table_of(cur.seq));
  ItemExt nxt_a = {}, nxt_b = {};
  Ids ids1 = {};  // block ids of the item's second chunk, requested an item early
  if (m > 0) {
    Ids ids;
    bool have_ids = false;
    if constexpr (!PART) {
      if (cur.c_lo == 0) {  // the ids requested with the lengths are those of chunk `tw`
#pragma unroll
        for (int t = 0; t < TPC; ++t) ids.v[t] = min((uint32_t)items.first_id(t, cur.seq), (uint32_t)p.max_block_id);
        have_ids = true;
      }
    }
    if (!have_ids) ids = wa.fetch_ids(table_of(cur.seq), cur.c_lo + tw, col_max);
    ids1 = wa.fetch_ids(table_of(cur.seq), cur.c_lo + tw + NT, col_max);
    wa.load_q(cur.seq, cur.kvh);
    wb.load_q(cur.seq, cur.kvh);
    wa.issue_k(R0, cur.kvh, cur.c_lo + tw, ids);
    wa.issue_v(R0, cur.kvh, cur.c_lo + tw, ids);
    ts0 = wa.fetch_scales(ids, cur.kvh, cur_a);
  }
  uint32_t sink_a = wa.load_sink(cur.kvh, tw == 0 && cur.part0 == 0), sink_b = wb.load_sink(cur.kvh, tw == 0 && cur.part0 == 0);
  Item prev = cur;  // the item whose merge is still owed (from the second item on)
  float prev_out_mul = 1.f;

  while (true) {
    Item nxt;
    const bool has_next = item_at(n + 1, nxt);
    int next_m = 0;
    if (has_next) {
      next_m = count_of(nxt);
      nxt_a = wa.fetch_item_ext(nxt.kvh, table_of(nxt.seq));
      nxt_b = wb.fetch_item_ext(nxt.kvh, table_of(nxt.seq));
    }
    const bool next_armed = next_m > 0;
    Ids nxt_ids = {}, nxt_ids1 = {};
    if (next_armed) {
      nxt_ids = wa.fetch_ids(table_of(nxt.seq), nxt.c_lo + tw, col_max);
      nxt_ids1 = wa.fetch_ids(table_of(nxt.seq), nxt.c_lo + tw + NT, col_max);
    }
    wa.reset(sink_a);
    wb.reset(sink_b);
    wa.set_item(cur_a, cur.ctx);
    wb.set_item(cur_b, cur.ctx);
    uint32_t next_a = W::kNoSink, next_b = W::kNoSink;
    if (has_next && !next_armed) {  // the sink goes with the item whether or not wavefront 0 has a chunk of it
      next_a = wa.load_sink(nxt.kvh, tw == 0 && nxt.part0 == 0);
      next_b = wb.load_sink(nxt.kvh, tw == 0 && nxt.part0 == 0);
    }
    // What the next item needs beyond K and V, once the last scores of this one are out.
    auto request_next_item = [&]() __attribute__((always_inline)) {
      wa.load_q(nxt.seq, nxt.kvh);
      wb.load_q(nxt.seq, nxt.kvh);
      next_a = wa.load_sink(nxt.kvh, tw == 0 && nxt.part0 == 0);
      next_b = wb.load_sink(nxt.kvh, tw == 0 && nxt.part0 == 0);
    };
    TileScales nts = {};
    bool owed = n > 0;  // finish(n - 1) still to do
    if (m > 0) {
      const int32_t *table = table_of(cur.seq);
      const int c0 = cur.c_lo + tw;  // chunk j of the wavefront is chunk c0 + j * NT of the item
      Scores sa, sb;
      Ids ids_a = {}, ids_b = {};  // ids of the chunks R0 and R1 take next
      int j = 0;
      if (m >= 4) {
        // The second chunk: K now; its V loads go out between the MFMAs of the first chunk's scores.
        int64_t vp0[TPC], vp1[TPC];  // where the V loads that R0 / R1 still wait for read from
        if (!k1_ready) wa.issue_k(R1, cur.kvh, c0 + NT, ids1);
#pragma unroll
        for (int t = 0; t < TPC; ++t) vp1[t] = wa.v_tile_at(cur.kvh, c0 + NT, t, ids1);
        ts1 = wa.fetch_scales(ids1, cur.kvh, cur_a);
        ids_a = wa.fetch_ids(table, c0 + 2 * NT, col_max);
        ids_b = wa.fetch_ids(table, c0 + 3 * NT, col_max);
        // One chunk: X holds chunk cx; the chunk two further on takes X over.  A wavefront that has
        // to wait at a load (the memory pipeline is full most of the time) computes nothing
        // meanwhile and there is no second wavefront on its SIMD, so the loads go out one at a
        // time between pieces of arithmetic: the V loads the OTHER set still waits for between
        // the MFMAs of the scores, the K loads of X's next chunk along softmax and P.V.
        auto steady = [&](Chunk &X, TileScales &tsx, int64_t (&vpx)[TPC], Chunk &Y, const int64_t (&vpy)[TPC], int cx,
                          Ids &ids) __attribute__((always_inline)) {
          constexpr int NS = W::KSTEPS * TPC, NV = 4 * TPC, NK = W::KL * TPC;
          W::qk_two(wa, wb, X, sa, sb, [&](int slot) __attribute__((always_inline)) {
#pragma unroll
            for (int v = slot * NV / NS; v < (slot + 1) * NV / NS; ++v) {
              __builtin_amdgcn_sched_barrier(0);
              wa.load_v_one(Y, v / 4, v % 4, vpy[v / 4]);
              __builtin_amdgcn_sched_barrier(0);
            }
          });
          int64_t kp[TPC];
#pragma unroll
          for (int t = 0; t < TPC; ++t) {
            kp[t] = wa.k_tile_at(cur.kvh, cx + 2 * NT, t, ids);
            vpx[t] = wa.v_tile_at(cur.kvh, cx + 2 * NT, t, ids);
          }
          nts = wa.fetch_scales(ids, cur.kvh, cur_a);
          ids = wa.fetch_ids(table, cx + 4 * NT, col_max);
          auto k_loads = [&](int part) __attribute__((always_inline)) {  // quarter `part` of the NK loads
#pragma unroll
            for (int k = part * NK / 4; k < (part + 1) * NK / 4; ++k) {
              __builtin_amdgcn_sched_barrier(0);
              wa.load_k_one(X, k / W::KL, k % W::KL, kp[k / W::KL]);
              __builtin_amdgcn_sched_barrier(0);
            }
          };
          k_loads(0);
          const auto pa = wa.template soft<false, true, true>(X, sa, cx, cur.tok_end, &tsx);
          k_loads(1);
          const auto pb = wb.template soft<false, true, true>(X, sb, cx, cur.tok_end, &tsx);
          k_loads(2);
          W::pv_two(wa, wb, X, pa, pb, [&](int slot) __attribute__((always_inline)) {
            if (slot == W::NP2 * W::NDT / 2 - 1) k_loads(3);
          });
          tsx = nts;
        };
        // Everything requested so far has to arrive before the loop is entered: most of it was
        // requested a step or more ago, and what the loop then waits for is decided by its own
        // loads alone, not by the worst of the paths that lead here (on some of which the
        // requests above were skipped).
        __builtin_amdgcn_s_waitcnt(kWaitVmcnt0);
        // steady: chunk j in R0 and j+1 in R1 are computed, chunks j+2 and j+3 requested
        while (j + 3 < m) {
          steady(R0, ts0, vp0, R1, vp1, c0 + j * NT, ids_a);
          if (owed) {  // a chunk into the item, the next requests on their way: the merge owed to the item before
            finish(n - 1, prev, prev_out_mul);
            owed = false;
          }
          steady(R1, ts1, vp1, R0, vp0, c0 + (j + 1) * NT, ids_b);
          j += 2;
        }
        // the V loads R1 still waits for
#pragma unroll
        for (int v = 0; v < 4 * TPC; ++v) wa.load_v_one(R1, v / 4, v % 4, vp1[v / 4]);
      } else if (m >= 2) {
        if (!k1_ready) wa.issue_k(R1, cur.kvh, c0 + NT, ids1);
        wa.issue_v(R1, cur.kvh, c0 + NT, ids1);
        ts1 = wa.fetch_scales(ids1, cur.kvh, cur_a);
        if (m == 3) ids_a = wa.fetch_ids(table, c0 + 2 * NT, col_max);
      }
      // The one to three chunks that end the item: j in R0, j+1 in R1, j+2 on its way into R0 or
      // requested now.  The last of these steps that uses R0 requests the next item's first chunk,
      // the step that uses R1 the K half of its second.
      k1_ready = false;
      const int rem = m - j;
      const int ca = c0 + j * NT;
      {
        W::qk_two(wa, wb, R0, sa, sb);
        if (rem == 3) {
          wa.issue_k(R0, cur.kvh, ca + 2 * NT, ids_a);
          nts = wa.fetch_scales(ids_a, cur.kvh, cur_a);
        } else if (next_armed) {
          if (rem == 1) request_next_item();
          wa.issue_k(R0, nxt.kvh, nxt.c_lo + tw, nxt_ids);
          nts = wa.fetch_scales(nxt_ids, nxt.kvh, nxt_a);
        }
        const auto pa = wa.template soft<true, true, true>(R0, sa, ca, cur.tok_end, &ts0);
        const auto pb = wb.template soft<true, true, true>(R0, sb, ca, cur.tok_end, &ts0);
        W::pv_two(wa, wb, R0, pa, pb);
        if (rem == 3) {
          wa.issue_v(R0, cur.kvh, ca + 2 * NT, ids_a);
        } else if (next_armed) {
          wa.issue_v(R0, nxt.kvh, nxt.c_lo + tw, nxt_ids);
        }
        ts0 = nts;
      }
      if (rem >= 2) {
        W::qk_two(wa, wb, R1, sa, sb);
        if (rem == 2 && next_armed) request_next_item();
        if (next_m >= 2) {
          wa.issue_k(R1, nxt.kvh, nxt.c_lo + tw + NT, nxt_ids1);
          k1_ready = true;
        }
        const auto pa = wa.template soft<true, true, true>(R1, sa, ca + NT, cur.tok_end, &ts1);
        const auto pb = wb.template soft<true, true, true>(R1, sb, ca + NT, cur.tok_end, &ts1);
        W::pv_two(wa, wb, R1, pa, pb);
      }
      if (rem == 3) {
        W::qk_two(wa, wb, R0, sa, sb);
        if (next_armed) {
          request_next_item();
          wa.issue_k(R0, nxt.kvh, nxt.c_lo + tw, nxt_ids);
          nts = wa.fetch_scales(nxt_ids, nxt.kvh, nxt_a);
        }
        const auto pa = wa.template soft<true, true, true>(R0, sa, ca + 2 * NT, cur.tok_end, &ts0);
        const auto pb = wb.template soft<true, true, true>(R0, sb, ca + 2 * NT, cur.tok_end, &ts0);
        W::pv_two(wa, wb, R0, pa, pb);
        if (next_armed) wa.issue_v(R0, nxt.kvh, nxt.c_lo + tw, nxt_ids);
        ts0 = nts;
      }
    } else if (next_armed) {  // nothing to do in `cur`, but the next item starts here
      k1_ready = false;
      request_next_item();
      wa.issue_k(R0, nxt.kvh, nxt.c_lo + tw, nxt_ids);
      wa.issue_v(R0, nxt.kvh, nxt.c_lo + tw, nxt_ids);
      ts0 = wa.fetch_scales(nxt_ids, nxt.kvh, nxt_a);
    }
    if (owed) finish(n - 1, prev, prev_out_mul);
    publish(n);

    if (!has_next) break;
    prev = cur;
    prev_out_mul = cur_a.out_mul;
    cur = nxt;
    m = next_m;
    ids1 = nxt_ids1;
    sink_a = next_a;
    sink_b = next_b;
    cur_a = nxt_a;
    cur_b = nxt_b;
    ++n;
  }
  finish(n, cur, cur_a.out_mul);
}

}  // namespace fa
