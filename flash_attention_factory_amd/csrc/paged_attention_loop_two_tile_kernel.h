// Single-pass ("loop") attention kernel, persistent form, for query blocks of two column tiles.
//
// The extended persistent loop kernel (paged_attention_loop_persistent_kernel.h) fills the 16
// MFMA columns of a kv head with (query token, head) pairs.  A launch of up to 32 such pairs --
// a speculative-decoding step of 4 tokens over a group of 8 heads, 32 tokens of one head -- needs
// two column tiles.  Here BOTH tiles live in the registers of the same wavefront: one chunk of K
// and V is loaded once, every operand is built once and feeds the MFMAs of both tiles
// (WaveAttn::qk_two, pv_two), each tile keeps its own queries, softmax state and accumulators,
// masks by its own columns' positions and is merged and stored for itself.  K and V cross HBM
// and the caches exactly once per launch, and all four wavefronts of a work-group interleave an
// item's chunks as in the one-tile kernel.  The price is registers (two sets of queries and
// accumulators: one work-group per compute unit) and twice the merge buffers in LDS.
//
// Item order, deferred merge, prefetch across items: as in the one-tile kernel.
#pragma once

#include "paged_attention_loop_persistent_kernel.h"

namespace fa {

template <int D, typename QT, int KVF, int NWG, int TPC, bool KROW = true>
__global__ void __launch_bounds__(NWG * 64) __attribute__((amdgpu_waves_per_eu(1)))
paged_attn_loop_two_tile_kernel(const PagedAttnParams p) {
  constexpr int NW = NWG;  // wavefronts that share an item's chunks and merge
  using W = WaveAttn<D, QT, KVF, TPC, Pipeline<(KVF != 0)>::stream_loads_loop, true, KROW>;
  using Chunk = typename W::Chunk;
  using Ids = typename W::Ids;
  using ItemExt = typename W::ItemExt;
  using TileScales = typename W::TileScales;
  using Scores = typename W::Scores;
  constexpr int CT = W::CT;
  constexpr int NR = W::NR;
  constexpr int NDT = W::NDT;
  constexpr int SL = NR / NW;
  static_assert(NW > 1 && NR % NW == 0 && SL >= 2, "merge slices the output across wavefronts");

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int S = p.num_seqs;
  const int Hk = p.num_kv_heads;
  const int T = S * Hk;
  const int G = gridDim.x;
  const int wg = blockIdx.x;
  const int max_ctx = p.max_blocks_per_seq << p.block_shift;
  const int col_max = p.max_blocks_per_seq - 1;

  // ---- rank the sequences by length, longest first; lane holds sequences lane, lane+64 --
  // Requested together with the lengths, so that the first K/V loads depend on one round
  // trip to memory, not two: for EVERY sequence, the block ids of the chunk this wavefront
  // would start with.  Once the ranking has named the first item its ids are a lane away.
  int len0 = -1, len1 = -1;
  int sid0[TPC] = {}, sid1[TPC] = {};
  if (lane < S) {
    len0 = max(0, min(p.context_lens[lane], max_ctx));
    const int32_t *row = p.block_tables + (int64_t)lane * p.max_blocks_per_seq;
#pragma unroll
    for (int t = 0; t < TPC; ++t) sid0[t] = row[min((wave * CT + t * kTileTokens) >> p.block_shift, col_max)];
  }
  if (S > 64 && lane + 64 < S) {
    len1 = max(0, min(p.context_lens[lane + 64], max_ctx));
    const int32_t *row = p.block_tables + (int64_t)(lane + 64) * p.max_blocks_per_seq;
#pragma unroll
    for (int t = 0; t < TPC; ++t) sid1[t] = row[min((wave * CT + t * kTileTokens) >> p.block_shift, col_max)];
  }
  // Sort key: length, then lower sequence number first; distinct for distinct sequences
  // (lengths stay below 2^24, the launcher sees to that).  Lanes without a sequence: -1.
  const int key0 = len0 < 0 ? -1 : (len0 << 7) | (127 - lane);
  const int key1 = len1 < 0 ? -1 : (len1 << 7) | (63 - lane);
  int rank0 = 0, rank1 = 0;  // how many sequences come before this one
  // eight sequences per trip; lanes past the batch hold -1 and count for nothing
  for (int u0 = 0; u0 < min(S, 64); u0 += 8) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int ku = __builtin_amdgcn_readlane(key0, u0 + j);
      rank0 += ku > key0;
      rank1 += ku > key1;
    }
  }
  for (int u0 = 0; u0 < S - 64; u0 += 8) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int ku = __builtin_amdgcn_readlane(key1, u0 + j);
      rank0 += ku > key0;
      rank1 += ku > key1;
    }
  }
  struct Item { int seq, kvh, ctx, c_end, c_lo; };  // c_lo: first chunk to read (0 unless EXT)
  // n-th item of this work-group: position n*G + j on even n, n*G + G-1-j on odd n
  auto item_at = [&](int n, Item &it) -> bool {
    const int pos = n * G + ((n & 1) ? G - 1 - wg : wg);
    if (pos >= T) return false;
    const int rho = __builtin_amdgcn_readfirstlane(pos / Hk);
    it.kvh = pos - rho * Hk;
    const unsigned long long b0 = __ballot(key0 >= 0 && rank0 == rho);
    const unsigned long long b1 = __ballot(key1 >= 0 && rank1 == rho);
    const int s = b0 ? __builtin_ctzll(b0) : 64 + __builtin_ctzll(b1);
    it.seq = __builtin_amdgcn_readfirstlane(s);
    it.ctx = s < 64 ? __builtin_amdgcn_readlane(len0, s) : __builtin_amdgcn_readlane(len1, s - 64);
    it.c_end = (it.ctx + CT - 1) / CT;
    it.c_lo = 0;
    return it.ctx > 0;  // sorted: nothing but empty sequences follows an empty one
  };

  // Partial states of two items in flight, per column tile: item n goes to buffer n & 1.
  __shared__ float sm_m[2][2][NW][16];
  __shared__ float sm_l[2][2][NW][16];
  __shared__ float sm_acc[2][2][NW][NR][64];
  __shared__ int sm_arrived[2];  // wavefronts that have published (both tiles) into the buffer, ever

  W wa(p, lane, 0), wb(p, lane, 1);  // the two column tiles
  const int r = wa.r, i = wa.i;
  Chunk R;

  int n = 0;
  Item cur;
  if (!item_at(0, cur)) return;  // the same for every wavefront of the work-group
  cur.c_lo = wa.first_visible_chunk(cur.ctx, 0);  // the launch's earliest query token decides: the same for both tiles
  if (threadIdx.x < 2) sm_arrived[threadIdx.x] = 0;
  __syncthreads();  // the only barrier: wavefronts meet through the counters from here on

  // A wavefront's states of item n go to LDS and the wavefront moves on; nobody waits here.
  auto publish_tile = [&](W &w, int tile, int b) {
    w.l = rows_sum(w.l);
    if (r == 0) {
      sm_m[tile][b][wave][i] = w.m;
      sm_l[tile][b][wave][i] = w.l;
    }
#pragma unroll
    for (int k = 0; k < NR; ++k) sm_acc[tile][b][wave][k][lane] = w.acc_at(k);
  };
  auto publish = [&](int item) {
    const int b = item & 1;
    publish_tile(wa, 0, b);
    publish_tile(wb, 1, b);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    if (lane == 0) __hip_atomic_fetch_add(&sm_arrived[b], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  };
  // Merge the NW published states of one tile of an item, normalise, store this wavefront's slice.
  auto finish_tile = [&](W &w, int tile, int b, int seq, int kvh, float out_mul) {
    float M = -INFINITY;
#pragma unroll
    for (int v = 0; v < NW; ++v) M = fmaxf(M, sm_m[tile][b][v][i]);
    float f[NW];
    float L = 0.f;
#pragma unroll
    for (int v = 0; v < NW; ++v) {
      const float mv = sm_m[tile][b][v][i];
      f[v] = (mv == -INFINITY) ? 0.f : fast_exp2(mv - M);  // a wavefront without chunks
      L += f[v] * sm_l[tile][b][v][i];
    }
    float o[SL];
#pragma unroll
    for (int k = 0; k < SL; ++k) {
      float a = 0.f;
#pragma unroll
      for (int v = 0; v < NW; ++v) a += f[v] * sm_acc[tile][b][v][wave * SL + k][lane];
      o[k] = a;
    }
    if (w.col_valid) {
      const int head = kvh * p.group + w.col_g;
      const int d0 = 4 * r * NDT + wave * SL;
      const int64_t row = (int64_t)seq * p.query_len + w.col_q;
      const float inv = L > 0.f ? out_mul / L : 0.f;  // L = 0: the query token sees no key
      W::template store_q<SL>(reinterpret_cast<char *>(p.out) + ((row * p.num_heads + head) * D + d0) * 2, o, inv);
    }
  };
  // Called one chunk into the following item (or after the last item): see the one-tile kernel for
  // why the wait always ends and why a buffer is never overwritten while somebody still reads it.
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
    if (!arrived && lane == 0) __hip_atomic_store(p.status, kStatusSpinLimit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    finish_tile(wa, 0, b, seq, kvh, out_mul);
    finish_tile(wb, 1, b, seq, kvh, out_mul);
  };
  // one chunk of the current item through both tiles
  auto scores_of = [&](Scores &sa, Scores &sb) { W::qk_two(wa, wb, R, sa, sb); };
  auto soft_pv = [&](auto tail, const Scores &sa, const Scores &sb, int ci, int ctx, const TileScales &ts) {
    const auto pa = wa.template soft<decltype(tail)::value, true>(R, sa, ci, ctx, &ts);
    const auto pb = wb.template soft<decltype(tail)::value, true>(R, sb, ci, ctx, &ts);
    W::pv_two(wa, wb, R, pa, pb);
  };
  auto table_of = [&](int seq) { return p.block_tables + (int64_t)seq * p.max_blocks_per_seq; };

  // first chunk of the first item
  bool armed = cur.c_lo + wave < cur.c_end;  // loads of this wavefront's first chunk of `cur` in flight
  ItemExt cur_a = wa.fetch_item_ext(cur.kvh, table_of(cur.seq)), cur_b = wb.fetch_item_ext(cur.kvh, table_of(cur.seq));
  ItemExt nxt_a = {}, nxt_b = {};
  TileScales ts = {}, nts = {}, nxt_ts = {};
  if (armed) {
    Ids ids;
#pragma unroll
    for (int t = 0; t < TPC; ++t) {
      const int raw = cur.seq < 64 ? __builtin_amdgcn_readlane(sid0[t], cur.seq)
                                   : __builtin_amdgcn_readlane(sid1[t], cur.seq - 64);
      ids.v[t] = min((uint32_t)raw, (uint32_t)p.max_block_id);
    }
    if (cur.c_lo != 0)  // the ids requested with the lengths are those of chunk `wave`
      ids = wa.fetch_ids(table_of(cur.seq), cur.c_lo + wave, col_max);
    wa.load_q(cur.seq, cur.kvh);
    wb.load_q(cur.seq, cur.kvh);
    wa.issue_k(R, cur.kvh, cur.c_lo + wave, ids);
    wa.issue_v(R, cur.kvh, cur.c_lo + wave, ids);
    ts = wa.fetch_scales(ids, cur.kvh, cur_a);
  }
  uint32_t sink_a = wa.load_sink(cur.kvh, wave == 0), sink_b = wb.load_sink(cur.kvh, wave == 0);
  Item prev = cur;  // the item whose merge is still owed (from the second item on)
  float prev_out_mul = 1.f;

  while (true) {
    Item nxt;
    const bool has_next = item_at(n + 1, nxt);
    if (has_next) {
      nxt.c_lo = wa.first_visible_chunk(nxt.ctx, 0);
      nxt_a = wa.fetch_item_ext(nxt.kvh, table_of(nxt.seq));
      nxt_b = wb.fetch_item_ext(nxt.kvh, table_of(nxt.seq));
    }
    const bool next_armed = has_next && nxt.c_lo + wave < nxt.c_end;
    Ids nxt_ids = {};
    if (next_armed) nxt_ids = wa.fetch_ids(table_of(nxt.seq), nxt.c_lo + wave, col_max);

    wa.reset(sink_a);
    wb.reset(sink_b);
    wa.set_item(cur_a, cur.ctx);
    wb.set_item(cur_b, cur.ctx);
    uint32_t next_a = W::kNoSink, next_b = W::kNoSink;
    if (has_next && !next_armed) {  // the sink goes with the item whether or not wavefront 0 has a chunk of it
      next_a = wa.load_sink(nxt.kvh, wave == 0);
      next_b = wb.load_sink(nxt.kvh, wave == 0);
    }
    bool owed = n > 0;
    if (armed) {
      const int32_t *table = table_of(cur.seq);
      int ci = cur.c_lo + wave;
      Ids nids = wa.fetch_ids(table, ci + NW, col_max);
      Scores sa, sb;
      bool first = true;
      while (ci + NW < cur.c_end) {  // the next chunk belongs to the same item
        const int cn = ci + NW;
        scores_of(sa, sb);
        wa.issue_k(R, cur.kvh, cn, nids);
        nts = wa.fetch_scales(nids, cur.kvh, cur_a);
        soft_pv(std::false_type{}, sa, sb, ci, cur.ctx, ts);
        wa.issue_v(R, cur.kvh, cn, nids);
        nids = wa.fetch_ids(table, cn + NW, col_max);
        ts = nts;
        ci = cn;
        if (first && owed) {  // one chunk into the item: the merge owed to the previous item
          finish(n - 1, prev.seq, prev.kvh, prev_out_mul);
          owed = false;
        }
        first = false;
      }
      // last chunk of this wavefront in `cur`: what goes out next belongs to `nxt`
      scores_of(sa, sb);
      if (next_armed) {
        wa.load_q(nxt.seq, nxt.kvh);  // Q registers are free once the last scores are out
        wb.load_q(nxt.seq, nxt.kvh);
        next_a = wa.load_sink(nxt.kvh, wave == 0);
        next_b = wb.load_sink(nxt.kvh, wave == 0);
        wa.issue_k(R, nxt.kvh, nxt.c_lo + wave, nxt_ids);
        nxt_ts = wa.fetch_scales(nxt_ids, nxt.kvh, nxt_a);
      }
      soft_pv(std::true_type{}, sa, sb, ci, cur.ctx, ts);
      if (next_armed) wa.issue_v(R, nxt.kvh, nxt.c_lo + wave, nxt_ids);
    } else if (next_armed) {  // nothing to do in `cur`, but the next item starts here
      wa.load_q(nxt.seq, nxt.kvh);
      wb.load_q(nxt.seq, nxt.kvh);
      next_a = wa.load_sink(nxt.kvh, wave == 0);
      next_b = wb.load_sink(nxt.kvh, wave == 0);
      wa.issue_k(R, nxt.kvh, nxt.c_lo + wave, nxt_ids);
      wa.issue_v(R, nxt.kvh, nxt.c_lo + wave, nxt_ids);
      nxt_ts = wa.fetch_scales(nxt_ids, nxt.kvh, nxt_a);
    }
    if (owed) finish(n - 1, prev.seq, prev.kvh, prev_out_mul);
    publish(n);

    if (!has_next) break;
    prev = cur;
    cur = nxt;
    armed = next_armed;
    sink_a = next_a;
    sink_b = next_b;
    prev_out_mul = cur_a.out_mul;
    cur_a = nxt_a;
    cur_b = nxt_b;
    ts = nxt_ts;
    ++n;
  }
  finish(n, cur.seq, cur.kvh, cur_a.out_mul);
}

}  // namespace fa
