// Split-context attention kernel, persistent form.
//
// Same results as the grid form (paged_attention_kernel.h with PART = true; upstream
// paged_attention_kernel_v2.hpp:572-587), different scheduling.  The grid form launches
// one work-group per (kv head, partition slot, sequence): with ragged lengths most slots
// are empty, and every live partition pays a dependent "length -> block ids -> K/V"
// start-up during which its wavefront has nothing in flight.  Here the launch holds just
// as many single-wavefront work-groups as the GPU keeps resident, and each of them walks
// the list of LIVE (sequence, partition, kv head) items k, k + gridDim.x, ... :
//   * the item list is built in registers from context_lens (a prefix sum over
//     sequences, one pass per wavefront) -- empty slots are never visited;
//   * the K/V loads of the next item's first chunk are issued before the current item's
//     last chunk is computed, so the stream never drains between items.
// Built for up to 256 sequences; larger batches use the grid form.
#pragma once

#include "paged_attention_kernel.h"

namespace fa {

constexpr int kPersistentMaxSeqs = 256;

template <int D, typename QT, bool KV8, int OCC, int TPC, int ORDER>
__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(OCC)))
paged_attn_split_persistent_kernel(const PagedAttnParams p) {
  using W = WaveAttn<D, QT, KV8, TPC, Pipeline<KV8>::stream_loads_split>;
  using Chunk = typename W::Chunk;
  using Ids = typename W::Ids;
  constexpr int CT = W::CT;
  constexpr int NQ = kPersistentMaxSeqs / 64;  // sequences per lane

  const int lane = threadIdx.x;
  const int S = p.num_seqs;
  const int Hk = p.num_kv_heads;
  const int max_ctx = p.max_blocks_per_seq << p.block_shift;

  // ---- item list: lane holds sequences lane, lane+64, ... ----------------------------
  int ctxv[NQ];  // context length, cut to what the block table holds
  int incl[NQ];  // partitions of all sequences up to and including this one
  int cnt[NQ];
  int running = 0;
#pragma unroll
  for (int j = 0; j < NQ; ++j) {
    const int s = lane + 64 * j;
    int c = 0;
    if (j * 64 < S) {  // wave-uniform
      if (s < S) c = max(0, min(p.context_lens[s], max_ctx));
    }
    ctxv[j] = c;
    cnt[j] = min((c + p.partition_size - 1) / p.partition_size, p.max_num_partitions);  // per lane
  }
#pragma unroll
  for (int j = 0; j < NQ; ++j) {
    int x = cnt[j];
    if (j * 64 < S) {
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int y = __shfl_up(x, o);
        if (lane >= o) x += y;
      }
    }
    incl[j] = x + running;
    running = __builtin_amdgcn_readlane(incl[j], 63);
  }
  const int total_items = running * Hk;

  // item k -> (sequence, kv head, partition).
  //   ORDER 0: kv head fastest, then partition, then sequence.
  //   ORDER 1: partition fastest, then kv head, then sequence -- neighbouring items write
  //            neighbouring tmp_out rows (the partitions of one head are contiguous there).
  struct Item { int seq, kvh, part, tok_end, c_begin, c_end; };
  auto decode = [&](int k) -> Item {
    Item it;
    // integer division runs on the vector unit: tell the compiler the results are uniform
    const int q = ORDER == 0 ? __builtin_amdgcn_readfirstlane(k / Hk) : k;
    int s = 0;
#pragma unroll
    for (int j = 0; j < NQ; ++j)
      if (j * 64 < S)
        s += __builtin_popcountll(
            __ballot(lane + 64 * j < S && (ORDER == 0 ? incl[j] : incl[j] * Hk) <= q));
    s = min(s, S - 1);
    int inc_s = 0, cnt_s = 0, ctx_s = 0;
#pragma unroll
    for (int j = 0; j < NQ; ++j)
      if ((s >> 6) == j) {
        inc_s = __builtin_amdgcn_readlane(incl[j], s & 63);
        cnt_s = __builtin_amdgcn_readlane(cnt[j], s & 63);
        ctx_s = __builtin_amdgcn_readlane(ctxv[j], s & 63);
      }
    it.seq = __builtin_amdgcn_readfirstlane(s);
    if constexpr (ORDER == 0) {
      it.kvh = k - q * Hk;
      it.part = q - (inc_s - cnt_s);
    } else {
      const int rem = k - (inc_s - cnt_s) * Hk;
      it.kvh = __builtin_amdgcn_readfirstlane(rem / max(cnt_s, 1));
      it.part = rem - it.kvh * cnt_s;
    }
    const int tok_begin = it.part * p.partition_size;
    it.tok_end = min(ctx_s, tok_begin + p.partition_size);
    it.c_begin = tok_begin / CT;
    it.c_end = (it.tok_end + CT - 1) / CT;
    return it;
  };

  // Which items this work-group walks: k_first, k_first + k_stride, ... below k_end.
  //   ORDER 0: all work-groups interleave over the whole list.
  //   ORDER 1: work-groups land on the 8 XCDs round-robin (id mod 8), each XCD with its own
  //            L2; give every XCD one contiguous eighth of the list, interleaved among its
  //            own work-groups, so rows that are neighbours in memory meet in one L2.
  int k_first = blockIdx.x, k_stride = gridDim.x, k_end = total_items;
  if constexpr (ORDER == 1) {
    const int xcd = blockIdx.x & 7;
    const int per_xcd = (total_items + 7) / 8;
    k_stride = ((int)gridDim.x + 7 - xcd) / 8;
    k_first = xcd * per_xcd + ((int)blockIdx.x >> 3);
    k_end = min(total_items, (xcd + 1) * per_xcd);
  }

  int k = k_first;
  if (k >= k_end) return;

  W wa(p, lane);
  const int col_max = p.max_blocks_per_seq - 1;  // ids are clamped into the pool or the
                                                 // launcher does not pick this kernel
  Item cur = decode(k);
  const int32_t *table = p.block_tables + (int64_t)cur.seq * p.max_blocks_per_seq;
  int ci = cur.c_begin;
  Ids ids = wa.fetch_ids(table, ci, col_max);
  wa.load_q(cur.seq, cur.kvh);
  wa.reset(wa.load_sink(cur.kvh, cur.part == 0));
  Chunk R;
  wa.issue_k(R, cur.kvh, ci, ids);
  wa.issue_v(R, cur.kvh, ci, ids);

  // (nxt, nci): the chunk after (cur, ci); its ids are fetched one step ahead
  auto advance = [&](const Item &it, int c, int kk, Item &nit, int &nc, int &nk) -> bool {
    if (c + 1 < it.c_end) {
      nit = it;
      nc = c + 1;
      nk = kk;
      return true;
    }
    nk = kk + k_stride;
    if (nk >= k_end) return false;
    nit = decode(nk);
    nc = nit.c_begin;
    return true;
  };

  Item nxt;
  int nci, nk;
  bool more = advance(cur, ci, k, nxt, nci, nk);
  Ids nids = ids;
  if (more) nids = wa.fetch_ids(p.block_tables + (int64_t)nxt.seq * p.max_blocks_per_seq, nci, col_max);

  while (more) {
    // ids of the chunk after next, requested now so they are there one step later
    Item nn;
    int nnc, nnk;
    const bool more2 = advance(nxt, nci, nk, nn, nnc, nnk);
    Ids nnids = nids;
    if (more2) nnids = wa.fetch_ids(p.block_tables + (int64_t)nn.seq * p.max_blocks_per_seq, nnc, col_max);

    // Order matters for the wait counters: everything the next item needs (Q, sink) is
    // requested BEFORE the K/V loads of its first chunk, so waiting for K never has to
    // wait for anything younger than the V loads.
    const bool item_done = nk != k;
    const auto s = wa.qk(R);
    uint32_t next_sink = W::kNoSink;
    if (item_done) {  // Q registers are free once the last score MFMAs of the item are out
      wa.load_q(nxt.seq, nxt.kvh);
      next_sink = wa.load_sink(nxt.kvh, nxt.part == 0);
    }
    wa.issue_k(R, nxt.kvh, nci, nids);
    const auto pb = wa.template soft<true>(R, s, ci, cur.tok_end);
    wa.pv(R, pb);
    wa.issue_v(R, nxt.kvh, nci, nids);
    if (item_done) {  // store the finished item; the next one's loads are already in flight
      merge_and_store<true, 1>(wa, p, lane, 0, cur.seq, cur.kvh, cur.part);
      wa.reset(next_sink);
    }
    cur = nxt;
    ci = nci;
    k = nk;
    nxt = nn;
    nci = nnc;
    nk = nnk;
    nids = nnids;
    more = more2;
  }
  const auto s = wa.qk(R);
  wa.pv(R, wa.template soft<true>(R, s, ci, cur.tok_end));
  merge_and_store<true, 1>(wa, p, lane, 0, cur.seq, cur.kvh, cur.part);
}

}  // namespace fa
