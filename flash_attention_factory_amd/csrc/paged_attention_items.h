// The work items of a persistent attention kernel, as every wavefront works them out for itself
// from the context lengths: which (sequence, kv head[, segment of partitions]) is the n-th item
// of this work-group.  Two lists, one interface:
//
//   LoopItems     loop path: one item per (sequence, kv head), sequences longest first.
//   SegmentItems  split path: one item per (sequence, kv head, segment of m partitions), all
//                 full segments first, then the sequences' last, shorter segments by length
//                 (what paged_attention_segment_kernel.h deals, and what the reduce kernel
//                 expects: one partial per segment, in the slot of its first partition).
//
// Both deal the sorted list to the work-groups in snake order: work-group j takes positions
// j, 2G-1-j, 2G+j, ... so that a handful of items per work-group still add up evenly.
#pragma once

#include "paged_attention_segment_policy.h"
#include "paged_attention_wave.h"

namespace fa {

// chunks c_lo .. c_end-1 of CT tokens; tok_end: where the item's keys end (the context's end, or
// the segment's); part0: slot of the item's partial (split path); ctx: the sequence's length
struct WorkItem { int seq, kvh, ctx, c_lo, c_end, tok_end, part0; };

__device__ __forceinline__ int snake_position(int nth, int groups, int group) {
  return nth * groups + ((nth & 1) ? groups - 1 - group : group);
}

template <int TPC>
struct LoopItems {
  static constexpr int kMaxSeqs = 128;
  int len0 = -1, len1 = -1, key0, key1, rank0 = 0, rank1 = 0;
  int sid0[TPC] = {}, sid1[TPC] = {};
  int S, Hk;

  // Lane holds sequences lane and lane + 64.  Requested together with the lengths, so that the
  // first K/V loads depend on one round trip to memory, not two: for EVERY sequence the block ids
  // of chunk `wave`, the one this wavefront starts an item with (first_id).
  // heads_per_item: adjacent kv heads that one work-group takes together (its wavefronts in teams)
  __device__ __forceinline__ void build(const PagedAttnParams &p, int lane, int wave, int groups, int chunk_tokens,
                                        int heads_per_item = 1) {
    S = p.num_seqs;
    Hk = p.num_kv_heads / heads_per_item;
    const int max_ctx = p.max_blocks_per_seq << p.block_shift;
    const int col_max = p.max_blocks_per_seq - 1;
    if (lane < S) {
      len0 = max(0, min(p.context_lens[lane], max_ctx));
      const int32_t *row = p.block_tables + (int64_t)lane * p.max_blocks_per_seq;
#pragma unroll
      for (int t = 0; t < TPC; ++t) sid0[t] = row[min((wave * chunk_tokens + t * kTileTokens) >> p.block_shift, col_max)];
    }
    if (S > 64 && lane + 64 < S) {
      len1 = max(0, min(p.context_lens[lane + 64], max_ctx));
      const int32_t *row = p.block_tables + (int64_t)(lane + 64) * p.max_blocks_per_seq;
#pragma unroll
      for (int t = 0; t < TPC; ++t) sid1[t] = row[min((wave * chunk_tokens + t * kTileTokens) >> p.block_shift, col_max)];
    }
    // Sort key: length, then lower sequence number first; distinct for distinct sequences
    // (lengths stay below 2^24, the launcher sees to that).  Lanes without a sequence: -1.
    key0 = len0 < 0 ? -1 : (len0 << 7) | (127 - lane);
    key1 = len1 < 0 ? -1 : (len1 << 7) | (63 - lane);
    // No more items than work-groups: nobody takes a second one, so any order deals them as well
    // as the sorted one -- skip the ranking (a third of a microsecond of a launch that then lasts
    // a handful).
    if (S * Hk <= groups) {
      rank0 = lane;
      rank1 = lane + 64;
      return;
    }
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
  }
  // n-th item of work-group `group`; false: the work-group has no such item (and none after it)
  __device__ __forceinline__ bool at(int n, int groups, int group, int chunk_tokens, WorkItem &it) const {
    const int pos = snake_position(n, groups, group);
    if (pos >= S * Hk) return false;
    const int rho = __builtin_amdgcn_readfirstlane(pos / Hk);
    it.kvh = pos - rho * Hk;
    const unsigned long long b0 = __ballot(key0 >= 0 && rank0 == rho);
    const unsigned long long b1 = __ballot(key1 >= 0 && rank1 == rho);
    const int s = b0 ? __builtin_ctzll(b0) : 64 + __builtin_ctzll(b1);
    it.seq = __builtin_amdgcn_readfirstlane(s);
    it.ctx = s < 64 ? __builtin_amdgcn_readlane(len0, s) : __builtin_amdgcn_readlane(len1, s - 64);
    it.tok_end = it.ctx;
    it.c_lo = 0;
    it.c_end = (it.ctx + chunk_tokens - 1) / chunk_tokens;
    it.part0 = 0;
    return it.ctx > 0;  // sorted: nothing but empty sequences follows an empty one
  }
  // block id of tile t of chunk `wave` of a sequence, as requested with the lengths
  __device__ __forceinline__ int first_id(int t, int seq) const {
    return seq < 64 ? __builtin_amdgcn_readlane(sid0[t], seq) : __builtin_amdgcn_readlane(sid1[t], seq - 64);
  }
};

struct SegmentItems {
  static constexpr int NQ = kSegmentMaxSeqs / 64;
  int ctxv[NQ], parts[NQ], incl[NQ], fullc[NQ], key[NQ], rank[NQ];
  int S, Hk, m, seg_tokens, full_total, total_items, lane;

  // Lane holds sequences lane, lane + 64, ...  m, the partitions per segment, follows from the
  // batch, the number of work-groups and the compute units they share (partitions_per_segment).
  // heads_per_item: adjacent kv heads that one work-group takes together (its wavefronts in teams);
  // item_row_bytes: bytes of one token's K row (as of its V row) of an item
  __device__ __forceinline__ void build(const PagedAttnParams &p, int lane_, int groups, int heads_per_item,
                                        int item_row_bytes) {
    lane = lane_;
    S = p.num_seqs;
    Hk = p.num_kv_heads / heads_per_item;
    const int max_ctx = p.max_blocks_per_seq << p.block_shift;
    const int total_parts = count_partitions<NQ>(p.context_lens, S, max_ctx, p.partition_size, p.max_num_partitions, lane, ctxv, parts);
    m = p.segment_force > 0 ? min(p.segment_force, kSegmentMaxPartitions)
                            : partitions_per_segment<NQ>(ctxv, parts, total_parts, S, p.partition_size, Hk, groups,
                                                         p.compute_units, p.kv_rows_apart != 0,
                                                         2 * p.partition_size * item_row_bytes);
    seg_tokens = m * p.partition_size;
    int running = 0, tails = 0;
#pragma unroll
    for (int j = 0; j < NQ; ++j) {
      const int cut = min(ctxv[j], parts[j] * p.partition_size);  // what the scratch arrays can hold
      ctxv[j] = cut;
      fullc[j] = cut / seg_tokens;
      const int rem = cut - fullc[j] * seg_tokens;
      // sort key of the last segment: length, then lower sequence number first; -1: none
      key[j] = rem > 0 ? (rem << 8) | (255 - (lane + 64 * j)) : -1;
      rank[j] = 0;
      int x = fullc[j];
      if (j * 64 < S) {
        tails += __builtin_popcountll(__ballot(rem > 0));
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
          const int y = __shfl_up(x, o);
          if (lane >= o) x += y;
        }
      }
      incl[j] = x + running;
      running = __builtin_amdgcn_readlane(incl[j], 63);
    }
    full_total = running;
    total_items = (full_total + tails) * Hk;
    // rank of every last segment among the last segments (how many are longer)
#pragma unroll
    for (int js = 0; js < NQ; ++js) {
      if (js * 64 < S) {
        for (int u0 = 0; u0 < min(S - js * 64, 64); u0 += 8) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int ku = __builtin_amdgcn_readlane(key[js], u0 + e);
#pragma unroll
            for (int jd = 0; jd < NQ; ++jd) rank[jd] += ku > key[jd];
          }
        }
      }
    }
  }
  // position in the sorted list -> (sequence, segment, kv head), kv head fastest
  __device__ __forceinline__ bool at(int n, int groups, int group, int chunk_tokens, WorkItem &it) const {
    const int pos = snake_position(n, groups, group);
    if (pos >= total_items) return false;
    const int q = __builtin_amdgcn_readfirstlane(pos / Hk);
    it.kvh = pos - q * Hk;
    int s = 0;
    const bool full = q < full_total;
    if (full) {
#pragma unroll
      for (int j = 0; j < NQ; ++j)
        if (j * 64 < S) s += __builtin_popcountll(__ballot(lane + 64 * j < S && incl[j] <= q));
    } else {
      const int rho = q - full_total;
#pragma unroll
      for (int j = 0; j < NQ; ++j)
        if (j * 64 < S) {
          const unsigned long long hit = __ballot(key[j] >= 0 && rank[j] == rho);
          if (hit) s = 64 * j + __builtin_ctzll(hit);
        }
    }
    s = min(s, S - 1);
    int inc_s = 0, full_s = 0, ctx_s = 0;
#pragma unroll
    for (int j = 0; j < NQ; ++j)
      if ((s >> 6) == j) {
        inc_s = __builtin_amdgcn_readlane(incl[j], s & 63);
        full_s = __builtin_amdgcn_readlane(fullc[j], s & 63);
        ctx_s = __builtin_amdgcn_readlane(ctxv[j], s & 63);
      }
    it.seq = __builtin_amdgcn_readfirstlane(s);
    const int seg = full ? q - (inc_s - full_s) : full_s;
    it.part0 = seg * m;
    const int tok_begin = seg * seg_tokens;
    it.tok_end = full ? tok_begin + seg_tokens : ctx_s;
    it.c_lo = tok_begin / chunk_tokens;
    it.c_end = (it.tok_end + chunk_tokens - 1) / chunk_tokens;
    it.ctx = ctx_s;
    return true;
  }
};

}  // namespace fa
