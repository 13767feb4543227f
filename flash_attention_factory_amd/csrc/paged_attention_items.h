// The work items of a persistent attention kernel, as every wavefront works them out for itself
// from the context lengths: which (sequence, kv head[, segment of partitions]) is the n-th item
// of this work-group.  Two lists, one interface:
//
//   LoopItems     loop path: one item per (sequence, kv head), sequences longest first.
//   SegmentItems  split path, one item per piece of a (sequence, kv head) row.  Either segments of m
//                 partitions -- all full segments first, then the sequences' last, shorter
//                 segments by length -- or even shares: the rows' partitions laid end to end
//                 (sequences in order, kv heads within a sequence) and cut into one contiguous share
//                 per work-group (paged_attention_segment_policy.h).  One partial per piece, in the
//                 slot of its first partition.
//
// Both deal the sorted list to the work-groups in snake order: work-group j takes positions
// j, 2G-1-j, 2G+j, ... so that a handful of items per work-group still add up evenly.
#pragma once

#include "paged_attention_segment_policy.h"
#include "paged_attention_wave.h"

namespace fa {

// chunks c_lo .. c_end-1 of CT tokens; tok_end: where the item's keys end (the context's end, or
// the piece's); part0: slot of the item's partial and parts: partitions it covers (split path);
// ctx: the sequence's length
struct WorkItem { int seq, kvh, ctx, c_lo, c_end, tok_end, part0, parts; };

__device__ __forceinline__ int snake_position(int nth, int groups, int group) {
  return nth * groups + ((nth & 1) ? groups - 1 - group : group);
}

template <int TPC>
struct LoopItems {
  static constexpr int kMaxSeqs = 128;
  int len0 = -1, len1 = -1, key0, key1, rank0 = 0, rank1 = 0;
  int sid0[TPC] = {}, sid1[TPC] = {};
  int S, Hk;
  int head_shift = -1;  // stack_affine_shift of the pool

  // Lane holds sequences lane and lane + 64.  Requested together with the lengths, so that the
  // first K/V loads depend on one round trip to memory, not two: for EVERY sequence the block ids
  // of chunk `wave`, the one this wavefront starts an item with (first_id).
  // heads_per_item: adjacent kv heads that one work-group takes together (its wavefronts in teams)
  __device__ __forceinline__ void build(const PagedAttnParams &p, int lane, int wave, int groups, int chunk_tokens,
                                        int heads_per_item = 1) {
    S = p.num_seqs;
    Hk = p.num_kv_heads / heads_per_item;
    head_shift = stack_affine_shift(p.kv_head_bytes * heads_per_item, Hk);
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
    it.kvh = stack_affine_head(pos - rho * Hk, head_shift);
    const unsigned long long b0 = __ballot(key0 >= 0 && rank0 == rho);
    const unsigned long long b1 = __ballot(key1 >= 0 && rank1 == rho);
    const int s = b0 ? __builtin_ctzll(b0) : 64 + __builtin_ctzll(b1);
    it.seq = __builtin_amdgcn_readfirstlane(s);
    it.ctx = s < 64 ? __builtin_amdgcn_readlane(len0, s) : __builtin_amdgcn_readlane(len1, s - 64);
    it.tok_end = it.ctx;
    it.c_lo = 0;
    it.c_end = (it.ctx + chunk_tokens - 1) / chunk_tokens;
    it.part0 = 0;
    it.parts = 1;
    return it.ctx > 0;  // sorted: nothing but empty sequences follows an empty one
  }
  // block id of tile t of chunk `wave` of a sequence, as requested with the lengths
  __device__ __forceinline__ int first_id(int t, int seq) const {
    return seq < 64 ? __builtin_amdgcn_readlane(sid0[t], seq) : __builtin_amdgcn_readlane(sid1[t], seq - 64);
  }
};

struct SegmentItems {
  static constexpr int NQ = kSegmentMaxSeqs / 64;
  int ctxv[NQ], parts[NQ], incl[NQ], fullc[NQ], key[NQ];
  int S, Hk, m, seg_tokens, full_total, total_items, lane, key_top_bit, psize;
  int head_shift = -1;  // stack_affine_shift of the pool
  // even shares (m == 0): tape[j] = cost of all rows up to and including the lane's sequence's (row_cost);
  // the work-group's share is [cursor, share_end) of that tape
  bool even;
  int tape[NQ], cursor, share_end, steps_per_partition;
  float inv_steps_per_partition;

  // Lane holds sequences lane, lane + 64, ...  m, the partitions per segment, follows from the
  // batch, the number of work-groups and the compute units they share (partitions_per_segment).
  // heads_per_item: adjacent kv heads that one work-group takes together (its wavefronts in teams);
  // item_row_bytes: bytes of one token's K row (as of its V row) of an item
  __device__ __forceinline__ void build(const PagedAttnParams &p, int lane_, int groups, int heads_per_item,
                                        int item_row_bytes) {
    lane = lane_;
    S = p.num_seqs;
    Hk = p.num_kv_heads / heads_per_item;
    head_shift = stack_affine_shift(p.kv_head_bytes * heads_per_item, Hk);
    const int max_ctx = p.max_blocks_per_seq << p.block_shift;
    psize = p.partition_size;
    const int total_parts = count_partitions<NQ>(p.context_lens, S, max_ctx, p.partition_size, p.max_num_partitions, lane, ctxv, parts);
    // (cost of the batch in steps of kShareTokens, from above: every partition full, every row a piece)
    const long long steps_at_most = ((long long)total_parts * (psize >> kShareTokensLog2) + (long long)S * kSharePieceCost) * Hk;
    even = p.segment_force == -1 && steps_at_most < (1 << 24);  // (a batch beyond that is cut into segments)
    if (even) {
      build_even_shares(groups, p.compute_units);
      return;
    }
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
      // sort key of the last segment: length in 32-token steps (what a wavefront takes at a time),
      // then lower sequence number first; -1: none
      key[j] = rem > 0 ? (((rem + 31) >> 5) << 8) | (255 - (lane + 64 * j)) : -1;
      int x = fullc[j];
      if (j * 64 < S) {
        tails += __builtin_popcountll(__ballot(rem > 0));
        x = wave_inclusive_sum(x);
      }
      incl[j] = x + running;
      running = __builtin_amdgcn_readlane(incl[j], 63);
    }
    full_total = running;
    total_items = (full_total + tails) * Hk;
    // highest pair of bits a key can have: lengths of last segments stay below seg_tokens
    key_top_bit = (31 - __builtin_clz(((unsigned)((min(seg_tokens, kSegmentMaxContext - 1) + 31) >> 5) << 8) | 255u)) & ~1;
  }
  // Even shares.  A row costs its keys in steps of kShareTokens plus kSharePieceCost steps for what
  // every piece costs whatever its length (a merge, a store, a start without loads in flight).  The
  // rows' costs lie end to end on a tape; a work-group's share is a contiguous stretch of it.
  __device__ __forceinline__ int row_cost(int ctx) const {
    return ctx > 0 ? ((ctx + kShareTokens - 1) >> kShareTokensLog2) + kSharePieceCost : 0;
  }
  __device__ __forceinline__ void build_even_shares(int groups, int cus) {
    m = 0;
    seg_tokens = 0;
    int running = 0;
#pragma unroll
    for (int j = 0; j < NQ; ++j) {
      ctxv[j] = min(ctxv[j], parts[j] * psize);  // what the scratch arrays can hold
      int x = row_cost(ctxv[j]);
      if (j * 64 < S) x = wave_inclusive_sum(x);
      tape[j] = (x + running) * Hk;
      running = __builtin_amdgcn_readlane(x + running, 63);
    }
    const int n = running * Hk;  // below 2^24: SegmentItems::build
    // Two work-groups on every compute unit (g and g + cus): the hardware serves the older of the two
    // first, so that with equal shares it is through early and the younger one streams on alone, below
    // the unit's rate.  The older half of the work-groups takes kShareOlderPermille of the tape, so
    // that both are through together.
    int count = groups, g = (int)blockIdx.x, begin = 0, length = n;
    if (groups == 2 * cus) {
      const int older = (int)((float)n * (kShareOlderPermille * 0.001f));
      count = cus;
      if (g >= cus) {
        g -= cus;
        begin = older;
        length = n - older;
      } else {
        length = older;
      }
    }
    int extra;
    const int each = quotient_below_2p24(length, count, __builtin_amdgcn_rcpf((float)count), extra);
    cursor = begin + g * each + min(g, extra);  // the first `extra` work-groups take one step more
    share_end = cursor + each + (g < extra ? 1 : 0);
    total_items = n;
    steps_per_partition = psize >> kShareTokensLog2;
    inv_steps_per_partition = __builtin_amdgcn_rcpf((float)steps_per_partition);
  }
  // The partition boundary of a row of `parts` partitions nearest to cost position x of the row: where a
  // share that ends (or begins) there really ends (begins), since a piece is whole partitions.  Two
  // neighbouring work-groups evaluate it at the same position of the same row.
  __device__ __forceinline__ int nearest_cut(int x, int parts_of_row) const {
    int rem;
    return min(parts_of_row, quotient_below_2p24(x + (steps_per_partition >> 1), steps_per_partition, inv_steps_per_partition, rem));
  }
  // Next piece of this work-group's share: what the share holds of the row the cursor lies in.
  __device__ __forceinline__ bool next_of_share(int chunk_tokens, WorkItem &it) {
    while (cursor < share_end) {  // (a row of which rounding leaves the share nothing is passed over)
      int s = 0;
#pragma unroll
      for (int j = 0; j < NQ; ++j)
        if (j * 64 < S) s += __builtin_popcountll(__ballot(lane + 64 * j < S && tape[j] <= cursor));
      s = min(s, S - 1);
      int tape_s = 0, parts_s = 1, ctx_s = 0;
#pragma unroll
      for (int j = 0; j < NQ; ++j)
        if ((s >> 6) == j) {
          tape_s = __builtin_amdgcn_readlane(tape[j], s & 63);
          parts_s = __builtin_amdgcn_readlane(parts[j], s & 63);
          ctx_s = __builtin_amdgcn_readlane(ctxv[j], s & 63);
        }
      const int cost = max(row_cost(ctx_s), 1);
      const int into = cursor - (tape_s - cost * Hk);  // into the sequence's rows: kv head x cost + position in the row
      int x;
      const int kvh = quotient_below_2p24(into, cost, __builtin_amdgcn_rcpf((float)cost), x);
      const int row_begin = cursor - x, row_end = row_begin + cost;
      const int from = x == 0 ? 0 : nearest_cut(x, parts_s);
      const int to = share_end >= row_end ? parts_s : nearest_cut(share_end - row_begin, parts_s);
      cursor = min(row_end, share_end);
      if (to > from) {
        it.seq = __builtin_amdgcn_readfirstlane(s);
        it.kvh = __builtin_amdgcn_readfirstlane(kvh);
        it.ctx = ctx_s;
        it.part0 = __builtin_amdgcn_readfirstlane(from);
        it.parts = __builtin_amdgcn_readfirstlane(to - from);
        it.tok_end = to == parts_s ? ctx_s : to * psize;
        it.c_lo = from * psize / chunk_tokens;
        it.c_end = (it.tok_end + chunk_tokens - 1) / chunk_tokens;
        return true;
      }
    }
    return false;
  }
  // The sequence whose last segment is the rho-th longest (0: the longest).  The keys are distinct, so
  // the one that exactly rho others exceed is found from the top, two bits at a time (three counts
  // that do not depend on each other) -- when an item is looked up, one at a time and as a rule
  // behind loads that are already in flight; ranking all sequences against each other before the
  // first load cost a launch of 128 sequences 4 to 7 microseconds.
  __device__ __forceinline__ int sequence_of_tail(int rho) const {
    int found = 0;
#pragma nounroll
    for (int bit = key_top_bit; bit >= 0; bit -= 2) {
      int at_least[3] = {0, 0, 0};
#pragma unroll
      for (int j = 0; j < NQ; ++j)
        if (j * 64 < S) {
#pragma unroll
          for (int c = 0; c < 3; ++c) at_least[c] += __builtin_popcountll(__ballot(key[j] >= (found | ((c + 1) << bit))));
        }
      // counts fall with the candidate: the largest one that more than rho keys still reach
      const int digit = (at_least[0] > rho) + (at_least[1] > rho) + (at_least[2] > rho);
      found |= digit << bit;
    }
    return 255 - (found & 255);
  }
  // n-th item of work-group `group`, asked for n = 0, 1, 2, ... in turn.  Segments: position in the
  // sorted list -> (sequence, segment, kv head), kv head fastest.
  __device__ __forceinline__ bool at(int n, int groups, int group, int chunk_tokens, WorkItem &it) {
    if (even) return next_of_share(chunk_tokens, it);
    const int pos = snake_position(n, groups, group);
    if (pos >= total_items) return false;
    const int q = __builtin_amdgcn_readfirstlane(pos / Hk);
    it.kvh = stack_affine_head(pos - q * Hk, head_shift);
    int s = 0;
    const bool full = q < full_total;
    if (full) {
#pragma unroll
      for (int j = 0; j < NQ; ++j)
        if (j * 64 < S) s += __builtin_popcountll(__ballot(lane + 64 * j < S && incl[j] <= q));
    } else {
      s = sequence_of_tail(q - full_total);
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
    it.parts = (it.tok_end - tok_begin + psize - 1) / psize;
    it.c_lo = tok_begin / chunk_tokens;
    it.c_end = (it.tok_end + chunk_tokens - 1) / chunk_tokens;
    it.ctx = ctx_s;
    return true;
  }
};

}  // namespace fa
