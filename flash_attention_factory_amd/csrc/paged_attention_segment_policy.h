// How the segment form of the split path cuts sequences.  The attention kernels
// (paged_attention_segment_kernel.h, the split form of paged_attention_loop_two_tile_kernel.h)
// choose the cuts from the batch, every wavefront for itself, and write one partial per piece into
// the slot of the piece's first partition.  Two ways of cutting:
//   segments     every row is cut into segments of m partitions (partitions_per_segment), the
//                segments are dealt to the work-groups longest first;
//   even shares  (on request) the rows, laid end to end, are cut into one contiguous share per
//                work-group, equal in keys (plus a cost per piece) to within half a partition: a
//                work-group's pieces are the end of one row, whole rows, and the beginning of another.
// The reduce kernel (paged_attention_reduce_kernel.h) finds the pieces in the scratch arrays
// themselves: every slot of max_logits that a piece covers beyond its first holds a mark
// (segment_mark), a NaN no maximum can be.
#pragma once

#include "paged_attention_utils.h"

namespace fa {

constexpr int kSegmentMaxSeqs = 256;
constexpr int kSegmentMaxContext = 1 << 23;  // lengths are packed into 23 bits of a sort key
// The most partitions one segment may span.
#ifndef FA_SEGMENT_MAX_PARTS
#define FA_SEGMENT_MAX_PARTS 64
#endif
constexpr int kSegmentMaxPartitions = FA_SEGMENT_MAX_PARTS;
// Where work-groups share a compute unit and each should have work throughout (see `halves` below):
// bytes of K and V that a unit must have per segment it is given.
#ifndef FA_SEGMENT_BYTES_WORTH_CUTTING
#define FA_SEGMENT_BYTES_WORTH_CUTTING (768 << 10)
#endif
constexpr int kSegmentBytesWorthCutting = FA_SEGMENT_BYTES_WORTH_CUTTING;

// a / b for 0 <= a < 2^24 and b >= 1, given inv_b close to 1 / b: both are exact in fp32, so the
// product is off by one at most, which the remainder tells.
__device__ __forceinline__ int quotient_below_2p24(int a, int b, float inv_b, int &rem) {
  int q = (int)((float)a * inv_b);
  rem = a - q * b;
  if (rem < 0) { --q; rem += b; }
  if (rem >= b) { ++q; rem -= b; }
  return q;
}

// Sum over the 64 lanes of a wavefront (all of them active), in data-parallel-primitive moves
// rather than trips through the LDS crossbar: the callers run once per wavefront, before the
// first load of a launch, where every cycle is latency.
__device__ __forceinline__ int wave_total(int v) {
  return __builtin_amdgcn_readfirstlane(__reduce_add_sync(~0ull, v));
}

// Inclusive prefix sum over the 64 lanes, in data-parallel-primitive moves: shifts by 1, 2, 4 and 8
// within each row of 16 lanes (lanes shifted in from outside a row read 0), then the total of row 0
// onto row 1 and of row 2 onto row 3, then that of rows 0-1 onto rows 2-3.
__device__ __forceinline__ int wave_inclusive_sum(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xF, 0xF, true);  // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xF, 0xF, true);  // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xF, 0xF, true);  // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xF, 0xF, true);  // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xA, 0xF, false);  // row_bcast:15 into rows 1 and 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xC, 0xF, false);  // row_bcast:31 into rows 2 and 3
  return v;
}

// Segment length as a share (in 1/1024) of a compute unit's mean load, against the sequences
// per compute unit (in 1/1024).  Every sequence ends in a segment shorter than the others, so
// with many sequences per compute unit the short ones alone fill the GPU and only sequences well
// above the mean are worth cutting; with few, the whole segments are the work and one of them
// should be what a work-group gets.  Measured on 27 batches of 1 to 256 sequences (the length
// that was fastest for each, to within a few per cent): 1.12 of the load up to one sequence per
// compute unit, 0.57 at two, 0.37 at four, 0.35 from eight on.
__device__ __forceinline__ int segment_share_of_load(int seqs_per_cu_1024) {
  // straight lines between the measured points; literals and shifts, so that nothing here is a
  // table in memory or a division
  const int x = seqs_per_cu_1024;
  if (x <= 1024) return 1147;
  if (x <= 2048) return 1147 - ((563 * (x - 1024)) >> 10);
  if (x <= 4096) return 584 - ((205 * (x - 2048)) >> 11);
  if (x <= 8192) return 379 - ((19 * (x - 4096)) >> 12);
  return 360;
}

// The mark in the slots of max_logits that a piece covers beyond its first: a NaN no maximum can be
// (maxima are finite or -inf, and a NaN that arithmetic makes has none of the low mantissa bits
// set); in its low byte the segment length m, or 0 under even shares (for whoever inspects the
// arrays: the reduce kernel only asks whether a slot holds a mark).
constexpr uint32_t kSegmentMarkBits = 0x7FD3A600u, kSegmentMarkMask = 0xFFFFFF00u;
static_assert(kSegmentMaxPartitions < 256, "the segment length is kept in one byte of the mark");
__device__ __forceinline__ float segment_mark(int m) { return __uint_as_float(kSegmentMarkBits | (uint32_t)m); }
__device__ __forceinline__ bool is_segment_mark(float slot) {
  return (__float_as_uint(slot) & kSegmentMarkMask) == kSegmentMarkBits;
}

// Marks the slots that a piece of `parts` partitions covers beyond its first, in the max_logits rows
// of `heads` consecutive heads; first_slot: the piece's own slot in the first of these rows;
// pitch: slots per row.  One wavefront, all lanes.
__device__ __forceinline__ void mark_covered_slots(float *max_logits, int64_t first_slot, int heads, int pitch,
                                                   int parts, int lane, int low_byte) {
  const float mark = segment_mark(low_byte);
  for (int h = 0; h < heads; ++h)
    for (int q = 1 + lane; q < parts; q += 64) max_logits[first_slot + (int64_t)h * pitch + q] = mark;
}

// Even shares are cut on request only (options->segment_partitions = -1).  They give every work-group
// the same number of keys to within half a partition, where dealing sorted segments leaves the most
// loaded compute unit of a serving mix 7-10 % above the mean -- and yet, measured on 130 batches of 1 to
// 256 sequences (both cache types, log-normal, long and short rows), segments are as fast or faster in
// nine of ten, by 1-7 % on the large mixes: what a compute unit streams is not a matter of keys alone.
// The older of a unit's two work-groups is served first and wants the larger share, rows of a few hundred
// keys cost more per key than long ones, and the fitted segment rule has both in it.
// The unit the shares are counted in: keys of one row, 32 at a time (what a wavefront takes at a time);
// and what a piece costs beyond its keys, in the same unit.
constexpr int kShareTokensLog2 = 5, kShareTokens = 1 << kShareTokensLog2;
#ifndef FA_SHARE_PIECE_COST
#define FA_SHARE_PIECE_COST 4
#endif
constexpr int kSharePieceCost = FA_SHARE_PIECE_COST;
// With two work-groups per compute unit: what the older one of a unit takes of the unit's work, in 1/1000.
#ifndef FA_SHARE_OLDER_PERMILLE
#define FA_SHARE_OLDER_PERMILLE 540
#endif
constexpr int kShareOlderPermille = FA_SHARE_OLDER_PERMILLE;
// Whole segments and segments in all (per kv head) that a segment length of m partitions
// leaves: lane holds sequences lane, lane + 64, ... of which ctxv / parts are the lengths and
// live partitions.
template <int NQ>
__device__ __forceinline__ void count_segments(const int (&ctxv)[NQ], const int (&parts)[NQ], int S,
                                               int partition_size, int m, int &whole, int &all) {
  const int seg_tokens = m * partition_size;
  const float inv = __builtin_amdgcn_rcpf((float)seg_tokens);
  int f = 0, t = 0;
#pragma unroll
  for (int j = 0; j < NQ; ++j)
    if (j * 64 < S) {  // wave-uniform
      const int cut = min(ctxv[j], parts[j] * partition_size);  // what the scratch arrays can hold
      int rem;
      f += quotient_below_2p24(cut, seg_tokens, inv, rem);  // lengths stay below 2^23 (kSegmentMaxContext)
      t += __builtin_popcountll(__ballot(rem > 0));
    }
  whole = wave_total(f);
  all = whole + t;
}

// How many partitions one segment spans, as every wavefront of an attention launch works it out
// from the same context lengths.  total_partitions: live partitions of all sequences
// (count_partitions); groups: work-groups of the launch; cus: compute units of the GPU.
//
// Work-groups g and g + cus share a compute unit, and what a compute unit streams is what
// bounds the launch: the length aims at a share of the mean load of a compute unit
// (segment_share_of_load), or, where two work-groups share a unit and the whole segments are the
// work, at the mean load of a work-group; with token rows that lie apart in the pools, or three
// work-groups on a unit, at half a work-group's load.  With contiguous rows and one or two work-groups per unit, whole segments
// -- all of one length -- must not pile up, for that length is then what the launch waits for;
// so: with at most one sequence per unit, one segment per unit if that fits (phase 0 below);
// else no more whole segments than work-groups (the length grows until that holds), and, with
// few sequences, not a count of segments between one per unit and most of the work-groups (some
// units would hold two and stream twice as long as the others; the length grows until every
// unit holds one).
template <int NQ>
__device__ __forceinline__ int partitions_per_segment(const int (&ctxv)[NQ], const int (&parts)[NQ],
                                                      int total_partitions, int S, int partition_size,
                                                      int num_kv_heads, int groups, int cus, bool rows_apart,
                                                      int partition_bytes) {
  const int units = max(1, min(groups, cus));  // compute units at work
  const int sharing = groups <= units ? 1 : groups <= 2 * units ? 2 : (groups + units - 1) / units;  // work-groups on each
  int live = 0;
#pragma unroll
  for (int j = 0; j < NQ; ++j)
    if (j * 64 < S) live += __builtin_popcountll(__ballot(parts[j] > 0));
  const float items = (float)total_partitions * (float)num_kv_heads;
  const float per_unit = __builtin_amdgcn_rcpf((float)units);
  const float seqs_per_cu = fminf((float)live * (float)num_kv_heads * per_unit, 1024.f);
  int share = segment_share_of_load((int)(seqs_per_cu * 1024.f));
  // Work-groups sharing a unit.  Token rows that lie apart in the pools (upstream's layout): two
  // segments per work-group whatever the batch -- a work-group alone on its unit does not stream
  // scattered rows at the unit's rate, so both of a unit's work-groups should have work
  // throughout (measured on 25 such batches: within 1.4 % of the best length on average, where the
  // rule for contiguous rows is 3-8 % off).  The same where three or more share a unit (the
  // head-size-64 instances: short items, and no batch of theirs measured more than 8 % off with it,
  // where a longer segment lost 20 % on one).  Contiguous rows, two on a unit: a whole segment is
  // what a work-group gets.
  const bool halves = sharing > 2 || (rows_apart && sharing > 1);
  if (halves) {
    // two segments per work-group, 2 * sharing per unit -- unless the unit's load is small: every segment
    // costs a merge, a store and a restart of the stream whatever its length, so a unit is given one
    // segment per kSegmentBytesWorthCutting of K and V at most (upstream's own perf shape, 64 sequences of
    // 1500 keys in byte caches with head size 64: 0.4 MB per unit, and the rows are best left whole)
    const float load_bytes = items * per_unit * (float)partition_bytes;
    const int n = max(1, min((int)(load_bytes * (1.0f / (float)kSegmentBytesWorthCutting) + 0.5f), 2 * sharing));
    share = 1024 / n;
  } else if (sharing == 2) share = min(share, 512);
  int m = (int)fminf(items * per_unit * ((float)share * (1.0f / 1024.f)) + 0.5f, (float)kSegmentMaxPartitions);
  m = max(m, 1);
  if (m == 1 && items <= (float)groups) return 1;  // a partition per work-group at most: nothing to weigh
  if (halves) return m;
  // At most one sequence per shared compute unit: first try one segment per unit (the shortest
  // length that leaves no more segments than units), as long as a segment is then at most 1.25 of
  // a unit's mean load -- a work-group alone on its unit streams that much faster than its share.
  const long long items_all = (long long)total_partitions * num_kv_heads;
  const bool few = sharing > 1 && 2 * live * num_kv_heads <= units;
  const int aimed = m;
  int phase = 1;  // 0: one segment per unit; 1: no more whole segments than work-groups; 2: not between
  if (sharing > 1 && live * num_kv_heads <= units && items_all > units) {
    phase = 0;
    m = (int)fminf(ceilf(items * per_unit), (float)kSegmentMaxPartitions);
  }
  // One loop, not unrolled: this code runs once per wavefront, at the speed instructions arrive
  // from memory, so its size is its cost.
  int before = 0, tries = 0;
#pragma nounroll
  for (int evaluations = 0; evaluations < 12; ++evaluations) {
    if (phase == 0 && (tries >= 4 || m > kSegmentMaxPartitions || 4LL * m * units > 5 * items_all)) {
      phase = 1;
      m = aimed;
      tries = 0;
    }
    int whole, all;
    count_segments<NQ>(ctxv, parts, S, partition_size, m, whole, all);
    const long long n = (long long)all * num_kv_heads;
    if (phase == 0) {
      if (n <= units) return m;
      ++m;
      ++tries;
      continue;
    }
    if (phase == 1) {
      if ((long long)whole * num_kv_heads > groups && tries < 3 && m < kSegmentMaxPartitions) {
        ++m;
        ++tries;
        continue;
      }
      if (!(few && n > units && n * 20 < (long long)groups * 17)) return m;
      phase = 2;
      before = m;
    } else if (n <= units) {
      return m;
    }
    if (m - before >= 4 || m >= kSegmentMaxPartitions) return before;
    ++m;
  }
  return before > 0 ? before : m;
}

// Live partitions of all sequences, as every wavefront of an attention launch computes them:
// lane holds sequences lane, lane+64, ...  Returns the total; per-lane counts in `parts`.
template <int NQ>
__device__ __forceinline__ int count_partitions(const int32_t *context_lens, int S, int max_ctx,
                                                int partition_size, int max_num_partitions, int lane,
                                                int (&ctxv)[NQ], int (&parts)[NQ]) {
  // every lane asks for its NQ lengths at once (lanes past the batch for the last one, which they
  // then drop): one trip to memory, not one per 64 sequences
  int len[NQ];
#pragma unroll
  for (int j = 0; j < NQ; ++j) len[j] = context_lens[min(lane + 64 * j, S - 1)];
  int local = 0;
  const float inv = __builtin_amdgcn_rcpf((float)partition_size);
#pragma unroll
  for (int j = 0; j < NQ; ++j) {
    const int c = lane + 64 * j < S ? max(0, min(len[j], max_ctx)) : 0;
    ctxv[j] = c;
    // lengths and the partition size stay below 2^23 (kSegmentMaxContext: the launcher sees to it)
    int rem;
    parts[j] = min(quotient_below_2p24(c + partition_size - 1, partition_size, inv, rem), max_num_partitions);
    local += parts[j];
  }
  return wave_total(local);
}

}  // namespace fa
