// Host launcher and dispatcher of the split-context path: the partition kernel
// followed by the reduce kernel.
//
// Same role and argument list as upstream paged_attention_reduce/launch_kernels_reduce.h:
// launch_paged_attn_v2 (:18-78) submits the attention kernel over
// (sequences, kv heads, partitions) and then the reduce kernel over (sequences, heads),
// returning both kernel times; dispatch_paged_attention (:80-197) picks the instance.
// Upstream waits on the host between the two kernels (:56); here they are ordered by
// the stream and nothing blocks unless timing is requested.
#pragma once

#include <algorithm>

#include "launch_common.h"
#include "launch_kernels_loop.h"

namespace fa {

// ---- which kernels a call of the split path runs ------------------------------------------------
// Upstream's split path always runs its two kernels (launch_kernels_reduce.h:18-78), and its own perf
// loop runs it on rows of 1500 keys (test_paged.py:607-631), where splitting has nothing to give: the
// second kernel costs 4-5 us of every call whatever it finds to do, and a row of a thousand keys is
// read by one work-group in little more than that.  What the host knows of a batch without reading
// device memory is an upper bound on its rows: max_context_len (upstream passes seqlen_k), the block
// table's width and the scratch arrays' capacity.  Measured over 113 batches (head sizes 64 and 128,
// 16-bit and byte caches, 2 to 128 sequences of up to 4096 keys, equal and ragged lengths), the loop
// kernel against the split kernels:
//   rows of at most kSplitNeverBelowTokens keys        the loop kernel is as fast or faster in all 33
//                                                      batches (1.0-1.9 times)
//   rows of at most kSplitFullGpuBelowTokens keys,     faster in 16 of 18 batches (by 2-18 %; slower
//   and a (sequence, kv head) row for every unit       by 6 and 18 % in two ragged ones)
//   anything longer, or fewer rows                     the split kernels win in 45 of 62 batches, up
//                                                      to 2.7 times (the loop kernel by at most 20 %)
// In the first two cases the call IS the loop kernel: one launch, the same `out`, the scratch
// arrays untouched, and {t, 0} as its two times.
constexpr int kSplitNeverBelowTokens = 1024;
constexpr int kSplitFullGpuBelowTokens = 2048;

// Upper bound on the keys of a row as far as the host knows it; the scratch arrays hold
// max_num_partitions * partition_size of them, and a call whose rows could exceed that is left to
// the split kernels (which cut such a row to what the arrays hold).
inline int64_t split_row_bound(const fa_paged_attention_shape &shape, int32_t partition_size, int32_t max_context_len) {
  const int64_t table = (int64_t)shape.max_blocks_per_seq * shape.block_size;
  const int64_t known = max_context_len > 0 ? std::min<int64_t>(max_context_len, table) : table;
  const int64_t scratch = (int64_t)shape.max_num_partitions * partition_size;
  return known <= scratch ? known : INT64_MAX;
}

// rows: (sequence, kv head) items as the loop kernel deals them (pairs or teams of kv heads count once)
inline bool split_call_runs_as_loop(int64_t row_bound, int64_t rows, int compute_units) {
  if (row_bound <= kSplitNeverBelowTokens) return true;
  return row_bound <= kSplitFullGpuBelowTokens && rows >= compute_units;
}

// (sequence, kv head) items of a batch as the persistent loop kernel deals them.
inline int64_t loop_rows_of(const fa_paged_attention_shape &shape, const Resolved &r, bool kv8) {
  int64_t heads = r.pair_heads ? shape.num_kv_heads / 2 : shape.num_kv_heads;
  // teams: two adjacent kv heads with 128-byte token rows per work-group (launch_kernels_loop.h)
  const bool rows_128 = shape.head_size * (kv8 ? 1 : 2) == 128;
  if (!r.pair_heads && rows_128 && shape.kv_token_stride != shape.head_size && shape.kv_head_stride == shape.head_size &&
      shape.num_kv_heads % 2 == 0)
    heads /= 2;
  return (int64_t)shape.num_seqs * heads;
}

#ifndef FA_STRICT_HEADS
#define FA_STRICT_HEADS 4
#endif
constexpr int kStrictHeads = FA_STRICT_HEADS;

enum SplitForm { kSplitFormGrid = 0, kSplitFormSegment = 1, kSplitFormLoop = 2 };  // = fa_split_form

// compute_units: of the GPU the call would run on
inline SplitForm split_form_of(const fa_paged_attention_shape &shape, const Resolved &r, bool kv8,
                               int32_t max_context_len, int compute_units) {
  if (r.schedule != FA_SCHEDULE_AUTO) return kSplitFormGrid;
  const bool loop_persistent = loop_persistent_fits(shape) && shape.num_seqs <= kLoopPersistentMaxSeqs;
  if (loop_persistent && r.segment_partitions == 0 && !r.keep_split &&
      split_call_runs_as_loop(split_row_bound(shape, r.partition_size, max_context_len), loop_rows_of(shape, r, kv8),
                              compute_units))
    return kSplitFormLoop;
  const bool segment = (kv8 ? SegmentSplit<true>::use : SegmentSplit<false>::use) && shape.num_pool_blocks > 0 &&
                       r.partition_size < kSegmentMaxContext &&
                       (int64_t)shape.max_blocks_per_seq * shape.block_size < kSegmentMaxContext;
  return segment ? kSplitFormSegment : kSplitFormGrid;
}

// Attention and reduce launches of one batch that a single attention launch can take (segment
// form for up to kSegmentMaxSeqs sequences, else the grid form).  Kernel times are ADDED to
// us_out[0] (attention) and us_out[1] (reduce) when the call is timed.
// HEAD_SIZE: head size of the attention kernel instance; OUT_D: elements of a row of out and
// tmp_out -- the same, except for pairs of kv heads (Resolved::pair_heads: 128 and 64).
template <int HEAD_SIZE, typename QT, int KVF, int OUT_D = HEAD_SIZE>
inline fa_status launch_paged_attn_v2_batch(void *out, const void *query, const void *key_cache,
                                            const void *value_cache, const int32_t *block_tables,
                                            const int32_t *context_lens, float scale,
                                            float *exp_sums, float *max_logits, float *tmp_out,
                                            const fa_paged_attention_shape &shape, const Resolved &r,
                                            float *us_out) {
  constexpr bool KV8 = KVF != kKv16;
  constexpr int NW = WavesPerGroup<true>::value;
  PagedAttnParams p = make_params(tmp_out, exp_sums, max_logits, query, key_cache, value_cache,
                                  block_tables, context_lens, scale, shape, r);
  KernelTimer timer(r.elapsed_us != nullptr, r.stream);
  // kernel 1.  Segment form when the batch fits it: as many multi-wavefront work-groups as
  // the GPU keeps resident share out segments of several partitions.  Otherwise one
  // work-group per (kv head, partition slot, sequence); slots past a sequence's length
  // return at once and write nothing (paged_attention_kernel_v2.hpp:577-579).
  int segment_groups = 0;  // > 0: the segment kernel ran with that many work-groups
  // score modifiers, several query tokens, per-head or per-block scales: the extended instances
  const bool ext = r.mask_flags != 0 || r.query_len > 1 || r.kv_scale_mode != 0;
  float attention_us = 0.f;
  const bool persistent_fits = SegmentSplit<KV8>::use && shape.num_seqs <= kSegmentMaxSeqs && shape.num_pool_blocks > 0 &&
                               r.partition_size < kSegmentMaxContext &&
                               (int64_t)shape.max_blocks_per_seq * shape.block_size < kSegmentMaxContext;
  const bool segment_form = persistent_fits && r.schedule == FA_SCHEDULE_AUTO;
  // Upstream's decomposition -- one partial per partition, every live slot of the scratch arrays
  // written as upstream writes it -- by resident work-groups: each wavefront takes one kv head of four
  // adjacent ones and walks whole partitions of it, its loads running on across the partitions'
  // ends; a partial goes from its registers to tmp_out, no LDS, nobody waited for.  (One work-group per
  // partition, the form below, starts its stream anew for every 512 keys.)
  const bool strict_form = persistent_fits && r.schedule == FA_SCHEDULE_GRID && !ext && !r.pair_heads &&
                           p.num_kv_heads % 4 == 0;
  // One launch per group of query tokens that fit the MFMA columns (one launch for decode): 16
  // columns, or in the segment form two tiles of 16 held by every wavefront.
  // Every launch fills its own rows of the scratch arrays, the reduce kernel runs once.
  if (segment_form) p.final_out = out;  // rows of one partial are stored as results (PagedAttnParams::final_out)
  const int per_tile = p.query_count;
  const int per_launch = (segment_form && r.query_len > per_tile) ? 2 * per_tile : per_tile;
  for (int q0 = 0; q0 < r.query_len; q0 += per_launch) {
    p.query_first = q0;
    p.query_count = std::min(per_launch, r.query_len - q0);
    if (strict_form) {
      constexpr int SW = SegmentSplit<KV8>::waves;
      static_assert(SW == 4, "four kv heads per work-group, one wavefront each");
      auto kernel = paged_attn_segment_kernel<HEAD_SIZE, QT, KVF, SW, SegmentSplit<KV8>::occ, Pipeline<KV8>::tiles_per_chunk, false, kStrictHeads>;
      int resident = 0, cus = 0;
      FA_HIP_CHECK(resident_groups(kernel, SW * 64, &resident, &cus));
      p.compute_units = cus;
      p.segment_force = 1;  // one partial per partition
      const int64_t max_items = (int64_t)shape.num_seqs * shape.max_num_partitions * (p.num_kv_heads / kStrictHeads);
      if (r.plan) {
        r.plan->work_groups = (int)std::min<int64_t>(resident, max_items);
        r.plan->kv_heads_per_item = kStrictHeads;
        return FA_OK;
      }
      FA_HIP_CHECK(timer.launch(kernel, dim3((unsigned)std::min<int64_t>(resident, max_items)), dim3(SW * 64), 0, p));
    } else if (segment_form) {
      // Segment form: multi-wavefront work-groups, one partial per segment of partitions.
      constexpr int SW = SegmentSplit<KV8>::waves;
      auto plain = paged_attn_segment_kernel<HEAD_SIZE, QT, KVF, SW, SegmentSplit<KV8>::occ,
                                             Pipeline<KV8>::tiles_per_chunk, false>;
      auto extended = paged_attn_segment_kernel<HEAD_SIZE, QT, KVF, SW, SegmentSplit<KV8>::occ,
                                                Pipeline<KV8>::tiles_per_chunk, true>;
      // two column tiles in the registers of every wavefront: K and V are loaded once for both
      auto two_tiles = paged_attn_loop_two_tile_kernel<HEAD_SIZE, QT, KVF, SW, TwoTile<KV8>::tiles_per_chunk, true, true>;
      auto kernel = !ext ? plain : p.query_count > per_tile ? two_tiles : extended;
      // Pools in upstream's layout whose token rows are 128 bytes (FP8 with head size 128, 16-bit
      // with head size 64): a token's row of one kv head is a single line, and the rows of its
      // neighbours lie next to it.  A work-group then takes two
      // adjacent kv heads of a segment, two wavefronts each, so that both lines are asked for at
      // about the same time (measured with loads alone: 5.8 -> 6.2-6.4 TB/s, what rows of 256
      // bytes reach; the serving-mix configuration 300 -> 282 us, upstream's 16-bit perf shape 44.4 ->
      // 42.0 us).  With rows of 256 bytes the same arrangement gained nothing.
      // Not for batches that cannot give every compute unit a pair even at one partition per
      // segment (a single sequence of 32 partitions and 8 kv heads: 19.2 us against 15.9 us).
      bool head_teams = false;
      if constexpr (HEAD_SIZE * (KV8 ? 1 : 2) == 128) {  // token rows of 128 bytes
        int units = 0, unused = 0;
        FA_HIP_CHECK(resident_groups(kernel, SW * 64, &unused, &units));
        const int64_t most_pairs = (int64_t)shape.num_seqs * shape.max_num_partitions * (p.num_kv_heads / 2);
        if (!r.pair_heads && p.kv_rows_apart && shape.kv_head_stride == shape.head_size && p.num_kv_heads % 2 == 0 &&
            most_pairs >= units) {
          if (kernel == two_tiles)
            kernel = paged_attn_loop_two_tile_kernel<HEAD_SIZE, QT, KVF, SW, TwoTile<KV8>::tiles_per_chunk, true, true, 2>;
          else
            kernel = ext ? paged_attn_segment_kernel<HEAD_SIZE, QT, KVF, SW, SegmentSplit<KV8>::occ,
                                                     Pipeline<KV8>::tiles_per_chunk, true, 2>
                         : paged_attn_segment_kernel<HEAD_SIZE, QT, KVF, SW, SegmentSplit<KV8>::occ,
                                                     Pipeline<KV8>::tiles_per_chunk, false, 2>;
          head_teams = true;
        }
      }
      if (q0 == 0) {
        // Every launch of the call gets the same number of work-groups: the segment length follows
        // from it.
        int resident = 0, cus = 0;
        FA_HIP_CHECK(resident_groups(kernel, SW * 64, &resident, &cus));
        p.compute_units = cus;
        // two teams in a work-group stream like two work-groups: one such work-group per compute
        // unit (measured on the serving mix: 293 us with two per unit, 282 us with one)
        if (head_teams) resident = std::min(resident, cus);
        if (ext && r.query_len > per_launch && r.query_len % per_launch <= per_tile) {  // a one-tile launch ends the call
          int other = 0;
          FA_HIP_CHECK(resident_groups(extended, SW * 64, &other));
          resident = std::min(resident, other);
        }
        const int64_t max_items =
            (int64_t)shape.num_seqs * shape.max_num_partitions * p.num_kv_heads;
        segment_groups = (int)std::min<int64_t>(resident, max_items);
      }
      if (r.plan) {
        r.plan->work_groups = segment_groups;
        r.plan->kv_heads_per_item = (head_teams || r.pair_heads) ? 2 : 1;
        return FA_OK;
      }
      FA_HIP_CHECK(timer.launch(kernel, dim3((unsigned)segment_groups), dim3(SW * 64), 0, p));
    } else if (r.plan) {
      return FA_OK;
    } else if (KV8 && HEAD_SIZE == 128 && !ext && !r.pair_heads && r.schedule == FA_SCHEDULE_GRID_LDS) {
      // grid form, K and V staged through LDS: one wavefront per partition
      if constexpr (KV8 && HEAD_SIZE == 128) {
        const dim3 grid(p.num_kv_heads, shape.max_num_partitions, shape.num_seqs);
        FA_HIP_CHECK(timer.launch(paged_attn_lds_kernel<HEAD_SIZE, QT, KVF, true, 1, 2>, grid, dim3(64), 0, p));
      }
    } else if (ext) {
      const dim3 grid(p.num_kv_heads, shape.max_num_partitions, shape.num_seqs);
      FA_HIP_CHECK(timer.launch(
          paged_attn_kernel<HEAD_SIZE, QT, KVF, true, NW, Pipeline<KV8>::occ,
                            Pipeline<KV8>::tiles_per_chunk, true>,
          grid, dim3(NW * 64), 0, p));
    } else {
      const dim3 grid(p.num_kv_heads, shape.max_num_partitions, shape.num_seqs);
      FA_HIP_CHECK(timer.launch(
          paged_attn_kernel<HEAD_SIZE, QT, KVF, true, NW, Pipeline<KV8>::occ,
                            Pipeline<KV8>::tiles_per_chunk>,
          grid, dim3(NW * 64), 0, p));
    }
    if (r.elapsed_us) FA_HIP_CHECK(timer.accumulate(0, &attention_us));
  }

  // kernel 2: one wavefront per (head, sequence)
  ReduceParams rp;
  rp.out = out;
  rp.exp_sums = exp_sums;
  rp.max_logits = max_logits;
  rp.tmp_out = tmp_out;
  rp.context_lens = context_lens;
  rp.num_heads = shape.num_heads;
  rp.max_num_partitions = shape.max_num_partitions;
  rp.partition_size = r.partition_size;
  rp.max_context = (int32_t)std::min<int64_t>((int64_t)shape.max_blocks_per_seq * shape.block_size, INT32_MAX);
  rp.num_seqs = shape.num_seqs;
  rp.num_kv_heads = p.num_kv_heads;  // what the attention kernel dealt by: pairs with r.pair_heads
  rp.query_len = r.query_len;
  rp.segment_groups = segment_groups;
  const dim3 rgrid((unsigned)((int64_t)shape.num_heads * shape.num_seqs * r.query_len));
  const bool one_wave = (int64_t)shape.num_heads * shape.num_seqs * r.query_len >= kReduceSingleWaveMinPairs;
  if (segment_groups > 0) {
    if (one_wave) FA_HIP_CHECK(timer.launch(paged_attn_reduce_kernel<OUT_D, QT, 1, true>, rgrid, dim3(64), 1, rp));
    else FA_HIP_CHECK(timer.launch(paged_attn_reduce_kernel<OUT_D, QT, 4, true>, rgrid, dim3(256), 1, rp));
  } else {
    if (one_wave) FA_HIP_CHECK(timer.launch(paged_attn_reduce_kernel<OUT_D, QT, 1, false>, rgrid, dim3(64), 1, rp));
    else FA_HIP_CHECK(timer.launch(paged_attn_reduce_kernel<OUT_D, QT, 4, false>, rgrid, dim3(256), 1, rp));
  }
  if (r.elapsed_us) {
    us_out[0] += attention_us;
    FA_HIP_CHECK(timer.accumulate(1, &us_out[1]));
  }
  return FA_OK;
}

// Pairs of kv heads (Resolved::pair_heads) run in the head-size-128 attention instance, everything
// else in the instance of its own head size.
template <int HEAD_SIZE, typename QT, int KVF>
inline fa_status launch_paged_attn_v2_instance(void *out, const void *query, const void *key_cache,
                                               const void *value_cache, const int32_t *block_tables,
                                               const int32_t *context_lens, float scale,
                                               float *exp_sums, float *max_logits, float *tmp_out,
                                               const fa_paged_attention_shape &shape, const Resolved &r,
                                               float *us_out) {
  if constexpr (KVF != kKv16 && HEAD_SIZE == 64) {
    if (r.pair_heads)
      return launch_paged_attn_v2_batch<128, QT, KVF, 64>(out, query, key_cache, value_cache, block_tables,
                                                          context_lens, scale, exp_sums, max_logits, tmp_out, shape,
                                                          r, us_out);
  }
  return launch_paged_attn_v2_batch<HEAD_SIZE, QT, KVF>(out, query, key_cache, value_cache, block_tables,
                                                        context_lens, scale, exp_sums, max_logits, tmp_out, shape, r,
                                                        us_out);
}

// Whether the segment kernel takes batches of this shape at all (given few enough sequences).
template <bool KV8>
inline bool segment_form_fits(const fa_paged_attention_shape &shape) {
  return SegmentSplit<KV8>::use && shape.num_pool_blocks > 0 &&
         (int64_t)shape.max_blocks_per_seq * shape.block_size < kSegmentMaxContext;
}

// A batch of more sequences than the segment kernel lists is cut into equal sub-batches, each
// with its own segment and reduce launch (every attention launch chooses its segment length and
// marks its rows with it): measured on a 512-sequence serving mix, 56 % of peak in the
// grid form against 71 % for 256 sequences in the segment form.
template <int HEAD_SIZE, typename QT, int KVF>
inline fa_status launch_paged_attn_v2(void *out, const void *query, const void *key_cache,
                                      const void *value_cache, const int32_t *block_tables,
                                      const int32_t *context_lens, float scale,
                                      int32_t max_context_len,
                                      float *exp_sums, float *max_logits, float *tmp_out,
                                      const fa_paged_attention_shape &shape, const Resolved &r) {
  float us[2] = {0.f, 0.f};
  // rows too short for splitting to pay: the call is the loop kernel (see split_call_runs_as_loop)
  int cus = 0;
  FA_HIP_CHECK(compute_units_of_current_device(&cus));
  const SplitForm form = split_form_of(shape, r, KVF != kKv16, max_context_len, cus);
  if (r.plan) {
    r.plan->form = form;
    r.plan->compute_units = cus;
    if (form != kSplitFormSegment) return FA_OK;
  }
  if (form == kSplitFormLoop) {
    const fa_status st = launch_paged_attn_loop<HEAD_SIZE, QT, KVF>(out, query, key_cache, value_cache, block_tables,
                                                                    context_lens, scale, max_context_len, shape, r);
    if (r.elapsed_us) r.elapsed_us[1] = 0.f;
    return st;
  }
  // most sequences one launch takes: what the segment kernel lists, or what the grid's third
  // dimension holds
  constexpr int kGridMaxSeqs = 65535;
  const bool segment_pieces = r.schedule == FA_SCHEDULE_AUTO && segment_form_fits<(KVF != kKv16)>(shape) &&
                              r.partition_size < kSegmentMaxContext &&
                              shape.num_seqs > kSegmentMaxSeqs;
  const int most = segment_pieces ? kSegmentMaxSeqs : kGridMaxSeqs;
  if (shape.num_seqs > most) {
    const int pieces = (shape.num_seqs + most - 1) / most;
    const int per = (shape.num_seqs + pieces - 1) / pieces;
    const int64_t rows = (int64_t)r.query_len * shape.num_heads;  // (query token, head) rows per sequence
    const int64_t row_bytes = rows * shape.head_size * 2;           // of query and out
    const int64_t slots = rows * shape.max_num_partitions;          // scratch slots per sequence
    for (int s0 = 0; s0 < shape.num_seqs; s0 += per) {
      fa_paged_attention_shape sub = shape;
      sub.num_seqs = std::min(per, shape.num_seqs - s0);
      const fa_status st = launch_paged_attn_v2_instance<HEAD_SIZE, QT, KVF>(
          reinterpret_cast<char *>(out) + s0 * row_bytes, reinterpret_cast<const char *>(query) + s0 * row_bytes,
          key_cache, value_cache, block_tables + (int64_t)s0 * shape.max_blocks_per_seq, context_lens + s0, scale,
          exp_sums + s0 * slots, max_logits + s0 * slots, tmp_out + s0 * slots * shape.head_size, sub, r, us);
      if (st != FA_OK) return st;
    }
  } else {
    const fa_status st = launch_paged_attn_v2_instance<HEAD_SIZE, QT, KVF>(
        out, query, key_cache, value_cache, block_tables, context_lens, scale, exp_sums, max_logits, tmp_out,
        shape, r, us);
    if (st != FA_OK) return st;
  }
  if (r.elapsed_us) {
    r.elapsed_us[0] = us[0];
    r.elapsed_us[1] = us[1];
  }
  return report_kernel_status(r);
}

template <bool KV8>
inline fa_status dispatch_paged_attention_any(void *out, const void *query, const void *key_cache,
                                              const void *value_cache,
                                              const int32_t *block_tables,
                                              const int32_t *context_lens, float scale,
                                              int32_t max_context_len, float *exp_sums,
                                              float *max_logits, float *tmp_out,
                                              const fa_paged_attention_shape *shape,
                                              const fa_paged_attention_options *options,
                                              fa_split_plan *plan = nullptr) {
  Resolved r;
  fa_status st = validate_and_resolve(out, query, key_cache, value_cache, block_tables, context_lens,
                                      max_context_len, exp_sums, max_logits, tmp_out, shape, options,
                                      KV8, /*split=*/true, &r);
  if (st != FA_OK || r.validate_only) return st;
  r.plan = plan;
  const bool bf16 = shape->q_dtype == FA_DTYPE_BF16;
#define FA_V2_CASE(HS, QT)                                                                       \
  do {                                                                                           \
    if (!KV8)                                                                                    \
      return launch_paged_attn_v2<HS, QT, kKv16>(out, query, key_cache, value_cache,             \
                                                 block_tables, context_lens, scale,              \
                                                 max_context_len, exp_sums, max_logits, tmp_out, \
                                                 *shape, r);                                     \
    if (r.e4m3)                                                                                  \
      return launch_paged_attn_v2<HS, QT, kKvE4M3>(out, query, key_cache, value_cache,           \
                                                   block_tables, context_lens, scale,            \
                                                   max_context_len, exp_sums, max_logits,        \
                                                   tmp_out, *shape, r);                          \
    return launch_paged_attn_v2<HS, QT, kKvE5M2>(out, query, key_cache, value_cache,             \
                                                 block_tables, context_lens, scale,              \
                                                 max_context_len, exp_sums, max_logits, tmp_out, \
                                                 *shape, r);                                     \
  } while (0)
  if (shape->head_size == 128) {
    if (bf16) FA_V2_CASE(128, BF16);
    FA_V2_CASE(128, F16);
  }
  if (bf16) FA_V2_CASE(64, BF16);
  FA_V2_CASE(64, F16);
#undef FA_V2_CASE
}

inline fa_status dispatch_paged_attention(void *out, const void *query, const void *key_cache,
                                          const void *value_cache, const int32_t *block_tables,
                                          const int32_t *context_lens, float scale,
                                          int32_t max_context_len, float *exp_sums,
                                          float *max_logits, float *tmp_out,
                                          const fa_paged_attention_shape *shape,
                                          const fa_paged_attention_options *options,
                                          fa_split_plan *plan = nullptr) {
  return dispatch_paged_attention_any<false>(out, query, key_cache, value_cache, block_tables,
                                             context_lens, scale, max_context_len, exp_sums,
                                             max_logits, tmp_out, shape, options, plan);
}

}  // namespace fa
