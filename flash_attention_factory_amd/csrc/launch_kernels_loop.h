// Host launcher and dispatcher of the single-pass ("loop") paged-attention kernel.
//
// Same role and argument list as upstream paged_attention_loop/launch_kernels_loop.h:
// launch_paged_attn_loop (:16-54) builds the launch geometry and submits one kernel,
// dispatch_paged_attention_loop (:56-173) maps the runtime (head_size, dtype) onto a
// template instance.  Block size and query-group size are runtime values here, so the
// 16-way switch of upstream collapses to head size x dtype.
#pragma once

#include <algorithm>

#include "launch_common.h"

// Persistent dot-product kernel: wavefronts per work-group, and a cap on work-groups per compute unit
// (0: as many as stay resident).  Measured on the two single-head benchmark batches (16-bit / E5M2 cache,
// us): four wavefronts and every resident work-group (three or four per unit) 104.6 / 59.5, eight
// wavefronts 104.6 / 56.4, four wavefronts and two work-groups per unit 102.4 / 56.4 -- and 101.6 / 55.3
// for the matrix-core kernel of the same schedule, which therefore stays the library's choice.
// Persistent loop kernel with eight wavefronts per work-group where a launch has work-groups for at most
// half the compute units (0: four wavefronts always).
#ifndef FA_PLOOP_WIDE
#define FA_PLOOP_WIDE 1
#endif
#ifndef FA_VALU_WAVES
#define FA_VALU_WAVES 4
#endif
// wavefronts per SIMD its registers are held to: a 16-bit cache keeps twice the bytes of a chunk in registers
#ifndef FA_VALU_OCC_16
#define FA_VALU_OCC_16 3
#endif
#ifndef FA_VALU_OCC_FP8
#define FA_VALU_OCC_FP8 4
#endif
#ifndef FA_VALU_GROUPS_PER_UNIT
#define FA_VALU_GROUPS_PER_UNIT 2
#endif

namespace fa {

// The launches of one batch that a single kernel launch can take: persistent form for up to
// kLoopPersistentMaxSeqs sequences, else grid (kv heads, 1, sequences) with NW wavefronts per
// work-group.  Kernel time is ADDED to *total_us when the call is timed.
// KVF selects the cache format: 16-bit, or E5M2 / E4M3 bytes (launch_kernels_fp8_loop.h).
template <int HEAD_SIZE, typename QT, int KVF, bool KROW>
inline fa_status launch_paged_attn_loop_rows(void *out, const void *query, const void *key_cache,
                                              const void *value_cache, const int32_t *block_tables,
                                              const int32_t *context_lens, float scale,
                                              const fa_paged_attention_shape &shape, const Resolved &r,
                                              float *total_us_out) {
  constexpr bool KV8 = KVF != kKv16;
  constexpr int NW = WavesPerGroup<false>::value;
  PagedAttnParams p = make_params(out, nullptr, nullptr, query, key_cache, value_cache,
                                  block_tables, context_lens, scale, shape, r);
  KernelTimer timer(r.elapsed_us != nullptr, r.stream);
  const int64_t items = (int64_t)shape.num_seqs * p.num_kv_heads;  // pairs of kv heads with r.pair_heads
  const int64_t max_ctx = (int64_t)shape.max_blocks_per_seq * shape.block_size;
  // score modifiers, several query tokens, per-head or per-block scales: the extended instances
  const bool ext = r.mask_flags != 0 || r.query_len > 1 || r.kv_scale_mode != 0;
  float total_us = 0.f;
  // lane dot products instead of the matrix cores (paged_attention_valu_kernel.h): groups of one head
  const bool dot_fits = HEAD_SIZE == 128 && std::is_same<QT, F16>::value && p.group == 1 && !ext && !r.pair_heads;
  const bool persistent = kUsePersistentLoop && (r.schedule == FA_SCHEDULE_AUTO || (r.schedule == FA_SCHEDULE_VALU && dot_fits)) &&
                          shape.num_seqs <= kLoopPersistentMaxSeqs && shape.num_pool_blocks > 0 &&
                          max_ctx < kLoopPersistentMaxContext;
  // One launch per group of query tokens that fit the MFMA columns (one launch for decode): 16
  // columns, or in the persistent form two tiles of 16 held by every wavefront.
  const int per_tile = p.query_count;
  const int per_launch = (persistent && r.query_len > per_tile) ? 2 * per_tile : per_tile;
  for (int q0 = 0; q0 < r.query_len; q0 += per_launch) {
    p.query_first = q0;
    p.query_count = std::min(per_launch, r.query_len - q0);
    if (persistent && r.schedule == FA_SCHEDULE_VALU) {
      if constexpr (HEAD_SIZE == 128 && std::is_same<QT, F16>::value) {
        constexpr int VW = FA_VALU_WAVES;
        auto kernel = paged_attn_valu_persistent_kernel<KVF, VW, Pipeline<KV8>::stream_loads_loop, (KV8 ? FA_VALU_OCC_FP8 : FA_VALU_OCC_16)>;
        int resident = 0, cus = 0;
        FA_HIP_CHECK(resident_groups(kernel, VW * 64, &resident, &cus));
        if (FA_VALU_GROUPS_PER_UNIT > 0) resident = std::min(resident, FA_VALU_GROUPS_PER_UNIT * cus);
        FA_HIP_CHECK(timer.launch(kernel, dim3((unsigned)std::min<int64_t>(resident, items)), dim3(VW * 64), 0, p));
      }
    } else if (persistent) {
      // Persistent form: resident work-groups walk the (sequence, kv head) items, longest
      // sequences first, with the next item's first loads issued before each merge.
      constexpr int PW = PersistentLoop<KV8>::waves;
      auto plain = paged_attn_loop_persistent_kernel<HEAD_SIZE, QT, KVF, PW, PersistentLoop<KV8>::occ,
                                                     Pipeline<KV8>::tiles_per_chunk, false, KROW>;
      auto extended = paged_attn_loop_persistent_kernel<HEAD_SIZE, QT, KVF, PW, PersistentLoop<KV8>::occ,
                                                        Pipeline<KV8>::tiles_per_chunk, true, KROW>;
      // two column tiles in the registers of every wavefront: K and V are loaded once for both
      auto two_tiles = paged_attn_loop_two_tile_kernel<HEAD_SIZE, QT, KVF, PW, TwoTile<KV8>::tiles_per_chunk, KROW>;
      auto kernel = !ext ? plain : p.query_count > per_tile ? two_tiles : extended;
      int resident = 0, cus = 0;
      FA_HIP_CHECK(resident_groups(kernel, PW * 64, &resident, &cus));
      int64_t groups = std::min<int64_t>(resident, items);
      // Pools in upstream's layout whose token rows are 128 bytes (FP8 with head size 128, 16-bit
      // with head size 64): a token's row of one kv head is a single line, and the rows of its
      // neighbours lie next to it.  A work-group then takes two adjacent kv heads of a sequence, two
      // wavefronts each, so that both lines are asked for at about the same time (the FP8 loop
      // configuration on such pools: 60.3 -> 54.2 us, what it takes on head-major pools; upstream's
      // 16-bit perf shape 39.0 -> 35.2 us).  Half as many items: unless they number twice the
      // resident work-groups, one work-group per compute unit takes them (1.5 items each would
      // leave half the work-groups waiting for the other half).  Rows of 256 bytes gain nothing.
      if constexpr (HEAD_SIZE * (KV8 ? 1 : 2) == 128) {  // token rows of 128 bytes
        // (with fewer pairs than compute units the GPU is short of work-groups, and halving their
        // number would cost more than the rows gain)
        if (!r.pair_heads && p.kv_rows_apart && shape.kv_head_stride == shape.head_size && p.num_kv_heads % 2 == 0 &&
            items / 2 >= cus) {
          if (kernel == two_tiles) {
            kernel = paged_attn_loop_two_tile_kernel<HEAD_SIZE, QT, KVF, PW, TwoTile<KV8>::tiles_per_chunk, KROW, false, 2>;
            FA_HIP_CHECK(resident_groups(kernel, PW * 64, &resident, &cus));
          } else {
            kernel = ext ? paged_attn_loop_persistent_kernel<HEAD_SIZE, QT, KVF, PW, PersistentLoop<KV8>::occ,
                                                             Pipeline<KV8>::tiles_per_chunk, true, KROW, 2>
                         : paged_attn_loop_persistent_kernel<HEAD_SIZE, QT, KVF, PW, PersistentLoop<KV8>::occ,
                                                             Pipeline<KV8>::tiles_per_chunk, false, KROW, 2>;
          }
          const int64_t pairs = items / 2;
          groups = pairs >= 2 * (int64_t)resident ? resident : std::min<int64_t>(cus, pairs);
        }
      }
      // Work-groups for at most half the compute units (a handful of sequences): the launch is bound by
      // what the few wavefronts keep in flight, and the same items with eight wavefronts per work-group keep
      // twice as much.  Measured with 1, 2 and 4 sequences of 32 heads (us, four -> eight wavefronts): byte
      // cache 17.5 -> 16.3, 17.0 -> 15.9, 18.4 -> 17.4; 16-bit cache 30.2 -> 29.4, 28.9 -> 28.6, 32.2 ->
      // 31.8.  With a work-group on every unit it is a wash or a loss (upstream's perf shape, 256 items:
      // 34.3 -> 35.0 us, byte cache 20.1 -> 20.8), and with head size 64 as well.
      int waves = PW;
      if constexpr (HEAD_SIZE == 128) {
        if (FA_PLOOP_WIDE && kernel == plain && 2 * groups <= cus) {  // (teams of two kv heads need a pair per unit)
          kernel = paged_attn_loop_persistent_kernel<HEAD_SIZE, QT, KVF, 2 * PW, PersistentLoop<KV8>::occ,
                                                     Pipeline<KV8>::tiles_per_chunk, false, KROW, 1>;
          waves = 2 * PW;
        }
      }
      const dim3 grid((unsigned)groups);
      FA_HIP_CHECK(timer.launch(kernel, grid, dim3(waves * 64), 0, p));
    } else if (KV8 && HEAD_SIZE == 128 && !ext && !r.pair_heads && r.schedule == FA_SCHEDULE_GRID_LDS) {
      // grid form, K and V staged through LDS: one work-group of eight wavefronts per compute unit
      if constexpr (KV8 && HEAD_SIZE == 128) {
        const dim3 grid(p.num_kv_heads, 1, shape.num_seqs);
        FA_HIP_CHECK(timer.launch(paged_attn_lds_kernel<HEAD_SIZE, QT, KVF, false, 8, 2>, grid, dim3(8 * 64), 0, p));
      }
    } else if (dot_fits && r.schedule == FA_SCHEDULE_GRID_VALU) {
      // grid form without the matrix cores: lane dot products, for query groups of one head
      if constexpr (HEAD_SIZE == 128 && std::is_same<QT, F16>::value) {
        const dim3 grid(p.num_kv_heads, 1, shape.num_seqs);
        FA_HIP_CHECK(timer.launch(paged_attn_valu_kernel<KVF, NW, Pipeline<KV8>::stream_loads_loop>, grid, dim3(NW * 64), 0, p));
      }
    } else if (ext) {
      const dim3 grid(p.num_kv_heads, 1, shape.num_seqs);
      FA_HIP_CHECK(timer.launch(
          paged_attn_kernel<HEAD_SIZE, QT, KVF, false, NW, Pipeline<KV8>::occ,
                            Pipeline<KV8>::tiles_per_chunk, true, KROW>,
          grid, dim3(NW * 64), 0, p));
    } else {
      const dim3 grid(p.num_kv_heads, 1, shape.num_seqs);
      FA_HIP_CHECK(timer.launch(
          paged_attn_kernel<HEAD_SIZE, QT, KVF, false, NW, Pipeline<KV8>::occ,
                            Pipeline<KV8>::tiles_per_chunk, false, KROW>,
          grid, dim3(NW * 64), 0, p));
    }
    if (r.elapsed_us) FA_HIP_CHECK(timer.accumulate(0, &total_us));
  }
  *total_us_out += total_us;
  return FA_OK;
}

// Picks how K tiles are loaded (see kRowLoadsLoop16Adjacent): whole lines, except for a 16-bit cache
// whose token rows are adjacent.
template <int HEAD_SIZE, typename QT, int KVF>
inline fa_status launch_paged_attn_loop_batch(void *out, const void *query, const void *key_cache,
                                              const void *value_cache, const int32_t *block_tables,
                                              const int32_t *context_lens, float scale,
                                              const fa_paged_attention_shape &shape, const Resolved &r,
                                              float *total_us_out) {
  if constexpr (KVF != kKv16 && HEAD_SIZE == 64) {
    if (r.pair_heads)  // pairs of kv heads as rows of 128 bytes: the head-size-128 instance
      return launch_paged_attn_loop_rows<128, QT, KVF, true>(out, query, key_cache, value_cache, block_tables,
                                                             context_lens, scale, shape, r, total_us_out);
  }
  if constexpr (KVF == kKv16 && !kRowLoadsLoop16Adjacent) {
    if (shape.kv_token_stride == shape.head_size)
      return launch_paged_attn_loop_rows<HEAD_SIZE, QT, KVF, false>(out, query, key_cache, value_cache, block_tables,
                                                                    context_lens, scale, shape, r, total_us_out);
  }
  return launch_paged_attn_loop_rows<HEAD_SIZE, QT, KVF, true>(out, query, key_cache, value_cache, block_tables,
                                                               context_lens, scale, shape, r, total_us_out);
}

// Whether the persistent kernel takes batches of this shape at all (given few enough sequences).
inline bool loop_persistent_fits(const fa_paged_attention_shape &shape) {
  return kUsePersistentLoop && shape.num_pool_blocks > 0 &&
         (int64_t)shape.max_blocks_per_seq * shape.block_size < kLoopPersistentMaxContext;
}

// A batch of more sequences than the persistent kernel ranks is cut into equal sub-batches,
// one persistent launch each, where that beats the grid form (PersistentLoop::sub_batches).
template <int HEAD_SIZE, typename QT, int KVF>
inline fa_status launch_paged_attn_loop(void *out, const void *query, const void *key_cache,
                                        const void *value_cache, const int32_t *block_tables,
                                        const int32_t *context_lens, float scale,
                                        int32_t /*max_context_len: validation only*/,
                                        const fa_paged_attention_shape &shape, const Resolved &r) {
  float total_us = 0.f;
  // most sequences one launch takes: what the persistent kernel ranks, or what the grid's third
  // dimension holds
  constexpr int kGridMaxSeqs = 65535;
  // Batches beyond what one persistent launch ranks, 16-bit cache, one query head per kv head: the grid
  // form by lane dot products (paged_attention_valu_kernel.h) beats both the sub-batches of persistent
  // launches and the grid form on the matrix cores -- 512 sequences of the Llama-7B decode shape: 1681 us
  // against 1712 and 1752, 200 sequences: 655 against 670 and 680.  (With a byte cache the two grid forms
  // time the same, 808 against 817 us, and the matrix-core one stays.)
  Resolved dot = r;
  if constexpr (KVF == kKv16 && HEAD_SIZE == 128 && std::is_same<QT, F16>::value) {
    const bool ext = r.mask_flags != 0 || r.query_len > 1 || r.kv_scale_mode != 0;
    if (r.schedule == FA_SCHEDULE_AUTO && shape.num_seqs > kLoopPersistentMaxSeqs && shape.num_heads == shape.num_kv_heads &&
        !ext && !r.pair_heads)
      dot.schedule = FA_SCHEDULE_GRID_VALU;
  }
  if (dot.schedule != r.schedule) return launch_paged_attn_loop<HEAD_SIZE, QT, KVF>(out, query, key_cache, value_cache, block_tables,
                                                                                    context_lens, scale, 0, shape, dot);
  const bool persistent_pieces = PersistentLoop<(KVF != kKv16)>::sub_batches && r.schedule == FA_SCHEDULE_AUTO &&
                                 loop_persistent_fits(shape) && shape.num_seqs > kLoopPersistentMaxSeqs;
  const int most = persistent_pieces ? kLoopPersistentMaxSeqs : kGridMaxSeqs;
  if (shape.num_seqs > most) {
    const int pieces = (shape.num_seqs + most - 1) / most;
    const int per = (shape.num_seqs + pieces - 1) / pieces;
    const int64_t row_bytes = (int64_t)r.query_len * shape.num_heads * shape.head_size * 2;  // of query and out
    for (int s0 = 0; s0 < shape.num_seqs; s0 += per) {
      fa_paged_attention_shape sub = shape;
      sub.num_seqs = std::min(per, shape.num_seqs - s0);
      const fa_status st = launch_paged_attn_loop_batch<HEAD_SIZE, QT, KVF>(
          reinterpret_cast<char *>(out) + s0 * row_bytes, reinterpret_cast<const char *>(query) + s0 * row_bytes,
          key_cache, value_cache, block_tables + (int64_t)s0 * shape.max_blocks_per_seq, context_lens + s0, scale,
          sub, r, &total_us);
      if (st != FA_OK) return st;
    }
  } else {
    const fa_status st = launch_paged_attn_loop_batch<HEAD_SIZE, QT, KVF>(
        out, query, key_cache, value_cache, block_tables, context_lens, scale, shape, r, &total_us);
    if (st != FA_OK) return st;
  }
  if (r.elapsed_us) r.elapsed_us[0] = total_us;
  return report_kernel_status(r);
}

template <bool KV8>
inline fa_status dispatch_paged_attention_loop_any(void *out, const void *query,
                                                   const void *key_cache, const void *value_cache,
                                                   const int32_t *block_tables,
                                                   const int32_t *context_lens, float scale,
                                                   int32_t max_context_len,
                                                   const fa_paged_attention_shape *shape,
                                                   const fa_paged_attention_options *options) {
  Resolved r;
  fa_status st = validate_and_resolve(out, query, key_cache, value_cache, block_tables, context_lens,
                                      max_context_len, nullptr, nullptr, nullptr, shape, options,
                                      KV8, /*split=*/false, &r);
  if (st != FA_OK || r.validate_only) return st;
  const bool bf16 = shape->q_dtype == FA_DTYPE_BF16;
#define FA_LOOP_CASE(HS, QT)                                                                      \
  do {                                                                                            \
    if (!KV8)                                                                                     \
      return launch_paged_attn_loop<HS, QT, kKv16>(out, query, key_cache, value_cache,            \
                                                   block_tables, context_lens, scale,             \
                                                   max_context_len, *shape, r);                   \
    if (r.e4m3)                                                                                   \
      return launch_paged_attn_loop<HS, QT, kKvE4M3>(out, query, key_cache, value_cache,          \
                                                     block_tables, context_lens, scale,           \
                                                     max_context_len, *shape, r);                 \
    return launch_paged_attn_loop<HS, QT, kKvE5M2>(out, query, key_cache, value_cache,            \
                                                   block_tables, context_lens, scale,             \
                                                   max_context_len, *shape, r);                   \
  } while (0)
  if (shape->head_size == 128) {
    if (bf16) FA_LOOP_CASE(128, BF16);
    FA_LOOP_CASE(128, F16);
  }
  if (bf16) FA_LOOP_CASE(64, BF16);
  FA_LOOP_CASE(64, F16);
#undef FA_LOOP_CASE
}

inline fa_status dispatch_paged_attention_loop(void *out, const void *query, const void *key_cache,
                                               const void *value_cache,
                                               const int32_t *block_tables,
                                               const int32_t *context_lens, float scale,
                                               int32_t max_context_len,
                                               const fa_paged_attention_shape *shape,
                                               const fa_paged_attention_options *options) {
  return dispatch_paged_attention_loop_any<false>(out, query, key_cache, value_cache, block_tables,
                                                  context_lens, scale, max_context_len, shape,
                                                  options);
}

}  // namespace fa
