// Compile-time tuning constants of the gfx950 kernels.  Plays the role of the
// upstream policy header (include/paged_attention_policy_v2.hpp:5-100), but the
// knobs are those of a wavefront-streaming design, not of sub-group tiling.
// Every default below is the measured best on MI355X; each can be overridden with -D
// for experiments.
#pragma once

namespace fa {

// One MFMA score tile covers 16 tokens; a chunk -- the unit of the software pipeline of
// one wavefront -- is 2 or 4 tiles (two tiles of scores feed one 32-deep P.V MFMA).
// Partition boundaries must fall on chunk boundaries of the largest chunk.
constexpr int kTileTokens = 16;
constexpr int kMaxChunkTokens = 64;

// Upstream partition sizes: 512 tokens for head size 128, 256 for head size 64
// (paged_attention_policy_v2.hpp:28,50; the tests mirror it, test_paged.py:411-412).
constexpr int default_partition_size(int head_size) { return head_size == 64 ? 256 : 512; }

// Query heads sharing one kv head are packed as the 16 columns of an MFMA tile.
constexpr int kMaxGroup = 16;

// ---- grid-form kernels (any batch size) ----------------------------------------------
// Wavefronts per work-group.
//  * loop kernel: one work-group owns a whole (sequence, kv head); its wavefronts
//    interleave chunks and merge once at the end through LDS.
//  * split kernel: one work-group owns one partition of one (sequence, kv head).
#ifndef FA_LOOP_WAVES
#define FA_LOOP_WAVES 8
#endif
#ifndef FA_SPLIT_WAVES
#define FA_SPLIT_WAVES 1
#endif
template <bool kPartitioned>
struct WavesPerGroup {
  static constexpr int value = kPartitioned ? FA_SPLIT_WAVES : FA_LOOP_WAVES;
};

// Per cache type: wavefronts per SIMD the register allocator must fit (4 SIMDs per CU),
// tiles per chunk, and whether K/V loads are marked non-temporal (the bytes are read once
// per launch).  Non-temporal loads measured +4..5 % on 16-bit caches in both paths and
// +10 % on the FP8 loop path, but -3 % on the grid form of the FP8 split path.
#ifndef FA_OCC
#define FA_OCC 3
#endif
#ifndef FA_OCC_FP8
#define FA_OCC_FP8 FA_OCC
#endif
#ifndef FA_TPC
#define FA_TPC 2
#endif
#ifndef FA_TPC_FP8
#define FA_TPC_FP8 2
#endif
#ifndef FA_STREAM_LOADS
#define FA_STREAM_LOADS 1
#endif
#ifndef FA_STREAM_LOADS_FP8_LOOP
#define FA_STREAM_LOADS_FP8_LOOP 1
#endif
#ifndef FA_STREAM_LOADS_FP8_SPLIT
#define FA_STREAM_LOADS_FP8_SPLIT 0
#endif
// Loop kernels on a 16-bit cache whose token rows lie next to each other (a block of one kv head
// is contiguous): whole-line K loads (WaveAttn::kRowLoads) measured 1 % slower there, and 3-12 %
// faster everywhere else (FP8 caches, the split path, rows that lie kv_heads rows apart).
#ifndef FA_K_ROW_LOADS_LOOP16_ADJACENT
#define FA_K_ROW_LOADS_LOOP16_ADJACENT 0
#endif
constexpr bool kRowLoadsLoop16Adjacent = FA_K_ROW_LOADS_LOOP16_ADJACENT != 0;

// FP8 caches with token rows of 64 bytes (head size 64) whose kv heads lie next to each other in
// memory: take two kv heads as one row of 128 bytes (WaveAttn::kPairable).  Every cache line is
// then fetched by one work-group instead of two.
#ifndef FA_PAIR_HEADS
#define FA_PAIR_HEADS 1
#endif
constexpr bool kPairHeads = FA_PAIR_HEADS != 0;

template <bool kKV8>
struct Pipeline {
  static constexpr int occ = kKV8 ? FA_OCC_FP8 : FA_OCC;
  static constexpr int tiles_per_chunk = kKV8 ? FA_TPC_FP8 : FA_TPC;
  static constexpr bool stream_loads_loop = (kKV8 ? FA_STREAM_LOADS_FP8_LOOP : FA_STREAM_LOADS) != 0;
  static constexpr bool stream_loads_split = (kKV8 ? FA_STREAM_LOADS_FP8_SPLIT : FA_STREAM_LOADS) != 0;
};

// Loop kernel that holds two column tiles per wavefront (paged_attention_loop_two_tile_kernel.h):
// one work-group per compute unit, so each wavefront has to keep more bytes in flight by itself.
#ifndef FA_TWO_TILE_TPC
#define FA_TWO_TILE_TPC 2
#endif
#ifndef FA_TWO_TILE_TPC_FP8
#define FA_TWO_TILE_TPC_FP8 FA_TPC_FP8
#endif
template <bool kKV8>
struct TwoTile {
  static constexpr int tiles_per_chunk = kKV8 ? FA_TWO_TILE_TPC_FP8 : FA_TWO_TILE_TPC;
};

// ---- persistent kernels (batches of up to 128 / 256 sequences) -------------------------
// Split path, segment form: multi-wavefront work-groups take segments of several partitions
// and write one partial per segment (paged_attention_segment_kernel.h).
#ifndef FA_SPLIT_SEGMENT
#define FA_SPLIT_SEGMENT 1
#endif
#ifndef FA_SPLIT_SEGMENT_FP8
#define FA_SPLIT_SEGMENT_FP8 FA_SPLIT_SEGMENT
#endif
#ifndef FA_SEGMENT_WAVES
#define FA_SEGMENT_WAVES 4
#endif
#ifndef FA_SEGMENT_OCC
#define FA_SEGMENT_OCC 2
#endif
#ifndef FA_SEGMENT_STREAM_LOADS
#define FA_SEGMENT_STREAM_LOADS 1
#endif
template <bool kKV8>
struct SegmentSplit {
  static constexpr bool use = (kKV8 ? FA_SPLIT_SEGMENT_FP8 : FA_SPLIT_SEGMENT) != 0;
  static constexpr int waves = FA_SEGMENT_WAVES;
  static constexpr int occ = FA_SEGMENT_OCC;
  // non-temporal K/V loads, as in the loop kernels (long streaming runs per wavefront):
  // measured +5 % with an FP8 cache
  static constexpr bool stream_loads = FA_SEGMENT_STREAM_LOADS != 0;
};

// Loop path: resident work-groups walk the (sequence, kv head) items, longest first.
#ifndef FA_PERSISTENT_LOOP
#define FA_PERSISTENT_LOOP 1
#endif
constexpr bool kUsePersistentLoop = FA_PERSISTENT_LOOP != 0;
// Its work-group size and register budget: it keeps the next item's first chunk in
// flight across the merge, so it needs more registers than the grid form.
#ifndef FA_PLOOP_WAVES
#define FA_PLOOP_WAVES 4
#endif
#ifndef FA_PLOOP_OCC
#define FA_PLOOP_OCC 2
#endif
#ifndef FA_PLOOP_WAVES_FP8
#define FA_PLOOP_WAVES_FP8 FA_PLOOP_WAVES
#endif
#ifndef FA_PLOOP_OCC_FP8
#define FA_PLOOP_OCC_FP8 FA_PLOOP_OCC
#endif
template <bool kKV8>
struct PersistentLoop {
  static constexpr int waves = kKV8 ? FA_PLOOP_WAVES_FP8 : FA_PLOOP_WAVES;
  static constexpr int occ = kKV8 ? FA_PLOOP_OCC_FP8 : FA_PLOOP_OCC;
  // Batches beyond what the kernel ranks in one launch: cut into sub-batches (one persistent
  // launch each), or left to the grid form?  Measured with 512 sequences of 512-2048 tokens:
  // 16-bit caches 82.4 % of peak in sub-batches against 80.2 % in the grid form; FP8 caches,
  // whose launches are half as long and so pay the fixed costs twice, 77.8 % against 79.6 %.
  static constexpr bool sub_batches = !kKV8;
};

// ---- reduce kernel ---------------------------------------------------------------------
// One wavefront per (sequence, head) from this many pairs on, four below.
#ifndef FA_REDUCE_1W_MIN_PAIRS
#define FA_REDUCE_1W_MIN_PAIRS 4096
#endif
constexpr int kReduceSingleWaveMinPairs = FA_REDUCE_1W_MIN_PAIRS;

}  // namespace fa
