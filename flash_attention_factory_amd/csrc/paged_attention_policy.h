// Compile-time tuning constants of the gfx950 kernels.  Plays the role of the
// upstream policy header (include/paged_attention_policy_v2.hpp:5-100), but the
// knobs are those of a wavefront-streaming design, not of sub-group tiling.
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

// Wavefronts per work-group.
//  * loop kernel: one work-group owns a whole (sequence, kv head); its wavefronts
//    interleave 32-token chunks and merge once at the end through LDS.
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

// Streaming pipeline of the attention kernel and the occupancy it is compiled for.
//   PIPE 0: two register sets, the whole next chunk in flight under the current one.
//   PIPE 1: one register set, K and V refilled separately right after their MFMAs.
//   OCC   : wavefronts per SIMD the register allocator must fit (4 SIMDs per CU).
#ifndef FA_PIPE
#define FA_PIPE 1
#endif
#ifndef FA_OCC
#define FA_OCC 3
#endif
#ifndef FA_PIPE_FP8
#define FA_PIPE_FP8 FA_PIPE
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
template <bool kKV8>
struct Pipeline {
  static constexpr int pipe = kKV8 ? FA_PIPE_FP8 : FA_PIPE;
  static constexpr int occ = kKV8 ? FA_OCC_FP8 : FA_OCC;
  static constexpr int tiles_per_chunk = kKV8 ? FA_TPC_FP8 : FA_TPC;
};

// Split path: use the persistent attention kernel when the batch allows it.
#ifndef FA_PERSISTENT_SPLIT
#define FA_PERSISTENT_SPLIT 1
#endif
constexpr bool kUsePersistentSplit = FA_PERSISTENT_SPLIT != 0;

// Longest-sequence-first assignment of sequences to work-groups (loop kernel).
#ifndef FA_LPT
#define FA_LPT 0
#endif

// Reduce kernel: four wavefronts per (sequence, head).
constexpr int kReduceThreads = 256;

}  // namespace fa
