// Compile-time tuning constants of the gfx950 kernels.  Plays the role of the
// upstream policy header (include/paged_attention_policy_v2.hpp:5-100), but the
// knobs are those of a wavefront-streaming design, not of sub-group tiling.
#pragma once

namespace fa {

// Tokens one wavefront consumes per software-pipeline step: two 16-token MFMA
// tiles of scores feed one 32-deep P.V MFMA.
constexpr int kChunkTokens = 32;
constexpr int kTileTokens = 16;

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
#define FA_LOOP_WAVES 4
#endif
#ifndef FA_SPLIT_WAVES
#define FA_SPLIT_WAVES 2
#endif
template <bool kPartitioned>
struct WavesPerGroup {
  static constexpr int value = kPartitioned ? FA_SPLIT_WAVES : FA_LOOP_WAVES;
};

// Reduce kernel: one wavefront per (sequence, head).
constexpr int kReduceThreads = 64;

}  // namespace fa
