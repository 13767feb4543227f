// How the segment form of the split path cuts sequences: shared by the attention kernel
// that writes one partial per segment (paged_attention_segment_kernel.h) and the reduce
// kernel that reads them (paged_attention_reduce_kernel.h) -- both evaluate the same
// function on the same context lengths, so they agree on where the partials lie.
#pragma once

#include "paged_attention_utils.h"

namespace fa {

constexpr int kSegmentMaxSeqs = 256;
constexpr int kSegmentMaxContext = 1 << 23;  // lengths are packed into 23 bits of a sort key
// Segments aimed at per resident work-group, and the most partitions one may span.  Measured
// on the long-context and the serving-mix configurations: 2 beats 1 (the long-context batch
// loses 12 %), 3, 4 and 8 (the serving mix loses 3, 15 and 16 %: every segment costs a
// merge, a scattered partial and a restart of the stream).
#ifndef FA_SEGMENT_ITEMS
#define FA_SEGMENT_ITEMS 2
#endif
#ifndef FA_SEGMENT_MAX_PARTS
#define FA_SEGMENT_MAX_PARTS 64
#endif
constexpr int kSegmentItemsPerGroup = FA_SEGMENT_ITEMS;
constexpr int kSegmentMaxPartitions = FA_SEGMENT_MAX_PARTS;

// How many partitions one segment spans.  total_partitions: live partitions of all
// sequences; groups: work-groups of the attention launch.
__device__ __forceinline__ int partitions_per_segment(int total_partitions, int num_kv_heads, int groups) {
  const long long items = (long long)total_partitions * num_kv_heads;
  const long long m = items / ((long long)kSegmentItemsPerGroup * max(groups, 1));
  return (int)max(1LL, min(m, (long long)kSegmentMaxPartitions));
}

// Live partitions of all sequences, as every wavefront of either kernel computes them:
// lane holds sequences lane, lane+64, ...  Returns the total; per-lane counts in `parts`.
template <int NQ>
__device__ __forceinline__ int count_partitions(const int32_t *context_lens, int S, int max_ctx,
                                                int partition_size, int max_num_partitions, int lane,
                                                int (&ctxv)[NQ], int (&parts)[NQ]) {
  int local = 0;
#pragma unroll
  for (int j = 0; j < NQ; ++j) {
    const int s = lane + 64 * j;
    int c = 0;
    if (j * 64 < S) {  // wave-uniform
      if (s < S) c = max(0, min(context_lens[s], max_ctx));
    }
    ctxv[j] = c;
    parts[j] = min((c + partition_size - 1) / partition_size, max_num_partitions);
    local += parts[j];
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) local += __shfl_xor(local, o);
  return __builtin_amdgcn_readfirstlane(local);
}

}  // namespace fa
