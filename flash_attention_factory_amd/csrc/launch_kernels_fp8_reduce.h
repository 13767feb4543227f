// Host launcher of the FP8-E5M2 KV-cache split-context path.
//
// Upstream: paged_attention_fp8_reduce/launch_kernels_fp8_reduce.h:16-196 -- an FP8
// attention kernel followed by the unchanged reduce kernel (:58-72).  The same holds
// here: only the partition kernel sees byte caches; the reduce kernel is shared.
#pragma once

#include "launch_kernels_reduce.h"

namespace fa {

inline fa_status dispatch_paged_attention_fp8(void *out, const void *query, const void *key_cache,
                                              const void *value_cache,
                                              const int32_t *block_tables,
                                              const int32_t *context_lens, float scale,
                                              int32_t max_context_len, float *exp_sums,
                                              float *max_logits, float *tmp_out,
                                              const fa_paged_attention_shape *shape,
                                              const fa_paged_attention_options *options,
                                              fa_split_plan *plan = nullptr) {
  return dispatch_paged_attention_any<true>(out, query, key_cache, value_cache, block_tables,
                                            context_lens, scale, max_context_len, exp_sums,
                                            max_logits, tmp_out, shape, options, plan);
}

}  // namespace fa
