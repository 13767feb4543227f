// Host launcher of the FP8-E5M2 KV-cache single-pass kernel.
//
// Upstream keeps a second copy of launcher and kernel for FP8
// (paged_attention_fp8_loop/launch_kernels_fp8_loop.h:17-175, fixed to E5M2 at
// paged_attention_fp8_loop.cpp:43) that differs from the fp16 one only in the cache
// element type and the extra `fp8_scale`.  Here the cache type is a template flag of
// the one kernel, so this launcher is the loop launcher with byte caches.
#pragma once

#include "launch_kernels_loop.h"

namespace fa {

inline fa_status dispatch_paged_attention_fp8_loop(void *out, const void *query,
                                                   const void *key_cache, const void *value_cache,
                                                   const int32_t *block_tables,
                                                   const int32_t *context_lens, float scale,
                                                   int32_t max_context_len,
                                                   const fa_paged_attention_shape *shape,
                                                   const fa_paged_attention_options *options) {
  return dispatch_paged_attention_loop_any<true>(out, query, key_cache, value_cache, block_tables,
                                                 context_lens, scale, max_context_len, shape,
                                                 options);
}

}  // namespace fa
