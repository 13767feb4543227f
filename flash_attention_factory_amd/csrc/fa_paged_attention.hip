// extern "C" surface of libfa_paged_attention.so: four decode entry points, one per host
// launcher, declared in include/fa_paged_attention.h, and the KV-cache writer declared in
// include/fa_kv_cache.h.
#include "../../include/fa_kv_cache.h"
#include "../../include/fa_paged_attention.h"

#include "launch_kernels_fp8_loop.h"
#include "launch_kernels_fp8_reduce.h"
#include "launch_kernels_loop.h"
#include "launch_kernels_reduce.h"
#include "launch_kv_cache_write.h"

#define FA_EXPORT extern "C" __attribute__((visibility("default")))

FA_EXPORT int32_t fa_paged_attention_loop(void *out, const void *query, const void *key_cache,
                                          const void *value_cache, const int32_t *block_tables,
                                          const int32_t *context_lens, float scale,
                                          int32_t max_context_len,
                                          const fa_paged_attention_shape *shape,
                                          const fa_paged_attention_options *options) {
  return fa::dispatch_paged_attention_loop(out, query, key_cache, value_cache, block_tables,
                                           context_lens, scale, max_context_len, shape, options);
}

FA_EXPORT int32_t fa_paged_attention_reduce(void *out, const void *query, const void *key_cache,
                                            const void *value_cache, const int32_t *block_tables,
                                            const int32_t *context_lens, float scale,
                                            int32_t max_context_len, float *exp_sums,
                                            float *max_logits, float *tmp_out,
                                            const fa_paged_attention_shape *shape,
                                            const fa_paged_attention_options *options) {
  return fa::dispatch_paged_attention(out, query, key_cache, value_cache, block_tables,
                                      context_lens, scale, max_context_len, exp_sums, max_logits,
                                      tmp_out, shape, options);
}

FA_EXPORT int32_t fa_paged_attention_fp8_loop(void *out, const void *query, const void *key_cache,
                                              const void *value_cache,
                                              const int32_t *block_tables,
                                              const int32_t *context_lens, float scale,
                                              int32_t max_context_len,
                                              const fa_paged_attention_shape *shape,
                                              const fa_paged_attention_options *options) {
  return fa::dispatch_paged_attention_fp8_loop(out, query, key_cache, value_cache, block_tables,
                                               context_lens, scale, max_context_len, shape,
                                               options);
}

FA_EXPORT int32_t fa_paged_attention_fp8_reduce(void *out, const void *query,
                                                const void *key_cache, const void *value_cache,
                                                const int32_t *block_tables,
                                                const int32_t *context_lens, float scale,
                                                int32_t max_context_len, float *exp_sums,
                                                float *max_logits, float *tmp_out,
                                                const fa_paged_attention_shape *shape,
                                                const fa_paged_attention_options *options) {
  return fa::dispatch_paged_attention_fp8(out, query, key_cache, value_cache, block_tables,
                                          context_lens, scale, max_context_len, exp_sums,
                                          max_logits, tmp_out, shape, options);
}

FA_EXPORT int32_t fa_kv_cache_write(const void *key, const void *value, void *key_cache,
                                    void *value_cache, const int64_t *slot_mapping,
                                    const fa_kv_cache_write_shape *shape,
                                    const fa_paged_attention_options *options) {
  return fa::launch_kv_cache_write(key, value, key_cache, value_cache, slot_mapping, shape, options);
}

FA_EXPORT const char *fa_last_error(void) { return fa::error_buffer(); }

FA_EXPORT int32_t fa_paged_attention_abi_version(void) { return 5; }
