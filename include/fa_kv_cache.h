/*
 * C ABI of the KV-cache writer of libfa_paged_attention.so: the step that runs before
 * the decode kernels of fa_paged_attention.h and produces the paged pools they read.
 *
 *   fa_kv_cache_write   scatters the K and V rows of new tokens into their slots of the
 *                       paged pools, rounding to FP8 E5M2 on the way when the pools hold
 *                       bytes.
 *
 * Upstream has this step only as test code: its tests build the paged pools on the host
 * side with tensor casts, `k_cache_paged.to(torch.float8_e5m2)`
 * (test_paged_fp8cache.py:171-203, `_generate_block_fp8kvcache`; the 16-bit pools of
 * test_paged.py:170-194 are plain copies).  The entry point below is that cast and that
 * placement as one device kernel, with the slot convention of serving engines
 * (slot = block * block_size + offset within the block).
 *
 * Shapes:
 *   key, value      [num_tokens, num_kv_heads, head_size]   src_dtype (fp16 / bf16);
 *                   element (n, h, d) = base[n*src_token_stride + h*src_head_stride + d]
 *   key_cache,      pools addressed exactly as in fa_paged_attention.h:
 *   value_cache       element(block b, token t, kv head h, dim d) =
 *                       base[b*kv_block_stride + t*kv_token_stride + h*kv_head_stride + d]
 *                     FA_KV_CACHE_16BIT: elements of src_dtype (bit copies)
 *                     FA_KV_CACHE_E5M2 : bytes, round-to-nearest-even of x / fp8_scale
 *                       (values beyond the E5M2 range become infinity, NaN stays NaN --
 *                       the behaviour of the tensor cast upstream uses)
 *                     FA_KV_CACHE_E4M3 : the same with the 1-4-3 format, whose cast turns
 *                       what lies beyond its range into NaN
 *   slot_mapping    [num_tokens] int64; token n goes to block slot / block_size, row
 *                   slot % block_size.  A negative slot, or one at or beyond
 *                   num_pool_blocks * block_size, is skipped (padding tokens).
 * Two tokens that map to the same slot race; the caller must not do that.
 */
#ifndef FA_KV_CACHE_H_
#define FA_KV_CACHE_H_

#include <stdint.h>

#include "fa_paged_attention.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef enum fa_kv_cache_dtype {
  FA_KV_CACHE_16BIT = 0,
  FA_KV_CACHE_E5M2 = 1,
  FA_KV_CACHE_E4M3 = 2 /* "fn" variant; beyond 448 becomes NaN, as torch.float8_e4m3fn casts */
} fa_kv_cache_dtype;

typedef struct fa_kv_cache_write_shape {
  uint32_t struct_size;     /* sizeof(fa_kv_cache_write_shape) in the caller's header */
  int32_t num_tokens;
  int32_t num_kv_heads;
  int32_t head_size;        /* multiple of 8 */
  int32_t block_size;       /* tokens per block, > 0 */
  int64_t kv_block_stride;  /* pool strides in elements, as in fa_paged_attention_shape */
  int64_t kv_token_stride;
  int64_t kv_head_stride;
  int64_t src_token_stride; /* key/value strides in elements; 0 = contiguous rows */
  int64_t src_head_stride;
  int32_t src_dtype;        /* fa_dtype of key and value */
  int32_t cache_dtype;      /* fa_kv_cache_dtype */
  int64_t num_pool_blocks;  /* blocks in each pool, > 0: slots outside the pool are skipped */
} fa_kv_cache_write_shape;
#define FA_KV_CACHE_WRITE_SHAPE_INIT {(uint32_t)sizeof(fa_kv_cache_write_shape)}

/* Of `options` this entry reads fp8_scale (FP8 pools only; 0 means 1.0), kv_scale_mode with
 * k_scales / v_scales (FP8 pools only: the byte stored is the rounding of x * (1 / scale), the
 * scale being that of the token's kv head or of its destination block and kv head), stream,
 * elapsed_us (1 float) and validate_only; the rest is ignored. */
int32_t fa_kv_cache_write(const void *key, const void *value, void *key_cache, void *value_cache,
                          const int64_t *slot_mapping, const fa_kv_cache_write_shape *shape,
                          const fa_paged_attention_options *options);

#ifdef __cplusplus
}
#endif

#endif /* FA_KV_CACHE_H_ */
