// Host launcher of the KV-cache writer (declared in include/fa_kv_cache.h).  Upstream has
// no launcher for this step -- its tests cast and place the pools with tensor operations
// (test_paged_fp8cache.py:171-203) -- so the argument checks follow the decode launchers
// of this library.
#pragma once

#include "../../include/fa_kv_cache.h"
#include "kv_cache_write_kernel.h"
#include <algorithm>

#include "launch_common.h"

namespace fa {

inline fa_status launch_kv_cache_write(const void *key, const void *value, void *key_cache,
                                       void *value_cache, const int64_t *slot_mapping,
                                       const fa_kv_cache_write_shape *s,
                                       const fa_paged_attention_options *o) {
  error_buffer()[0] = 0;
  if (!s) return fail(FA_ERR_NULL_POINTER, "shape is NULL");
  // an empty batch has nothing to point at
  if (s->num_tokens != 0 && (!key || !value || !key_cache || !value_cache || !slot_mapping))
    return fail(FA_ERR_NULL_POINTER, "key, value, key_cache, value_cache and slot_mapping must all be non-NULL");
  if (s->src_dtype != FA_DTYPE_F16 && s->src_dtype != FA_DTYPE_BF16)
    return fail(FA_ERR_UNSUPPORTED_DTYPE, "src_dtype %d is neither fp16 (0) nor bf16 (1)", s->src_dtype);
  if (s->cache_dtype != FA_KV_CACHE_16BIT && s->cache_dtype != FA_KV_CACHE_E5M2 && s->cache_dtype != FA_KV_CACHE_E4M3)
    return fail(FA_ERR_UNSUPPORTED_DTYPE, "cache_dtype %d is none of 16-bit (0), E5M2 (1), E4M3 (2)", s->cache_dtype);
  if (s->num_tokens < 0 || s->num_kv_heads <= 0 || s->block_size <= 0 || s->num_pool_blocks <= 0)
    return fail(FA_ERR_BAD_SHAPE, "num_tokens must be >= 0; num_kv_heads, block_size and num_pool_blocks positive");
  if (s->head_size <= 0 || s->head_size % 8)
    return fail(FA_ERR_UNSUPPORTED_HEAD_OR_BLOCK_SIZE, "head_size %d must be a positive multiple of 8", s->head_size);
  const bool kv8 = s->cache_dtype != FA_KV_CACHE_16BIT;
  const bool e4m3 = s->cache_dtype == FA_KV_CACHE_E4M3;
  const int64_t eb = kv8 ? 1 : 2;
  const int64_t src_head = s->src_head_stride > 0 ? s->src_head_stride : s->head_size;
  const int64_t src_token = s->src_token_stride > 0 ? s->src_token_stride : src_head * s->num_kv_heads;
  if (s->kv_block_stride <= 0 || s->kv_token_stride < s->head_size || s->kv_head_stride < s->head_size)
    return fail(FA_ERR_BAD_SHAPE, "kv strides must be positive and cover one head_size row");
  if ((s->kv_block_stride * eb) % 8 || (s->kv_token_stride * eb) % 8 || (s->kv_head_stride * eb) % 8)
    return fail(FA_ERR_BAD_SHAPE, "kv strides must be multiples of 8 bytes");
  if (!kv8 && ((s->kv_block_stride | s->kv_token_stride | s->kv_head_stride) % 8))
    return fail(FA_ERR_BAD_SHAPE, "strides of a 16-bit pool must be multiples of 16 bytes");
  if (src_head < s->head_size || src_token < s->head_size || (src_head % 8) || (src_token % 8))
    return fail(FA_ERR_BAD_SHAPE, "source strides must cover one head_size row and be multiples of 16 bytes");
  if (((uintptr_t)key | (uintptr_t)value | (uintptr_t)key_cache | (uintptr_t)value_cache) % 16 ||
      (uintptr_t)slot_mapping % 8)
    return fail(FA_ERR_BAD_SHAPE, "key, value and the pools must be 16-byte aligned, slot_mapping 8-byte aligned");
  const int scale_mode = (kv8 && o) ? o->kv_scale_mode : FA_KV_SCALE_TENSOR;
  if (scale_mode != FA_KV_SCALE_TENSOR) {
    if (scale_mode != FA_KV_SCALE_HEAD && scale_mode != FA_KV_SCALE_BLOCK)
      return fail(FA_ERR_BAD_SHAPE, "kv_scale_mode %d is none of tensor (0), head (1), block (2)", scale_mode);
    if (!o->k_scales || !o->v_scales)
      return fail(FA_ERR_NULL_POINTER, "kv_scale_mode %d needs k_scales and v_scales", scale_mode);
    if (((uintptr_t)o->k_scales | (uintptr_t)o->v_scales) % 4)
      return fail(FA_ERR_BAD_SHAPE, "k_scales and v_scales must be 4-byte aligned");
  }
  if (o && o->validate_only) return FA_OK;
  if (s->num_tokens == 0) {
    if (o && o->elapsed_us) o->elapsed_us[0] = 0.f;
    return FA_OK;
  }

  const int64_t num_slots = s->num_pool_blocks * s->block_size;
  if (num_slots > 0xffffffffLL)
    return fail(FA_ERR_BAD_SHAPE, "pools of more than 2^32 - 1 token slots are not supported");
  const int64_t pieces_per_token = (int64_t)s->num_kv_heads * (s->head_size / 8);
  if (pieces_per_token > 0x7fffffff) return fail(FA_ERR_BAD_SHAPE, "num_kv_heads * head_size is too large");

  KvWriteParams p;
  p.key = reinterpret_cast<const char *>(key);
  p.value = reinterpret_cast<const char *>(value);
  p.key_cache = reinterpret_cast<char *>(key_cache);
  p.value_cache = reinterpret_cast<char *>(value_cache);
  p.slot_mapping = slot_mapping;
  const float scale = (kv8 && o && o->fp8_scale != 0.f && scale_mode == FA_KV_SCALE_TENSOR) ? o->fp8_scale : 1.0f;
  p.inv_scale = 1.0f / scale;
  p.num_tokens = s->num_tokens;
  p.pieces_per_row = s->head_size / 8;
  p.pieces_per_token = (int32_t)pieces_per_token;
  p.tokens_per_group = (int32_t)std::max<int64_t>(1, 256 / pieces_per_token);
  p.block_size = s->block_size;
  p.block_shift = is_pow2(s->block_size) ? ilog2(s->block_size) : -1;
  p.num_slots = (uint32_t)num_slots;
  p.kv_block_bytes = s->kv_block_stride * eb;
  p.kv_token_bytes = s->kv_token_stride * eb;
  p.kv_head_bytes = s->kv_head_stride * eb;
  p.src_token_bytes = src_token * 2;
  p.src_head_bytes = src_head * 2;
  p.k_scales = scale_mode != FA_KV_SCALE_TENSOR ? o->k_scales : nullptr;
  p.v_scales = scale_mode != FA_KV_SCALE_TENSOR ? o->v_scales : nullptr;
  p.scale_block_pitch = scale_mode == FA_KV_SCALE_BLOCK ? s->num_kv_heads : 0;

  hipStream_t stream = o ? reinterpret_cast<hipStream_t>(o->stream) : nullptr;
  KernelTimer timer(o && o->elapsed_us, stream);
  // one work-group per group of tokens (the kernel strides if a grid cannot hold them all)
  const int64_t groups_needed = ((int64_t)s->num_tokens + p.tokens_per_group - 1) / p.tokens_per_group;
  const dim3 grid((unsigned)std::min<int64_t>(groups_needed, 0x7fffffff)), block(256);
  const bool bf16 = s->src_dtype == FA_DTYPE_BF16;
  const int scaled = scale_mode != FA_KV_SCALE_TENSOR ? kWriteScaleArrays
                     : scale != 1.0f                   ? kWriteScaleScalar
                                                       : kWriteUnscaled;
#define FA_KVW_LAUNCH(ST, KVF, SC) FA_HIP_CHECK(timer.launch(kv_cache_write_kernel<ST, KVF, SC>, grid, block, 0, p))
#define FA_KVW_SCALED(ST, KVF)                                             \
  do {                                                                     \
    if (scaled == kWriteScaleArrays) FA_KVW_LAUNCH(ST, KVF, kWriteScaleArrays);       \
    else if (scaled == kWriteScaleScalar) FA_KVW_LAUNCH(ST, KVF, kWriteScaleScalar);  \
    else FA_KVW_LAUNCH(ST, KVF, kWriteUnscaled);                           \
  } while (0)
  if (!kv8) {  // a 16-bit pool takes bit copies whatever the 16-bit type
    FA_KVW_LAUNCH(F16, kKv16, kWriteUnscaled);
  } else if (e4m3) {
    if (bf16) FA_KVW_SCALED(BF16, kKvE4M3); else FA_KVW_SCALED(F16, kKvE4M3);
  } else {
    if (bf16) FA_KVW_SCALED(BF16, kKvE5M2); else FA_KVW_SCALED(F16, kKvE5M2);
  }
#undef FA_KVW_SCALED
#undef FA_KVW_LAUNCH
  if (o && o->elapsed_us) FA_HIP_CHECK(timer.read(0, &o->elapsed_us[0]));
  return FA_OK;
}

}  // namespace fa
