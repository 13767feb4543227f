/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the KV-cache writer.
 *
 * The checker for fa_kv_cache_write, never the product: only tests/, the smoke check and
 * the bench's cpu_baseline leg may build, load or call it.
 *
 * What it restates: the way the upstream tests produce the pools their kernels read --
 * a tensor cast to torch.float8_e5m2 of fp16 data laid out in paged blocks
 * (test_paged_fp8cache.py:171-203 `_generate_block_fp8kvcache`; 16-bit pools are plain
 * copies, test_paged.py:170-194) -- written as the scatter serving engines use: token n
 * goes to slot_mapping[n] = block * block_size + row.
 *
 * Pinning status:
 *   oracle_f32_to_e5m2,     pinned against the torch casts (float8_e5m2, float8_e4m3fn) on
 *   oracle_f32_to_e4m3      every fp16 and every bf16 bit pattern and on fp32 values around
 *                           every rounding boundary (tests/test_oracle_kv_cache.py).
 *   oracle_kv_cache_write   pinned against a torch index_put of cast tensors, both layouts,
 *                           skipped slots included.
 *   fp8_scale != 1, scale   PARITY UNPINNED: upstream never quantises with a scale; the
 *   arrays                  reading implemented is byte = fp8(fp32(x) * (1 / scale)),
 *                           rounded once, the scale being the scalar, that of the kv head or
 *                           that of the destination block and kv head.
 */
#include <stdint.h>
#include <string.h>

#define ORACLE_API __attribute__((visibility("default")))

float oracle_f16_to_f32(uint16_t h);
float oracle_bf16_to_f32(uint16_t h);

/* fp32 -> E5M2 (1 sign, 5 exponent bits with bias 15, 2 mantissa bits), round to nearest,
 * ties to even, overflow to infinity, NaN kept (mantissa 3) with its sign. */
ORACLE_API uint8_t oracle_f32_to_e5m2(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint8_t sign = (uint8_t)((x >> 24) & 0x80u);
  uint32_t ax = x & 0x7FFFFFFFu;
  if (ax > 0x7F800000u) return (uint8_t)(sign | 0x7Fu);
  if (ax == 0x7F800000u) return (uint8_t)(sign | 0x7Cu);
  if (ax == 0) return sign;
  int32_t e = (int32_t)(ax >> 23) - 127;
  uint64_t m = (ax & 0x7FFFFFu) | 0x800000u; /* 24-bit significand, value = m * 2^(e-23) */
  if ((ax >> 23) == 0) { /* fp32 subnormal: far below half of the smallest E5M2 step */
    return sign;
  }
  /* target step: 2^(e-2) for normal results (e >= -14), 2^-16 below */
  int32_t step_exp = e >= -14 ? e - 2 : -16;
  int32_t shift = step_exp - (e - 23); /* >= 21 */
  if (shift > 40) return sign;          /* less than 2^-17 by a wide margin */
  uint64_t q = m >> shift;
  uint64_t rem = m & (((uint64_t)1 << shift) - 1);
  uint64_t half = (uint64_t)1 << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) q++;
  /* q counts steps of 2^step_exp */
  uint32_t out;
  if (e >= -14) {
    /* q in [4, 8]: 4..7 = 1.00b..1.11b, 8 = carry into the next binade */
    uint32_t be = (uint32_t)(e + 15);
    if (q == 8) {
      be += 1;
      q = 4;
    }
    if (be >= 31) return (uint8_t)(sign | 0x7Cu);
    out = (be << 2) | (uint32_t)(q - 4);
  } else {
    out = (uint32_t)q; /* 0..4; 4 is the smallest normal, encoded as exponent 1 */
  }
  return (uint8_t)(sign | out);
}

/* fp32 -> E4M3 "fn" (bias 7, 3 mantissa bits, no infinities), round to nearest, ties to
 * even; what rounds beyond the largest number 448 (that is, 480 and above) becomes NaN, as
 * the tensor cast to torch.float8_e4m3fn does; NaN is 0x7f with the sign kept. */
ORACLE_API uint8_t oracle_f32_to_e4m3(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint8_t sign = (uint8_t)((x >> 24) & 0x80u);
  uint32_t ax = x & 0x7FFFFFFFu;
  if (ax >= 0x43F00000u) return (uint8_t)(sign | 0x7Fu); /* 480 and beyond, infinity, NaN */
  if ((ax >> 23) == 0) return sign;                      /* zero and fp32 subnormals */
  int32_t e = (int32_t)(ax >> 23) - 127;
  uint64_t m = (ax & 0x7FFFFFu) | 0x800000u;
  int32_t step_exp = e >= -6 ? e - 3 : -9; /* 3 mantissa bits; subnormal step 2^-9 */
  int32_t shift = step_exp - (e - 23);
  if (shift > 40) return sign;
  uint64_t q = m >> shift;
  uint64_t rem = m & (((uint64_t)1 << shift) - 1);
  uint64_t half = (uint64_t)1 << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) q++;
  uint32_t out;
  if (e >= -6) {
    uint32_t be = (uint32_t)(e + 7);
    if (q == 16) {
      be += 1;
      q = 8;
    }
    out = (be << 3) | (uint32_t)(q - 8);
  } else {
    out = (uint32_t)q; /* 0..8; 8 is the smallest normal */
  }
  return (uint8_t)(sign | out);
}

ORACLE_API void oracle_f32_to_e4m3_array(const float *src, uint8_t *dst, int64_t n) {
  for (int64_t k = 0; k < n; ++k) dst[k] = oracle_f32_to_e4m3(src[k]);
}

ORACLE_API void oracle_f32_to_e5m2_array(const float *src, uint8_t *dst, int64_t n) {
  for (int64_t k = 0; k < n; ++k) dst[k] = oracle_f32_to_e5m2(src[k]);
}

typedef struct oracle_kv_write {
  int32_t num_tokens, num_kv_heads, head_size, block_size;
  int64_t kv_block_stride, kv_token_stride, kv_head_stride; /* elements */
  int64_t src_token_stride, src_head_stride;                /* elements */
  int32_t src_dtype;   /* 0 fp16, 1 bf16 */
  int32_t cache_dtype; /* 0 16-bit copy, 1 E5M2, 2 E4M3 */
  int64_t num_pool_blocks;
  float fp8_scale;
} oracle_kv_write;

static void write_row(const uint16_t *src, void *cache, int64_t dst, const oracle_kv_write *w, float inv) {
  if (w->cache_dtype == 0) {
    memcpy((uint16_t *)cache + dst, src, (size_t)w->head_size * 2);
    return;
  }
  uint8_t *out = (uint8_t *)cache + dst;
  for (int d = 0; d < w->head_size; ++d) {
    float x = w->src_dtype == 1 ? oracle_bf16_to_f32(src[d]) : oracle_f16_to_f32(src[d]);
    out[d] = w->cache_dtype == 2 ? oracle_f32_to_e4m3(x * inv) : oracle_f32_to_e5m2(x * inv);
  }
}

/* k_scales / v_scales NULL: the scalar w->fp8_scale.  Otherwise the scale of a row is
 * scales[b * scale_block_pitch + h]: per kv head with pitch 0, per destination block and kv
 * head with pitch num_kv_heads.  The byte is the rounding of fp32(x) * (1.0f / scale). */
ORACLE_API int oracle_kv_cache_write_scaled(const uint16_t *key, const uint16_t *value, void *key_cache,
                                            void *value_cache, const int64_t *slot_mapping,
                                            const float *k_scales, const float *v_scales,
                                            int32_t scale_block_pitch, const oracle_kv_write *w) {
  const float inv = 1.0f / (w->fp8_scale != 0.f ? w->fp8_scale : 1.0f);
  const int64_t slots = w->num_pool_blocks * w->block_size;
  for (int64_t n = 0; n < w->num_tokens; ++n) {
    const int64_t slot = slot_mapping[n];
    if (slot < 0 || slot >= slots) continue;
    const int64_t b = slot / w->block_size, t = slot % w->block_size;
    for (int h = 0; h < w->num_kv_heads; ++h) {
      const int64_t src = n * w->src_token_stride + h * w->src_head_stride;
      const int64_t dst = b * w->kv_block_stride + t * w->kv_token_stride + h * w->kv_head_stride;
      const float k_inv = k_scales ? 1.0f / k_scales[b * scale_block_pitch + h] : inv;
      const float v_inv = v_scales ? 1.0f / v_scales[b * scale_block_pitch + h] : inv;
      write_row(key + src, key_cache, dst, w, k_inv);
      write_row(value + src, value_cache, dst, w, v_inv);
    }
  }
  return 0;
}

ORACLE_API int oracle_kv_cache_write(const uint16_t *key, const uint16_t *value, void *key_cache,
                                     void *value_cache, const int64_t *slot_mapping,
                                     const oracle_kv_write *w) {
  return oracle_kv_cache_write_scaled(key, value, key_cache, value_cache, slot_mapping, NULL, NULL, 0, w);
}
