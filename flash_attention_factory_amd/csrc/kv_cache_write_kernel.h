// KV-cache writer for gfx950: scatters the K and V rows of new tokens into the paged
// pools the decode kernels read, with FP8 E5M2 rounding in registers.
//
// Upstream builds its pools on the host with tensor casts
// (test_paged_fp8cache.py:171-203); this is the same cast (round to nearest even, overflow
// to infinity, NaN kept) and the same placement as one bandwidth-bound kernel.
//
// One thread moves 8 consecutive head-dim elements of one (token, kv head) row of K and
// of V: a 16-byte load each, a 16-byte (16-bit pool) or 8-byte (E5M2 pool) store each.
// The threads of a row sit next to each other, so loads and stores of a row are one
// contiguous segment.  A work-group covers 256 / (pieces per token) whole tokens, so a
// thread's place inside the token (kv head, piece of the row) costs two small divisions
// and the slot one shift.  One work-group per token group, nothing looped or unrolled:
// measured, a resident grid striding over tokens with 1, 2 or 4 tokens in flight per
// thread is 3-18 % slower -- a read stream mixed with a write stream wants less in flight,
// not more.  Nor is it the scatter that bounds the kernel: with the slots a prefill writes
// (consecutive per sequence), and with the threads laid out so that those rows go out as runs of
// 2 KiB per kv head, it takes the same 44-45 us as with random slots (built, verified, timed, not kept).
#pragma once

#include <type_traits>

#include "paged_attention_utils.h"

namespace fa {

struct KvWriteParams {
  const char *key;
  const char *value;
  char *key_cache;
  char *value_cache;
  const int64_t *slot_mapping;
  float inv_scale;            // 1 / fp8_scale
  int32_t num_tokens;
  int32_t pieces_per_row;     // head_size / 8
  int32_t pieces_per_token;   // num_kv_heads * pieces_per_row
  int32_t tokens_per_group;   // tokens one work-group covers per step: max(1, 256 / pieces_per_token)
  int32_t block_size;
  int32_t block_shift;        // log2(block_size), or -1 if block_size is no power of two
  uint32_t num_slots;         // num_pool_blocks * block_size
  int64_t kv_block_bytes;     // pool strides in BYTES
  int64_t kv_token_bytes;
  int64_t kv_head_bytes;
  int64_t src_token_bytes;    // source strides in BYTES
  int64_t src_head_bytes;
  // SCALED == kWriteScaleArrays: per kv head ([Hk], scale_block_pitch 0) or per destination
  // block and kv head ([pool blocks, Hk], scale_block_pitch Hk) fp32 scales of K and of V
  const float *k_scales;
  const float *v_scales;
  int32_t scale_block_pitch;
};

// How the writer scales before rounding: not at all, by one scalar, by scales from arrays.
constexpr int kWriteUnscaled = 0, kWriteScaleScalar = 1, kWriteScaleArrays = 2;

template <typename ST>
__device__ __forceinline__ float f32_from_half_of(uint32_t w, int hi) {
  if constexpr (std::is_same<ST, BF16>::value) {
    return __builtin_bit_cast(float, hi ? (w & 0xffff0000u) : (w << 16));
  } else {
    const f16x2 v = __builtin_bit_cast(f16x2, w);
    return (float)v[hi];
  }
}

// 8 source elements (4 dwords) -> 8 FP8 bytes (2 dwords).
// E5M2: v_cvt_pk_bf8_f32 rounds two fp32 values to nearest even, sends what lies beyond the
// range to infinity and handles subnormals -- checked against the tensor cast on every fp16
// and bf16 input -- but it has its own NaN pattern, so NaN bytes (exponent 31, mantissa not
// 0) are spotted in the result and rewritten to the cast's 0x7f | sign.
// E4M3: v_cvt_pk_fp8_f32 likewise; the format has no infinity and the cast turns everything
// that rounds beyond 448 (480 and above, NaN included) into NaN, 0x7f | sign, which is
// decided here from the inputs, whatever the instruction does with them.
template <typename ST, int KVF, int SCALED>
__device__ __forceinline__ u32x2 fp8_from_row_piece(u32x4 src, float mul) {
  float f[8];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    f[2 * k] = f32_from_half_of<ST>(src[k], 0);
    f[2 * k + 1] = f32_from_half_of<ST>(src[k], 1);
  }
  if constexpr (SCALED != kWriteUnscaled) {
#pragma unroll
    for (int k = 0; k < 8; ++k) f[k] *= mul;
  }
  u32x2 out;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    uint32_t u;
    bool fix;
    if constexpr (KVF == kKvE4M3) {
      int w = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * h], f[4 * h + 1], 0, false);
      w = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * h + 2], f[4 * h + 3], w, true);
      u = (uint32_t)w;
      // 480 and above, infinity and NaN all have magnitude bits >= those of 480.0f
      uint32_t big = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) big = max(big, __builtin_bit_cast(uint32_t, f[4 * h + e]) & 0x7fffffffu);
      fix = big >= 0x43f00000u;
    } else {
      int w = __builtin_amdgcn_cvt_pk_bf8_f32(f[4 * h], f[4 * h + 1], 0, false);
      w = __builtin_amdgcn_cvt_pk_bf8_f32(f[4 * h + 2], f[4 * h + 3], w, true);
      u = (uint32_t)w;
      // any byte with magnitude bits above 0x7c is a NaN
      fix = (((u & 0x7f7f7f7fu) + 0x03030303u) & 0x80808080u) != 0;
    }
    if (fix) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t x = __builtin_bit_cast(uint32_t, f[4 * h + e]);
        const uint32_t mag = x & 0x7fffffffu;
        const bool special = KVF == kKvE4M3 ? mag >= 0x43f00000u /* 480.0f */ : mag > 0x7f800000u /* NaN */;
        if (special) u = (u & ~(0xffu << (8 * e))) | ((0x7fu | ((x >> 24) & 0x80u)) << (8 * e));
      }
    }
    out[h] = u;
  }
  return out;
}

template <typename ST, int KVF, int SCALED>
__global__ void __launch_bounds__(256) kv_cache_write_kernel(const KvWriteParams p) {
  constexpr bool KV8 = KVF != kKv16;
  const int ppt = p.pieces_per_token;
  // place inside the group of tokens a work-group covers per step
  const int local_token = (int)threadIdx.x / ppt;  // 0 when a token has more pieces than threads
  if (local_token >= p.tokens_per_group) return;
  const int q_first = (int)threadIdx.x - local_token * ppt;
  const int64_t token_stride = (int64_t)gridDim.x * p.tokens_per_group;

  for (int q = q_first; q < ppt; q += 256) {  // one trip unless a token has more than 256 pieces
    const int head = q / p.pieces_per_row;
    const int part = q - head * p.pieces_per_row;
    const int64_t src_off = (int64_t)head * p.src_head_bytes + part * 16;
    const int64_t dst_off = (int64_t)head * p.kv_head_bytes + part * (KV8 ? 8 : 16);
    // one trip as well unless the batch needs more work-groups than a grid holds
    for (int64_t token = (int64_t)blockIdx.x * p.tokens_per_group + local_token; token < p.num_tokens;
         token += token_stride) {
      const int64_t slot = p.slot_mapping[token];
      const int64_t src = token * p.src_token_bytes + src_off;
      const u32x4 k = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p.key + src));
      const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p.value + src));
      if (slot < 0 || slot >= (int64_t)p.num_slots) continue;  // padding token
      const uint32_t s = (uint32_t)slot;
      const uint32_t block = p.block_shift >= 0 ? s >> p.block_shift : s / (uint32_t)p.block_size;
      const uint32_t row = s - block * (uint32_t)p.block_size;
      const int64_t dst = (int64_t)block * p.kv_block_bytes + (int64_t)row * p.kv_token_bytes + dst_off;
      if constexpr (KV8) {
        float k_mul = p.inv_scale, v_mul = p.inv_scale;
        if constexpr (SCALED == kWriteScaleArrays) {
          const int64_t at = (int64_t)block * p.scale_block_pitch + head;
          k_mul = 1.0f / p.k_scales[at];  // correctly rounded, as the host's 1.0f / scale
          v_mul = 1.0f / p.v_scales[at];
        }
        *reinterpret_cast<u32x2 *>(p.key_cache + dst) = fp8_from_row_piece<ST, KVF, SCALED>(k, k_mul);
        *reinterpret_cast<u32x2 *>(p.value_cache + dst) = fp8_from_row_piece<ST, KVF, SCALED>(v, v_mul);
      } else {
        *reinterpret_cast<u32x4 *>(p.key_cache + dst) = k;
        *reinterpret_cast<u32x4 *>(p.value_cache + dst) = v;
      }
    }
  }
}

}  // namespace fa
