// KV-cache writer for gfx950: scatters the K and V rows of new tokens into the paged
// pools the decode kernels read, with FP8 E5M2 rounding in registers.
//
// Upstream builds its pools on the host with tensor casts
// (test_paged_fp8cache.py:171-203); this is the same cast (round to nearest even, overflow
// to infinity, NaN kept) and the same placement as one bandwidth-bound kernel.
//
// One thread moves 8 consecutive head-dim elements of one (token, kv head) row of K and
// of V: a 16-byte load each, a 16-byte (16-bit pool) or 8-byte (E5M2 pool) store each.
// The 16 (head 128) or 8 (head 64) threads of a row sit next to each other, so loads and
// stores of a row are one contiguous segment.
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
  float inv_scale;          // 1 / fp8_scale
  int32_t num_kv_heads;
  int32_t pieces_per_row;   // head_size / 8
  int64_t total_pieces;     // num_tokens * num_kv_heads * pieces_per_row
  int32_t block_size;
  int64_t num_slots;        // num_pool_blocks * block_size
  int64_t kv_block_bytes;   // pool strides in BYTES
  int64_t kv_token_bytes;
  int64_t kv_head_bytes;
  int64_t src_token_bytes;  // source strides in BYTES
  int64_t src_head_bytes;
};

// Two fp16 values in one dword -> their two E5M2 bytes in bits 0..7 and 16..23.
// E5M2 is binary16 cut to its top byte, so rounding to nearest even is an integer add on
// the magnitude bits: + 0x7f + (lowest kept bit).  A carry out of the mantissa moves into
// the exponent, which is exactly what rounding up to the next binade -- or to infinity --
// needs, and binary16 subnormals land on E5M2 subnormals the same way.  NaN keeps a
// non-zero mantissa (0x7f) and its sign.
__device__ __forceinline__ uint32_t e5m2_from_f16_pair(uint32_t w) {
  const uint32_t mag = w & 0x7fff7fffu;
  const uint32_t sign = (w >> 8) & 0x00800080u;
  const uint32_t odd = (mag >> 8) & 0x00010001u;
  const uint32_t rounded = ((mag + 0x007f007fu + odd) >> 8) & 0x00ff00ffu;
  const uint32_t is_nan = ((mag + 0x03ff03ffu) >> 15) & 0x00010001u;  // magnitude above 0x7c00
  const uint32_t nan_mask = is_nan * 0xffu;
  return ((rounded & ~nan_mask) | (is_nan * 0x7fu)) | sign;
}

// One fp32 value -> its E5M2 byte, rounded once (to nearest even).  Used where the value
// is not an fp16 to begin with (bf16 sources) or has been scaled, so that no second
// rounding through fp16 can creep in.
__device__ __forceinline__ uint32_t e5m2_from_f32(float f) {
  const uint32_t x = __builtin_bit_cast(uint32_t, f);
  const uint32_t sign = (x >> 24) & 0x80u;
  const uint32_t mag = x & 0x7fffffffu;
  uint32_t r;
  if (mag < 0x38800000u) {
    // below 2^-14: E5M2 subnormals are multiples of 2^-16, which is the spacing of fp32
    // in [128, 256) -- adding 128 makes the fp32 adder do the rounding
    r = __builtin_bit_cast(uint32_t, __builtin_bit_cast(float, mag) + 128.0f) - 0x43000000u;
  } else {
    // keep 2 mantissa bits: add half of the dropped 21 bits (less one, plus the lowest kept
    // bit, for ties to even), re-bias the exponent from 127 to 15
    r = (mag + 0x000fffffu + ((mag >> 21) & 1u) - (112u << 23)) >> 21;
  }
  r = mag >= 0x47800000u ? 0x7cu : r;  // 65536 and beyond, infinity included
  r = mag > 0x7f800000u ? 0x7fu : r;   // NaN
  return r | sign;
}

template <typename ST>
__device__ __forceinline__ float f32_from_half_of(uint32_t w, int hi) {
  if constexpr (std::is_same<ST, BF16>::value) {
    return __builtin_bit_cast(float, hi ? (w & 0xffff0000u) : (w << 16));
  } else {
    const f16x2 v = __builtin_bit_cast(f16x2, w);
    return (float)v[hi];
  }
}

// 8 source elements (4 dwords) -> 8 E5M2 bytes (2 dwords).
template <typename ST, bool SCALED>
__device__ __forceinline__ u32x2 e5m2_from_row_piece(u32x4 src, float mul) {
  uint32_t b[4];  // bytes of elements 2k and 2k+1 at bits 0..7 and 16..23
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    if constexpr (std::is_same<ST, F16>::value && !SCALED) {
      b[k] = e5m2_from_f16_pair(src[k]);
    } else {
      b[k] = e5m2_from_f32(f32_from_half_of<ST>(src[k], 0) * mul) |
             (e5m2_from_f32(f32_from_half_of<ST>(src[k], 1) * mul) << 16);
    }
  }
  // gather bytes 0 and 2 of b[0], b[1] into one dword, and of b[2], b[3] into the next
  u32x2 out;
  out[0] = __builtin_amdgcn_perm(b[1], b[0], 0x06040200u);
  out[1] = __builtin_amdgcn_perm(b[3], b[2], 0x06040200u);
  return out;
}

template <typename ST, bool KV8, bool SCALED>
__global__ void __launch_bounds__(256) kv_cache_write_kernel(const KvWriteParams p) {
  const int64_t piece = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (piece >= p.total_pieces) return;
  const int64_t row = piece / p.pieces_per_row;
  const int part = (int)(piece - row * p.pieces_per_row);
  const int64_t token = row / p.num_kv_heads;
  const int head = (int)(row - token * p.num_kv_heads);
  const int64_t slot = p.slot_mapping[token];
  if (slot < 0 || slot >= p.num_slots) return;  // padding token
  const int64_t block = slot / p.block_size;
  const int64_t offset = slot - block * p.block_size;

  const int64_t src = token * p.src_token_bytes + head * p.src_head_bytes + part * 16;
  const u32x4 k = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p.key + src));
  const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p.value + src));
  const int64_t dst = block * p.kv_block_bytes + offset * p.kv_token_bytes + head * p.kv_head_bytes +
                      part * (KV8 ? 8 : 16);
  if constexpr (KV8) {
    *reinterpret_cast<u32x2 *>(p.key_cache + dst) = e5m2_from_row_piece<ST, SCALED>(k, p.inv_scale);
    *reinterpret_cast<u32x2 *>(p.value_cache + dst) = e5m2_from_row_piece<ST, SCALED>(v, p.inv_scale);
  } else {
    *reinterpret_cast<u32x4 *>(p.key_cache + dst) = k;
    *reinterpret_cast<u32x4 *>(p.value_cache + dst) = v;
  }
}

}  // namespace fa
