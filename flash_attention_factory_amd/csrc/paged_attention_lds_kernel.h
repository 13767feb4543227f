// Grid-form attention kernel with K and V staged through LDS (FP8 caches, head size 128).
//
// Same work decomposition, arithmetic and results as paged_attn_kernel (paged_attention_kernel.h);
// what differs is how K/V bytes travel.  There a wavefront loads its operands into registers;
// here it copies whole 128-byte token rows from HBM straight into LDS with
// global_load_lds_dwordx4 (no registers in between, every instruction covers eight whole rows)
// into a ring of two chunk buffers of its own, and reads them back in MFMA operand layout:
//   chunk n+1 and, once chunk n's buffer is free, chunk n+2 are in flight while chunk n is
//   computed: 8-16 KiB per wavefront against 4-8 KiB of the register pipeline.
// LDS image of a 16-token tile: row-major, row t at t * 128, its eight 16-byte pieces stored at
// slot (piece ^ (t & 7)) so that the operand reads (lane 16r+i: row i, or rows 4r+e) spread over
// all banks.  A direct-to-LDS load writes lane l's 16 bytes at instruction base + 16 l, so the
// swizzle is made by choosing which global piece each lane fetches.
//
// The wavefront waits for its own copies with s_waitcnt vmcnt and reads only what it copied
// itself, so there is no barrier in the streaming loop; the buffers are handed to the final merge
// after one barrier at the end.
#pragma once

#include "paged_attention_kernel.h"

namespace fa {

typedef __attribute__((address_space(3))) void lds_void_t;
typedef __attribute__((address_space(3))) char lds_char_t;

// LDS address (byte offset inside the work-group's allocation) of a generic pointer into __shared__
__device__ __forceinline__ uint32_t lds_offset(const void *p) {
  return (uint32_t)(uintptr_t)((lds_char_t *)p);
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit field");
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// LDS reads the compiler does not see as such: it would otherwise wait for every outstanding
// direct-to-LDS copy (the prefetched chunks included) before each of them.
template <int OFFSET>
__device__ __forceinline__ u32x4 lds_read_b128(uint32_t addr) {
  u32x4 v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFFSET) : "memory");
  return v;
}
template <int OFFSET>
__device__ __forceinline__ u32x2 lds_read_b64(uint32_t addr) {
  u32x2 v;
  asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFFSET) : "memory");
  return v;
}

template <int D, typename QT, int KVF, bool PART, int NW, int OCC>
__global__ void __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(OCC)))
paged_attn_lds_kernel(const PagedAttnParams p) {
  // the compute half is WaveAttn's, on a register image filled from LDS in post-exchange layout
  using W = WaveAttn<D, QT, KVF, 2, false, false, false>;
  using Chunk = typename W::Chunk;
  using Ids = typename W::Ids;
  static_assert(KVF != kKv16 && D == 128, "built for 128-byte token rows");
  constexpr int CT = W::CT;                 // 32 tokens per chunk
  constexpr int TILE_BYTES = 16 * 128;      // one 16-token tile of K or of V
  constexpr int CHUNK_BYTES = 4 * TILE_BYTES;  // K tiles 0,1 then V tiles 0,1
  constexpr int KI = 4, VI = 4;             // direct-to-LDS loads per chunk: K, V
  constexpr int MERGE_BYTES = NW > 1 ? NW * (W::NR * 64 + 32) * 4 : 0;
  constexpr int RING_BYTES = NW * 2 * CHUNK_BYTES;
  __shared__ __attribute__((aligned(1024))) char smem[RING_BYTES > MERGE_BYTES ? RING_BYTES : MERGE_BYTES];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int kvh = blockIdx.x;
  const int part = blockIdx.y;
  const int seq = blockIdx.z;

  W wa(p, lane);
  const int r = wa.r, i = wa.i;
  const int tok_begin = PART ? part * p.partition_size : 0;
  const int c_begin = tok_begin / CT;
  const int32_t *table = p.block_tables + (int64_t)seq * p.max_blocks_per_seq;
  const int ctx = min(p.context_lens[seq], p.max_blocks_per_seq << p.block_shift);
  const int tok_end = PART ? min(ctx, tok_begin + p.partition_size) : ctx;
  if (tok_begin >= tok_end) return;  // empty partition / empty sequence: nothing is written
  const int c_end = (tok_end + CT - 1) / CT;
  const bool pool_known = p.max_block_id != INT32_MAX;
  const int last_blk = pool_known ? p.max_blocks_per_seq - 1 : (ctx - 1) >> p.block_shift;

  wa.load_q(seq, kvh);
  wa.reset(wa.load_sink(kvh, wave == 0 && (!PART || part == 0)));

  char *ring = smem + wave * 2 * CHUNK_BYTES;
  // what this lane copies: row lane >> 3 of each group of eight rows, piece (lane & 7) ^ (row & 7)
  const int copy_row = lane >> 3;
  const int64_t copy_off = (int64_t)copy_row * p.kv_token_bytes + (((lane & 7) ^ (copy_row & 7)) * 16);
  // whole chunk `ci` -> ring buffer `b`
  auto issue = [&](int ci, int b, const Ids &ids) {
    char *dst = ring + b * CHUNK_BYTES;
#pragma unroll
    for (int kv = 0; kv < 2; ++kv) {
      const char *pool = kv == 0 ? p.key_cache : p.value_cache;
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const char *src = pool + wa.tile_offset(kvh, ci, t, ids) + copy_off;
#pragma unroll
        for (int h = 0; h < 2; ++h)
          __builtin_amdgcn_global_load_lds(reinterpret_cast<const u32x4 *>(src + (int64_t)(8 * h) * p.kv_token_bytes),
                                           (lds_void_t *)(dst + (kv * 2 + t) * TILE_BYTES + h * 1024), 16, 0,
                                           /*non-temporal*/ 2);
      }
    }
  };
  // LDS -> the register image WaveAttn computes on
  auto fill_k = [&](Chunk &R, int b) {
    const uint32_t base = lds_offset(ring + b * CHUNK_BYTES) + i * 128;
    const uint32_t a0 = base + ((r ^ (i & 7)) * 16), a1 = base + (((4 + r) ^ (i & 7)) * 16);
    R.k[0][0] = lds_read_b128<0>(a0);
    R.k[0][1] = lds_read_b128<0>(a1);
    R.k[1][0] = lds_read_b128<TILE_BYTES>(a0);
    R.k[1][1] = lds_read_b128<TILE_BYTES>(a1);
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(R.k[0][0]), "+v"(R.k[0][1]), "+v"(R.k[1][0]), "+v"(R.k[1][1])::"memory");
  };
  auto fill_v = [&](Chunk &R, int b) {
    const uint32_t base = lds_offset(ring + b * CHUNK_BYTES) + 2 * TILE_BYTES + (i & 1) * 8;
    u32x2 v[8];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int row = 4 * r + e;
      const uint32_t a = base + row * 128 + (((i >> 1) ^ (row & 7)) * 16);
      v[e] = lds_read_b64<0>(a);
      v[4 + e] = lds_read_b64<TILE_BYTES>(a);
    }
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7])::"memory");
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      R.v[e][0] = v[e][0];
      R.v[e][1] = v[e][1];
    }
  };

  int ci = c_begin + wave;
  if (ci < c_end) {
    Chunk R;
    issue(ci, 0, wa.fetch_ids(table, ci, last_blk));
    if (ci + NW < c_end) issue(ci + NW, 1, wa.fetch_ids(table, ci + NW, last_blk));
    Ids nids = wa.fetch_ids(table, ci + 2 * NW, last_blk);  // of the chunk issued next
    int b = 0;
    for (; ci < c_end; ci += NW, b ^= 1) {
      const bool has_next = ci + NW < c_end;  // chunk ci + NW is in flight behind this one
      if (has_next) wait_vmcnt<VI + KI + VI>(); else wait_vmcnt<VI>();
      fill_k(R, b);
      const auto s = wa.qk(R);
      if (has_next) wait_vmcnt<KI + VI>(); else wait_vmcnt<0>();
      fill_v(R, b);
      if (has_next) {
        wa.pv(R, wa.template soft<false>(R, s, ci, tok_end));
        if (ci + 2 * NW < c_end) {  // the buffer just read takes the chunk after next
          issue(ci + 2 * NW, b, nids);
          nids = wa.fetch_ids(table, ci + 3 * NW, last_blk);
        }
      } else {
        wa.pv(R, wa.template soft<true>(R, s, ci, tok_end));  // only a wavefront's last chunk can pass the end
      }
    }
  }
  if constexpr (NW > 1) __syncthreads();  // every wavefront is through with its ring: the merge may have it
  merge_and_store<PART, NW>(wa, p, lane, wave, seq, kvh, part, reinterpret_cast<float *>(smem));
}

}  // namespace fa
