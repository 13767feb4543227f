// Paged-attention decode kernel for gfx950 (MI355X): the single-pass "loop" form
// and the split-context "partition" form share this one template.
//
// Work decomposition (upstream: one work-group per (sequence, kv head[, partition]),
// paged_attention_kernel_loop.hpp:602-607, paged_attention_kernel_v2.hpp:562-569;
// the same here so K/V are read once per kv head):
//   grid  = (num_kv_heads, partitions or 1, num_seqs)
//   block = NW wavefronts; wavefront w takes the chunks (32 or 64 tokens) w, w+NW, ... of the
//           token range and keeps its own online-softmax state; states merge once at
//           the end through LDS.  There is no barrier inside the streaming loop.
//
// Per chunk and wavefront (the query group's G <= 16 heads are the 16 MFMA columns):
//   S^T[token, head] = K[token, :] . Q^T[:, head]      per 16-token tile: D/32 MFMA 16x16x32
//   online softmax over tokens, fp32, base 2            VALU + two cross-row shuffles
//   O^T[d, head]    += V^T[d, token] . P^T[token, head] per 32 tokens: D/16 MFMA 16x16x32
// K rows enter the MFMA "A" operand exactly as they lie in HBM (lane 16r+i loads 16 B
// of token i); V rows are loaded row-wise (16 lanes cover one token row) and
// transposed inside each lane with byte permutes, so neither needs LDS.  The scores
// come out of the first MFMA in the register layout the second MFMA wants for P^T.
//
// Arithmetic follows the upstream kernels (loop: paged_attention_kernel_loop.hpp:610-636,
// split: paged_attention_kernel_v2.hpp:572-587, FP8: paged_attention_kernel_fp8_loop.hpp:
// 328-333,540-545): fp32 scores scaled after the dot, tail tokens masked to -inf, sink
// only in the first partition, probabilities rounded to the query dtype before P.V,
// split form normalised inside the partition with (max, sum) written to scratch.
#pragma once

#include <type_traits>

#include "paged_attention_policy.h"
#include "paged_attention_utils.h"

namespace fa {

struct PagedAttnParams {
  void *out;              // loop: [S,H,D] q dtype.  split: tmp_out [S,H,NP,D] fp32
  float *exp_sums;        // split only: [S,H,NP]
  float *max_logits;      // split only: [S,H,NP]
  const void *query;      // [S,H,D]
  const char *key_cache;
  const char *value_cache;
  const int32_t *block_tables;  // [S,MB]
  const int32_t *context_lens;  // [S]
  const void *sinks;            // [H] q dtype or nullptr
  float score_scale_log2;       // sm_scale * fp8_scale * log2(e)
  float out_scale;              // fp8_scale (1 for 16-bit caches)
  int32_t num_heads;
  int32_t group;                // query heads per kv head
  int32_t max_blocks_per_seq;
  int32_t max_num_partitions;
  int32_t partition_size;       // tokens; multiple of 32
  int32_t block_shift;          // log2(block_size)
  int32_t max_block_id;         // block ids are clamped into [0, max_block_id]
  int64_t kv_block_bytes;       // strides in BYTES
  int64_t kv_token_bytes;
  int64_t kv_head_bytes;
};

// Register image of one chunk (TPC tiles of 16 tokens) of K and V in one wavefront.
template <int D, bool KV8, int TPC>
struct KVChunk {
  static constexpr int ROWB = D * (KV8 ? 1 : 2);  // bytes per token row
  static constexpr int KL = ROWB / 64;            // 16-byte K loads per lane and tile
  static constexpr int VW = ROWB / 64;            // dwords of V per lane and token
  u32x4 k[TPC][KL];
  uint32_t v[4 * TPC][VW];
};

// TPC: 16-token tiles per chunk (2 or 4).  One chunk is the unit of the software
// pipeline; 4 tiles give an FP8 cache the same bytes in flight as 2 tiles of fp16.
template <int D, typename QT, bool KV8, bool PART, int NW, int PIPE, int OCC, bool LPT, int TPC>
__global__ void __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(OCC)))
paged_attn_kernel(const PagedAttnParams p) {
  static_assert(TPC == 2 || TPC == 4, "a chunk is one or two 32-token P.V steps");
  constexpr int ROWB = D * (KV8 ? 1 : 2);
  constexpr int KL = ROWB / 64;
  constexpr int KSTEPS = D / 32;   // MFMA k-steps across the head dimension
  constexpr int NDT = D / 16;      // output d-tiles; lane row i of tile dt is d = i*NDT + dt
  constexpr int VW = ROWB / 64;
  constexpr int VB = VW * 4;       // bytes of V per lane and token
  constexpr int CT = TPC * kTileTokens;  // tokens per chunk
  constexpr int NP2 = TPC / 2;           // 32-token P.V steps per chunk
  using Chunk = KVChunk<D, KV8, TPC>;
  struct Ids { int v[TPC]; };

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane >> 4;  // 16-lane row of the wavefront
  const int i = lane & 15;  // position in the row: token (K), head (Q, P, O) or d-row (V)

  const int kvh = blockIdx.x;
  const int part = blockIdx.y;
  // Which sequence this work-group takes.  Work-groups are dispatched in blockIdx
  // order (z slowest); handing the longest sequences to the lowest z means the tail of
  // the launch is made of the shortest ones.  Every wavefront ranks the context lengths
  // by itself (no LDS, no barrier); done for up to 128 sequences, identity beyond.
  int seq = blockIdx.z;
  if constexpr (LPT) {
    const int S = gridDim.z;
    if (S > 1 && S <= 128) {
      const int len0 = lane < S ? p.context_lens[lane] : -1;
      const int len1 = lane + 64 < S ? p.context_lens[lane + 64] : -1;
      int rank0 = 0, rank1 = 0;
      for (int u = 0; u < S; ++u) {
        const int lu = u < 64 ? __builtin_amdgcn_readlane(len0, u)
                              : __builtin_amdgcn_readlane(len1, u - 64);
        rank0 += (lu > len0) || (lu == len0 && u < lane);
        rank1 += (lu > len1) || (lu == len1 && u < lane + 64);
      }
      const unsigned long long b0 = __ballot(lane < S && rank0 == (int)blockIdx.z);
      const unsigned long long b1 = __ballot(lane + 64 < S && rank1 == (int)blockIdx.z);
      seq = b0 ? __builtin_ctzll(b0) : 64 + __builtin_ctzll(b1);
      seq = __builtin_amdgcn_readfirstlane(seq);
    }
  }
  const int G = p.group;

  const int tok_begin = PART ? part * p.partition_size : 0;
  const int c_begin = tok_begin / CT;
  const int blk_mask = (1 << p.block_shift) - 1;
  const int32_t *table = p.block_tables + (int64_t)seq * p.max_blocks_per_seq;

  // Physical block id of every 16-token tile of chunk ci.  Columns are clamped to
  // `col_max` and ids into the pool, so a tile wholly past the context re-reads memory
  // that exists; it is masked later.
  auto fetch_ids = [&](int ci, int col_max) -> Ids {
    Ids ids;
#pragma unroll
    for (int t = 0; t < TPC; ++t) {
      const int col = min((ci * CT + t * kTileTokens) >> p.block_shift, col_max);
      ids.v[t] = min((uint32_t)table[col], (uint32_t)p.max_block_id);
    }
    return ids;
  };

  // Ids of this wavefront's first chunk.  When the pool size is known any column of the
  // table row is safe to read, so the ids are requested together with the context length
  // instead of after it.
  const bool pool_known = p.max_block_id != INT32_MAX;
  Ids ids0 = {};
  if (pool_known) ids0 = fetch_ids(c_begin + wave, p.max_blocks_per_seq - 1);

  // a length the block table cannot hold is cut to what it holds
  const int ctx = min(p.context_lens[seq], p.max_blocks_per_seq << p.block_shift);
  const int tok_end = PART ? min(ctx, tok_begin + p.partition_size) : ctx;
  if (tok_begin >= tok_end) return;  // empty partition / empty sequence: nothing is written

  const int c_end = (tok_end + CT - 1) / CT;
  // highest block-table column that may be read
  const int last_blk = pool_known ? p.max_blocks_per_seq - 1 : (ctx - 1) >> p.block_shift;

  // ---- Q^T as the MFMA "B" operand, one dword quad per k-step -------------------
  // k-slot (r, e) of step c stands for head-dim element qd(c, r) + e; K uses the same map.
  u32x4 qB[KSTEPS];
  {
    const int head = kvh * G + i;
    const char *qrow = reinterpret_cast<const char *>(p.query) +
                       ((int64_t)seq * p.num_heads + head) * (D * 2);
#pragma unroll
    for (int c = 0; c < KSTEPS; ++c) {
      const int d0 = KV8 ? ((c >> 1) * 4 + r) * 16 + (c & 1) * 8 : (c * 4 + r) * 8;
      u32x4 z = {0u, 0u, 0u, 0u};
      qB[c] = (i < G) ? *reinterpret_cast<const u32x4 *>(qrow + d0 * 2) : z;
    }
  }

  const char *kbase = p.key_cache + (int64_t)kvh * p.kv_head_bytes + r * 16;
  const char *vbase = p.value_cache + (int64_t)kvh * p.kv_head_bytes + i * VB;

  // ---- online softmax state, per lane ------------------------------------------------
  // m: running max (base-2 units) of head i, identical in the four rows r.
  // l: this lane's share of the running sum (its own tokens); rows are added at the end.
  // acc[dt][e]: O^T[d = (4r+e)*NDT + dt][head i], un-normalised.
  float m = -INFINITY, l = 0.f;
  f32x4 acc[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

  if (p.sinks != nullptr && wave == 0 && (!PART || part == 0) && i < G) {
    // The sink is one more logit with a zero value row; it joins partition 0 only
    // (paged_attention_kernel_loop.hpp:387-391, paged_attention_kernel_v2.hpp:373-376).
    m = load_scalar16<QT>(reinterpret_cast<const char *>(p.sinks) + (kvh * G + i) * 2) * kLog2e;
    l = (r == 0) ? 1.f : 0.f;
  }

  // Issue the K loads / the V loads of chunk ci into R (K and V go out separately so
  // that either half of the register set can be refilled as soon as it has been consumed).
  auto tile_offset = [&](int ci, int t, const Ids &ids) -> int64_t {
    return (int64_t)ids.v[t] * p.kv_block_bytes +
           (int64_t)((ci * CT + t * kTileTokens) & blk_mask) * p.kv_token_bytes;
  };
  auto issue_k = [&](Chunk &R, int ci, const Ids &ids) {
#pragma unroll
    for (int t = 0; t < TPC; ++t) {
      const char *kp = kbase + tile_offset(ci, t, ids) + (int64_t)i * p.kv_token_bytes;
#pragma unroll
      for (int c = 0; c < KL; ++c) R.k[t][c] = *reinterpret_cast<const u32x4 *>(kp + c * 64);
    }
  };
  auto issue_v = [&](Chunk &R, int ci, const Ids &ids) {
#pragma unroll
    for (int t = 0; t < TPC; ++t) {
      const char *vp = vbase + tile_offset(ci, t, ids) + (int64_t)(4 * r) * p.kv_token_bytes;
#pragma unroll
      for (int e = 0; e < 4; ++e) VLoad<VW>::ld(R.v[t * 4 + e], vp + e * p.kv_token_bytes);
    }
  };

  // K "A" operand of k-step c for one tile: row i = token, 8 head-dim elements.
  auto k_operand = [&](const Chunk &R, int tile, int c) -> u32x4 {
    if constexpr (!KV8) {
      return R.k[tile][c];
    } else {
      const u32x4 src = R.k[tile][c >> 1];
      const int h = c & 1;
      u32x4 o;
      o[0] = e5m2_adjacent_pair<QT>(src[2 * h], 0);
      o[1] = e5m2_adjacent_pair<QT>(src[2 * h], 1);
      o[2] = e5m2_adjacent_pair<QT>(src[2 * h + 1], 0);
      o[3] = e5m2_adjacent_pair<QT>(src[2 * h + 1], 1);
      return o;
    }
  };

  // V^T "A" operand of d-tile dt for the 32-token step `pr` of the chunk: row i = d-row,
  // k-slots = this lane row's 8 tokens of the step.  In-lane transpose: R.v[e] holds
  // token e's NDT consecutive head-dim elements.
  auto v_operand = [&](const Chunk &R, int pr, int dt) -> u32x4 {
    u32x4 o;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int e0 = pr * 8 + 2 * c;
      if constexpr (!KV8) {
        const uint32_t y = R.v[e0][dt >> 1], x = R.v[e0 + 1][dt >> 1];
        o[c] = (dt & 1) ? ((y >> 16) | (x & 0xffff0000u)) : ((y & 0xffffu) | (x << 16));
      } else {
        const uint32_t y = (R.v[e0][dt >> 2] >> (8 * (dt & 3))) & 0xffu;
        const uint32_t x = (R.v[e0 + 1][dt >> 2] >> (8 * (dt & 3))) & 0xffu;
        o[c] = e5m2_pair<QT>(y, x);
      }
    }
    return o;
  };

  struct Scores { f32x4 v[TPC]; };
  struct Probs { u32x4 v[NP2]; };

  // scores: S^T tile rows are tokens 4r+e of the tile, column i is the head
  auto qk = [&](const Chunk &R) -> Scores {
    Scores s;
#pragma unroll
    for (int t = 0; t < TPC; ++t) s.v[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < KSTEPS; ++c)
#pragma unroll
      for (int t = 0; t < TPC; ++t) s.v[t] = mfma_16x16x32<QT>(k_operand(R, t, c), qB[c], s.v[t]);
    return s;
  };

  // Online softmax step over the chunk's tokens; returns the P^T "B" operands.
  // `last` (compile time) marks the one chunk of a wavefront that can hold the tail of
  // the token range: only there are tokens masked and their V rows cleared.
  auto soft = [&](Chunk &R, const Scores &s, int ci, auto last) -> Probs {
    constexpr int NT = 4 * TPC;  // this lane's tokens in the chunk: tile e/4, row 4r + e%4
    float t[NT];
#pragma unroll
    for (int e = 0; e < NT; ++e) t[e] = s.v[e >> 2][e & 3] * p.score_scale_log2;
    if constexpr (decltype(last)::value) {
      const int t0 = ci * CT;
      if (t0 + CT > tok_end) {  // wave-uniform
#pragma unroll
        for (int e = 0; e < NT; ++e) {
          const int tok = t0 + (e >> 2) * kTileTokens + 4 * r + (e & 3);
          if (tok >= tok_end) {
            t[e] = -INFINITY;  // select, never multiply: the pool may hold NaN there
#pragma unroll
            for (int w = 0; w < VW; ++w) R.v[e][w] = 0u;
          }
        }
      }
    }
    float mx = t[0];
#pragma unroll
    for (int e = 1; e < NT; ++e) mx = fmaxf(mx, t[e]);
    mx = rows_max(mx);
    const float m_new = fmaxf(m, mx);
    const float alpha = fast_exp2(m - m_new);  // exp2(-inf) = 0 on the first chunk
    float ps = 0.f;
#pragma unroll
    for (int e = 0; e < NT; ++e) {
      t[e] = fast_exp2(t[e] - m_new);
      ps += t[e];
    }
    l = l * alpha + ps;
    m = m_new;
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) acc[dt] *= alpha;
    }
    // k-slots (r, e) of step pr = this lane's eight tokens of the step, rounded to the q
    // dtype (paged_attention_kernel_loop.hpp:404-407)
    Probs pb;
#pragma unroll
    for (int pr = 0; pr < NP2; ++pr)
#pragma unroll
      for (int c = 0; c < 4; ++c) pb.v[pr][c] = pack2<QT>(t[pr * 8 + 2 * c], t[pr * 8 + 2 * c + 1]);
    return pb;
  };

  auto pv = [&](const Chunk &R, const Probs &pb) {
#pragma unroll
    for (int pr = 0; pr < NP2; ++pr)
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt)
        acc[dt] = mfma_16x16x32<QT>(v_operand(R, pr, dt), pb.v[pr], acc[dt]);
  };

  using Steady = std::integral_constant<bool, false>;
  using Last = std::integral_constant<bool, true>;

  // ---- streaming loop ------------------------------------------------------------------
  // The last chunk of a wavefront is computed outside the issuing path, so no wait on the
  // loads of the current chunk ever has to cover a path on which nothing more was issued.
  int ci = c_begin + wave;
  if (ci < c_end) {
    if (!pool_known) ids0 = fetch_ids(ci, last_blk);
    if constexpr (PIPE == 1) {
      // One register set.  K of chunk n+1 is requested as soon as the score MFMAs of
      // chunk n have read K, V of chunk n+1 as soon as the P.V MFMAs have read V: about
      // half a chunk is in flight per wavefront at any time, at half the registers.
      Chunk R;
      issue_k(R, ci, ids0);
      issue_v(R, ci, ids0);
      Ids nids = fetch_ids(ci + NW, last_blk);
      while (ci + NW < c_end) {
        const int cn = ci + NW;
        const Scores s = qk(R);
        issue_k(R, cn, nids);
        const Probs pb = soft(R, s, ci, Steady{});
        pv(R, pb);
        issue_v(R, cn, nids);
        nids = fetch_ids(cn + NW, last_blk);
        ci = cn;
      }
      const Scores s = qk(R);
      pv(R, soft(R, s, ci, Last{}));
    } else {
      // Two register sets: all loads of chunk n+1 are in flight under chunk n.
      Chunk A, B;
      issue_k(A, ci, ids0);
      issue_v(A, ci, ids0);
      Ids nids = fetch_ids(ci + NW, last_blk);
      while (true) {
        int cn = ci + NW;
        if (cn >= c_end) {
          pv(A, soft(A, qk(A), ci, Last{}));
          break;
        }
        issue_k(B, cn, nids);
        issue_v(B, cn, nids);
        nids = fetch_ids(cn + NW, last_blk);
        pv(A, soft(A, qk(A), ci, Steady{}));
        ci = cn;
        cn = ci + NW;
        if (cn >= c_end) {
          pv(B, soft(B, qk(B), ci, Last{}));
          break;
        }
        issue_k(A, cn, nids);
        issue_v(A, cn, nids);
        nids = fetch_ids(cn + NW, last_blk);
        pv(B, soft(B, qk(B), ci, Steady{}));
        ci = cn;
      }
    }
  }

  l = rows_sum(l);

  // ---- merge the NW wavefront states, normalise, store -------------------------------
  // A lane's NR accumulator values are NR consecutive head-dim elements of head i:
  // d = 4r*NDT + idx with idx = e*NDT + dt.  After the merge wavefront w owns the slice
  // idx in [w*SL, (w+1)*SL) of every lane and stores it.
  constexpr int NR = NDT * 4;
  constexpr int SL = NR / NW;
  static_assert(NR % NW == 0 && SL >= 2, "output slice per wavefront must hold >= 2 elements");
  float M = m, L = l;
  float o[SL];
  if constexpr (NW == 1) {
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e * NDT + dt] = acc[dt][e];
  } else {
    __shared__ float sm_m[NW][16];
    __shared__ float sm_l[NW][16];
    __shared__ float sm_acc[NW][NR][64];
    if (r == 0) {
      sm_m[wave][i] = m;
      sm_l[wave][i] = l;
    }
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
      for (int e = 0; e < 4; ++e) sm_acc[wave][e * NDT + dt][lane] = acc[dt][e];
    __syncthreads();
    M = -INFINITY;
#pragma unroll
    for (int w = 0; w < NW; ++w) M = fmaxf(M, sm_m[w][i]);
    float f[NW];
    L = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float mw = sm_m[w][i];
      f[w] = (mw == -INFINITY) ? 0.f : fast_exp2(mw - M);  // a wavefront without chunks
      L += f[w] * sm_l[w][i];
    }
#pragma unroll
    for (int k = 0; k < SL; ++k) {
      float a = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) a += f[w] * sm_acc[w][wave * SL + k][lane];
      o[k] = a;
    }
  }

  if (i >= G) return;
  const float inv = p.out_scale / L;
  const int head = kvh * G + i;
  const int d0 = 4 * r * NDT + wave * SL;  // first head-dim element this lane stores (wave = 0 if NW == 1)
  if constexpr (PART) {
    const int64_t slot = ((int64_t)seq * p.num_heads + head) * p.max_num_partitions + part;
    float *dst = reinterpret_cast<float *>(p.out) + slot * D + d0;
    if constexpr (SL % 4 == 0) {
#pragma unroll
      for (int k = 0; k < SL; k += 4) {
        f32x4 v = {o[k] * inv, o[k + 1] * inv, o[k + 2] * inv, o[k + 3] * inv};
        *reinterpret_cast<f32x4 *>(dst + k) = v;
      }
    } else {
#pragma unroll
      for (int k = 0; k < SL; ++k) dst[k] = o[k] * inv;
    }
    if (r == 0 && wave == 0) {
      p.max_logits[slot] = M * kLn2;  // natural-log units, as upstream stores them
      p.exp_sums[slot] = L;
    }
  } else {
    char *dst = reinterpret_cast<char *>(p.out) +
                (((int64_t)seq * p.num_heads + head) * D + d0) * 2;
    uint32_t w2[SL / 2];
#pragma unroll
    for (int k = 0; k < SL / 2; ++k) w2[k] = pack2<QT>(o[2 * k] * inv, o[2 * k + 1] * inv);
    if constexpr (SL % 8 == 0) {
#pragma unroll
      for (int k = 0; k < SL / 2; k += 4) {
        u32x4 v = {w2[k], w2[k + 1], w2[k + 2], w2[k + 3]};
        *reinterpret_cast<u32x4 *>(dst + k * 4) = v;
      }
    } else if constexpr (SL % 4 == 0) {
#pragma unroll
      for (int k = 0; k < SL / 2; k += 2) {
        u32x2 v = {w2[k], w2[k + 1]};
        *reinterpret_cast<u32x2 *>(dst + k * 4) = v;
      }
    } else {
#pragma unroll
      for (int k = 0; k < SL / 2; ++k) *reinterpret_cast<uint32_t *>(dst + k * 4) = w2[k];
    }
  }
}

}  // namespace fa
