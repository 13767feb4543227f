// Reduce kernel of the split-context path: merges the per-partition softmax pieces
// (max_logits, exp_sums, tmp_out) of one (sequence, head) into the final output.
//
// Upstream: paged_attention_reduce, paged_attention_kernel_v2.hpp:957-969
//   M = max_p m_p; w_p = l_p * exp(m_p - M)            (rescale_exp_sums :736-764)
//   out = sum_p (w_p / sum_q w_q) * tmp_out[p, :]      (compute_out :771-864, collect_out :868-934)
// Only the ceil(context_len / partition_size) live partitions are read (:679,716).
// After the segment attention kernels a partial may cover several partitions: it sits in the slot
// of the first, the others hold a mark (paged_attention_segment_policy.h); and a row of a single
// partial is left alone: the attention kernel has stored it into `out` already.
//
// One work-group of one or four wavefronts per (sequence, head).  The kernel is a chain
// of dependent memory round trips, so it is built to have as few of them as possible:
// wavefront w owns partitions w, w+NW, w+2NW, ... and requests up to 16 (4) of their tmp_out
// rows (one coalesced 512-byte row per load) together with the partition scalars, before
// anything is waited for; the weights are applied when both have arrived; with four
// wavefronts the partial sums meet in LDS.  Lane j owns D/64 consecutive output elements.
#pragma once

#ifndef FA_REDUCE_SEGMENT_ROWS
#define FA_REDUCE_SEGMENT_ROWS 4
#endif

#include "paged_attention_segment_policy.h"
#include "paged_attention_utils.h"

namespace fa {

struct ReduceParams {
  void *out;                // [S,H,D] q dtype
  const float *exp_sums;    // [S,H,NP]
  const float *max_logits;  // [S,H,NP]
  const float *tmp_out;     // [S,H,NP,D]
  const int32_t *context_lens;
  int32_t num_heads;
  int32_t max_num_partitions;
  int32_t partition_size;
  int32_t max_context;  // max_blocks_per_seq * block_size: lengths are cut to it
  int32_t num_seqs;
  int32_t num_kv_heads;
  int32_t query_len;       // query tokens per sequence: rows of out / scratch are (sequence, query token) pairs
  int32_t segment_groups;  // > 0: a segment attention kernel wrote the partials (one per piece of
                           // several partitions, into the piece's first slot, marks into the
                           // others: segment_mark); 0: one partial per partition
};

// Rows requested per wavefront and batch: 16 when every partition has a partial (dozens per
// sequence); 4 after the segment kernel, which leaves a handful per sequence -- the smaller
// register set then lets twice as many work-groups stay resident.
template <bool SEGMENTS>
constexpr int reduce_rows_in_flight() { return SEGMENTS ? FA_REDUCE_SEGMENT_ROWS : 16; }

// kReduceWaves wavefronts per (sequence, head): 4 when there are few (sequence, head)
// pairs -- the launch is then short of parallelism and each pair's rows should be in
// flight at once -- 1 when there are thousands and every wavefront slot of the GPU is
// filled anyway (no LDS, no barrier, more groups resident).
// Every live slot holds a partial (the grid form of the attention kernels).
template <int D, typename QT, int kReduceWaves>
__device__ __forceinline__ void reduce_every_partition(const ReduceParams &p) {
  constexpr bool SEGMENTS = false;
  constexpr int EPL = D / 64;  // output elements per lane (2 or 1)
  constexpr int R = reduce_rows_in_flight<SEGMENTS>();
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // one work-group per (row, head), heads fastest; a row of out and of the scratch arrays is a
  // sequence, or a (sequence, query token) pair
  const int seq = blockIdx.x / p.num_heads;
  const int head = blockIdx.x - seq * p.num_heads;
  const int64_t base = ((int64_t)seq * p.num_heads + head) * p.max_num_partitions;
  const int ctx = min(p.context_lens[p.query_len > 1 ? seq / p.query_len : seq], p.max_context);
  if (ctx <= 0) return;
  int np = (ctx + p.partition_size - 1) / p.partition_size;
  np = min(np, p.max_num_partitions);
  constexpr int stride = 1;
  const float *ml = p.max_logits + base;
  const float *es = p.exp_sums + base;
  const float *tmp = p.tmp_out + base * D + lane * EPL;

  // Partitions are handled in groups of 64 (lane q of the wavefront holds the weight of
  // partition 64g + q); inside a group the rows go out in batches of R per wavefront.
  // The first batch of rows and the scalars are requested together, before any wait.
  constexpr int BATCH = kReduceWaves * R;  // rows per batch over the whole work-group
  static_assert(64 % BATCH == 0, "a group of 64 partitions is a whole number of batches");
  float v[R][EPL];
  auto request_rows = [&](int q0) {
#pragma unroll
    for (int u = 0; u < R; ++u) {
      const int q = q0 + wave + kReduceWaves * u;
#pragma unroll
      for (int e = 0; e < EPL; ++e) v[u][e] = (q < np) ? tmp[(int64_t)q * stride * D + e] : 0.f;
    }
  };
  request_rows(0);
  // lane q keeps the scalars of partition q (first group) in registers
  const float ml0 = (lane < np) ? ml[lane * stride] : -INFINITY;
  const float es0 = (lane < np) ? es[lane * stride] : 0.f;
  float M = ml0;
  for (int q = 64 + lane; q < np; q += 64) M = fmaxf(M, ml[q * stride]);
  M = wave_max(M);
  // a row none of whose partitions saw a key (a query token placed before key 0): every
  // max is -inf and every sum 0; keep exp(m - M) finite so that the row comes out as zeros
  if (M == -INFINITY) M = 0.f;

  float acc[EPL];
#pragma unroll
  for (int e = 0; e < EPL; ++e) acc[e] = 0.f;
  float W = 0.f;
  for (int g0 = 0; g0 < np; g0 += 64) {
    const int ql = g0 + lane;
    const float w_lane = g0 == 0 ? es0 * __expf(ml0 - M)
                                 : ((ql < np) ? es[ql * stride] * __expf(ml[ql * stride] - M) : 0.f);
    W += w_lane;
    for (int b0 = 0; b0 < 64 && g0 + b0 < np; b0 += BATCH) {
      if (g0 + b0 > 0) request_rows(g0 + b0);
#pragma unroll
      for (int u = 0; u < R; ++u) {
        const float w = __shfl(w_lane, b0 + wave + kReduceWaves * u);  // 0 past the last partition
#pragma unroll
        for (int e = 0; e < EPL; ++e) acc[e] += w * v[u][e];
      }
    }
  }
  W = wave_sum(W);

  const float inv = W > 0.f ? 1.0f / W : 0.f;
  float o[EPL];
  if constexpr (kReduceWaves == 1) {
#pragma unroll
    for (int e = 0; e < EPL; ++e) o[e] = acc[e] * inv;
  } else {
    __shared__ float part[kReduceWaves][D];
#pragma unroll
    for (int e = 0; e < EPL; ++e) part[wave][lane * EPL + e] = acc[e];
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      float a = 0.f;
#pragma unroll
      for (int w = 0; w < kReduceWaves; ++w) a += part[w][lane * EPL + e];
      o[e] = a * inv;
    }
  }
  char *dst = reinterpret_cast<char *>(p.out) +
              (((int64_t)seq * p.num_heads + head) * D + lane * EPL) * 2;
  if constexpr (EPL == 2) {
    *reinterpret_cast<uint32_t *>(dst) = pack2<QT>(o[0], o[1]);
  } else {
    const uint32_t w = pack2<QT>(o[0], 0.f);
    *reinterpret_cast<uint16_t *>(dst) = (uint16_t)(w & 0xffffu);
  }
}


// Partials wherever a slot does not hold the mark of a covered slot (the segment attention kernels).
template <int D, typename QT, int kReduceWaves>
__device__ __forceinline__ void reduce_marked_partials(const ReduceParams &p) {
  constexpr bool SEGMENTS = true;
  constexpr int EPL = D / 64;  // output elements per lane (2 or 1)
  constexpr int R = reduce_rows_in_flight<SEGMENTS>();
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // one work-group per (row, head), heads fastest; a row of out and of the scratch arrays is a
  // sequence, or a (sequence, query token) pair
  const int seq = blockIdx.x / p.num_heads;
  const int head = blockIdx.x - seq * p.num_heads;
  const int64_t base = ((int64_t)seq * p.num_heads + head) * p.max_num_partitions;
  const float *ml = p.max_logits + base;
  const float *es = p.exp_sums + base;
  const float *tmp = p.tmp_out + base * D + lane * EPL;
  // The scalars of the row's first 64 slots are requested together with the length, whether or not
  // the row turns out to have that many partitions, so that one wait covers both (slots past the
  // live ones are read and dropped: they lie inside the row).
  const int first_slots = min(p.max_num_partitions, 64);
  const float ml_first = lane < first_slots ? ml[lane] : -INFINITY;
  const float es_first = lane < first_slots ? es[lane] : 0.f;
  const int ctx = min(p.context_lens[p.query_len > 1 ? seq / p.query_len : seq], p.max_context);
  if (ctx <= 0) return;
  int np = (ctx + p.partition_size - 1) / p.partition_size;
  np = min(np, p.max_num_partitions);
  // After a segment attention kernel a slot holds a partial unless it holds the mark of a slot that a
  // longer piece covers (segment_mark); after the grid form every live slot holds a partial.
  auto holds_partial = [&](int q, float m_q) { return q < np && !(SEGMENTS && is_segment_mark(m_q)); };
  if constexpr (SEGMENTS) {
    // one partial: the segment kernel has stored it into `out` as the row's result
    // (PagedAttnParams::final_out), and its tmp_out row holds nothing
    if (np == 1) return;
  }

  // Partitions are handled in groups of 64 (lane q of the wavefront holds the weight of
  // partition 64g + q).  First the maximum over all partials, and how many there are.
  float M = holds_partial(lane, ml_first) ? ml_first : -INFINITY;
  int partials = __builtin_popcountll(__ballot(holds_partial(lane, ml_first)));
  for (int g0 = 64; g0 < np; g0 += 64) {
    const float m_q = g0 + lane < np ? ml[g0 + lane] : -INFINITY;
    const bool there = holds_partial(g0 + lane, m_q);
    if (there) M = fmaxf(M, m_q);
    partials += __builtin_popcountll(__ballot(there));
  }
  if constexpr (SEGMENTS) {
    if (partials <= 1) return;  // a row that one piece covers: stored into `out` by the attention kernel
  }
  M = wave_max(M);
  // a row none of whose partitions saw a key (a query token placed before key 0): every
  // max is -inf and every sum 0; keep exp(m - M) finite so that the row comes out as zeros
  if (M == -INFINITY) M = 0.f;

  float acc[EPL];
#pragma unroll
  for (int e = 0; e < EPL; ++e) acc[e] = 0.f;
  float W = 0.f;
  int nth = 0;  // partials met so far: wavefront w takes those with nth % kReduceWaves == w
  for (int g0 = 0; g0 < np; g0 += 64) {
    const int ql = g0 + lane;
    const float m_q = g0 == 0 ? ml_first : (ql < np ? ml[ql] : -INFINITY);
    const bool there = holds_partial(ql, m_q);
    const float e_q = g0 == 0 ? es_first : (there ? es[ql] : 0.f);
    const float w_lane = there ? e_q * __expf(m_q - M) : 0.f;
    W += w_lane;
    unsigned long long todo = __ballot(there);
    while (todo) {  // wave-uniform: R rows of tmp_out per wavefront in flight at a time
      int slot[R];
      float v[R][EPL];
#pragma unroll
      for (int u = 0; u < R; ++u) {
        slot[u] = -1;
        while (todo && slot[u] < 0) {
          const int q = __builtin_ctzll(todo);
          todo &= todo - 1;
          if ((nth++ % kReduceWaves) == wave) slot[u] = q;
        }
#pragma unroll
        for (int e = 0; e < EPL; ++e) v[u][e] = slot[u] >= 0 ? tmp[(int64_t)(g0 + slot[u]) * D + e] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < R; ++u) {
        const float w = slot[u] >= 0 ? __int_as_float(__builtin_amdgcn_readlane(__float_as_int(w_lane), __builtin_amdgcn_readfirstlane(slot[u]))) : 0.f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) acc[e] += w * v[u][e];
      }
    }
  }
  W = wave_sum(W);

  const float inv = W > 0.f ? 1.0f / W : 0.f;
  float o[EPL];
  if constexpr (kReduceWaves == 1) {
#pragma unroll
    for (int e = 0; e < EPL; ++e) o[e] = acc[e] * inv;
  } else {
    __shared__ float part[kReduceWaves][D];
#pragma unroll
    for (int e = 0; e < EPL; ++e) part[wave][lane * EPL + e] = acc[e];
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      float a = 0.f;
#pragma unroll
      for (int w = 0; w < kReduceWaves; ++w) a += part[w][lane * EPL + e];
      o[e] = a * inv;
    }
  }
  char *dst = reinterpret_cast<char *>(p.out) +
              (((int64_t)seq * p.num_heads + head) * D + lane * EPL) * 2;
  if constexpr (EPL == 2) {
    *reinterpret_cast<uint32_t *>(dst) = pack2<QT>(o[0], o[1]);
  } else {
    const uint32_t w = pack2<QT>(o[0], 0.f);
    *reinterpret_cast<uint16_t *>(dst) = (uint16_t)(w & 0xffffu);
  }
}

template <int D, typename QT, int kReduceWaves, bool SEGMENTS = false>
__global__ void __launch_bounds__(kReduceWaves * 64) paged_attn_reduce_kernel(const ReduceParams p) {
  if constexpr (SEGMENTS) reduce_marked_partials<D, QT, kReduceWaves>(p);
  else reduce_every_partition<D, QT, kReduceWaves>(p);
}

}  // namespace fa
