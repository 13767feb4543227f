// Reduce kernel of the split-context path: merges the per-partition softmax pieces
// (max_logits, exp_sums, tmp_out) of one (sequence, head) into the final output.
//
// Upstream: paged_attention_reduce, paged_attention_kernel_v2.hpp:957-969
//   M = max_p m_p; w_p = l_p * exp(m_p - M)            (rescale_exp_sums :736-764)
//   out = sum_p (w_p / sum_q w_q) * tmp_out[p, :]      (compute_out :771-864, collect_out :868-934)
// Only the ceil(context_len / partition_size) live partitions are read (:679,716).
//
// One wavefront per (sequence, head): lane j owns D/64 consecutive output elements, so
// every tmp_out row is read with one fully coalesced wave load; partition weights are
// computed 64 at a time, one per lane, and broadcast with lane shuffles.
#pragma once

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
};

template <int D, typename QT>
__global__ void __launch_bounds__(64) paged_attn_reduce_kernel(const ReduceParams p) {
  constexpr int EPL = D / 64;  // output elements per lane (2 or 1)
  const int lane = threadIdx.x;
  const int head = blockIdx.x;
  const int seq = blockIdx.y;
  const int ctx = min(p.context_lens[seq], p.max_context);
  if (ctx <= 0) return;
  int np = (ctx + p.partition_size - 1) / p.partition_size;
  np = min(np, p.max_num_partitions);
  const int64_t base = ((int64_t)seq * p.num_heads + head) * p.max_num_partitions;
  const float *ml = p.max_logits + base;
  const float *es = p.exp_sums + base;
  const float *tmp = p.tmp_out + base * D + lane * EPL;

  float M = -INFINITY;
  for (int q = lane; q < np; q += 64) M = fmaxf(M, ml[q]);
  M = wave_max(M);

  float acc[EPL];
#pragma unroll
  for (int e = 0; e < EPL; ++e) acc[e] = 0.f;
  float W = 0.f;
  for (int q0 = 0; q0 < np; q0 += 64) {
    const int q = q0 + lane;
    const float w_lane = (q < np) ? es[q] * __expf(ml[q] - M) : 0.f;
    W += w_lane;
    const int cnt = min(64, np - q0);
    int j = 0;
    for (; j + 4 <= cnt; j += 4) {  // four rows in flight
      float v[4][EPL];
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int e = 0; e < EPL; ++e) v[u][e] = tmp[(int64_t)(q0 + j + u) * D + e];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const float w = __shfl(w_lane, j + u);
#pragma unroll
        for (int e = 0; e < EPL; ++e) acc[e] += w * v[u][e];
      }
    }
    for (; j < cnt; ++j) {
      const float w = __shfl(w_lane, j);
#pragma unroll
      for (int e = 0; e < EPL; ++e) acc[e] += w * tmp[(int64_t)(q0 + j) * D + e];
    }
  }
  W = wave_sum(W);
  const float inv = 1.0f / W;
  char *dst = reinterpret_cast<char *>(p.out) + (((int64_t)seq * p.num_heads + head) * D + lane * EPL) * 2;
  if constexpr (EPL == 2) {
    *reinterpret_cast<uint32_t *>(dst) = pack2<QT>(acc[0] * inv, acc[1] * inv);
  } else {
    const uint32_t w = pack2<QT>(acc[0] * inv, 0.f);
    *reinterpret_cast<uint16_t *>(dst) = (uint16_t)(w & 0xffffu);
  }
}

}  // namespace fa
