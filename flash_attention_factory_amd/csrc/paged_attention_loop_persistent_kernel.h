// Single-pass ("loop") attention kernel, persistent form.
//
// Same results as the grid form (paged_attention_kernel.h with PART = false; upstream
// paged_attention_kernel_loop.hpp:610-636).  The grid form launches one work-group per
// (sequence, kv head); a decode batch of a few hundred such items of very different
// lengths then runs as a handful of waves of work-groups, each of which pays its own
// start-up (length -> block ids -> first K/V) and its own merge with nothing in flight.
// Here the launch holds only as many work-groups as stay resident, and each of them walks
// a list of items:
//   * items are ordered longest first (every wavefront ranks context_lens in registers)
//     and dealt to the work-groups in snake order, so the work-groups' totals are even;
//   * before a wavefront enters the merge of an item it has already requested the query
//     rows and the first K/V chunk of the next item, so its stream never drains.
// Built for up to 128 sequences; larger batches use the grid form.
#pragma once

#include "paged_attention_kernel.h"

namespace fa {

constexpr int kLoopPersistentMaxSeqs = 128;

template <int D, typename QT, bool KV8, int NW, int OCC, int TPC>
__global__ void __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(OCC)))
paged_attn_loop_persistent_kernel(const PagedAttnParams p) {
  using W = WaveAttn<D, QT, KV8, TPC, Pipeline<KV8>::stream_loads_loop>;
  using Chunk = typename W::Chunk;
  using Ids = typename W::Ids;
  constexpr int CT = W::CT;
  constexpr int NR = W::NR;
  constexpr int NDT = W::NDT;
  constexpr int SL = NR / NW;
  static_assert(NW > 1 && NR % NW == 0 && SL >= 2, "merge slices the output across wavefronts");

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int S = p.num_seqs;
  const int Hk = p.num_kv_heads;
  const int T = S * Hk;
  const int G = gridDim.x;
  const int wg = blockIdx.x;
  const int max_ctx = p.max_blocks_per_seq << p.block_shift;
  const int col_max = p.max_blocks_per_seq - 1;

  // ---- rank the sequences by length, longest first; lane holds sequences lane, lane+64 --
  int len0 = -1, len1 = -1;
  if (lane < S) len0 = max(0, min(p.context_lens[lane], max_ctx));
  if (S > 64 && lane + 64 < S) len1 = max(0, min(p.context_lens[lane + 64], max_ctx));
  int rank0 = 0, rank1 = 0;
  for (int u = 0; u < S; ++u) {
    const int lu = u < 64 ? __builtin_amdgcn_readlane(len0, u) : __builtin_amdgcn_readlane(len1, u - 64);
    rank0 += (lu > len0) || (lu == len0 && u < lane);
    rank1 += (lu > len1) || (lu == len1 && u < lane + 64);
  }

  struct Item { int seq, kvh, ctx, c_end; };
  // n-th item of this work-group: position n*G + j on even n, n*G + G-1-j on odd n
  auto item_at = [&](int n, Item &it) -> bool {
    const int pos = n * G + ((n & 1) ? G - 1 - wg : wg);
    if (pos >= T) return false;
    const int rho = __builtin_amdgcn_readfirstlane(pos / Hk);
    it.kvh = pos - rho * Hk;
    const unsigned long long b0 = __ballot(lane < S && rank0 == rho);
    const unsigned long long b1 = __ballot(lane + 64 < S && rank1 == rho);
    const int s = b0 ? __builtin_ctzll(b0) : 64 + __builtin_ctzll(b1);
    it.seq = __builtin_amdgcn_readfirstlane(s);
    it.ctx = s < 64 ? __builtin_amdgcn_readlane(len0, s) : __builtin_amdgcn_readlane(len1, s - 64);
    it.c_end = (it.ctx + CT - 1) / CT;
    return it.ctx > 0;  // sorted: nothing but empty sequences follows an empty one
  };

  __shared__ float sm_m[NW][16];
  __shared__ float sm_l[NW][16];
  __shared__ float sm_acc[NW][NR][64];

  W wa(p, lane);
  const int r = wa.r, i = wa.i;
  Chunk R;

  int n = 0;
  Item cur;
  if (!item_at(0, cur)) return;
  // first chunk of the first item
  bool armed = wave < cur.c_end;  // loads of this wavefront's first chunk of `cur` in flight
  if (armed) {
    const Ids ids = wa.fetch_ids(p.block_tables + (int64_t)cur.seq * p.max_blocks_per_seq, wave, col_max);
    wa.load_q(cur.seq, cur.kvh);
    wa.issue_k(R, cur.kvh, wave, ids);
    wa.issue_v(R, cur.kvh, wave, ids);
  }
  uint32_t sink_raw = wa.load_sink(cur.kvh, wave == 0);

  while (true) {
    Item nxt;
    const bool has_next = item_at(n + 1, nxt);
    const bool next_armed = has_next && wave < nxt.c_end;
    Ids nxt_ids = {};
    if (next_armed)
      nxt_ids = wa.fetch_ids(p.block_tables + (int64_t)nxt.seq * p.max_blocks_per_seq, wave, col_max);

    wa.reset(sink_raw);
    uint32_t next_sink = W::kNoSink;
    if (armed) {
      const int32_t *table = p.block_tables + (int64_t)cur.seq * p.max_blocks_per_seq;
      int ci = wave;
      Ids nids = wa.fetch_ids(table, ci + NW, col_max);
      while (ci + NW < cur.c_end) {  // steady state: the next chunk belongs to the same item
        const int cn = ci + NW;
        const auto s = wa.qk(R);
        wa.issue_k(R, cur.kvh, cn, nids);
        const auto pb = wa.template soft<false>(R, s, ci, cur.ctx);
        wa.pv(R, pb);
        wa.issue_v(R, cur.kvh, cn, nids);
        nids = wa.fetch_ids(table, cn + NW, col_max);
        ci = cn;
      }
      // last chunk of this wavefront in `cur`: what goes out next belongs to `nxt`
      const auto s = wa.qk(R);
      if (next_armed) {
        wa.load_q(nxt.seq, nxt.kvh);  // Q registers are free once the last scores are out
        next_sink = wa.load_sink(nxt.kvh, wave == 0);
        wa.issue_k(R, nxt.kvh, wave, nxt_ids);
      }
      const auto pb = wa.template soft<true>(R, s, ci, cur.ctx);
      wa.pv(R, pb);
      if (next_armed) wa.issue_v(R, nxt.kvh, wave, nxt_ids);
    } else if (next_armed) {  // nothing to do in `cur`, but the next item starts here
      wa.load_q(nxt.seq, nxt.kvh);
      next_sink = wa.load_sink(nxt.kvh, wave == 0);
      wa.issue_k(R, nxt.kvh, wave, nxt_ids);
      wa.issue_v(R, nxt.kvh, wave, nxt_ids);
    }

    // ---- merge the NW wavefront states of `cur`, normalise, store ----------------------
    wa.l = rows_sum(wa.l);
    if (n > 0) __syncthreads();  // the previous item's partials have been read by everyone
    if (r == 0) {
      sm_m[wave][i] = wa.m;
      sm_l[wave][i] = wa.l;
    }
#pragma unroll
    for (int k = 0; k < NR; ++k) sm_acc[wave][k][lane] = wa.acc_at(k);
    __syncthreads();
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < NW; ++w) M = fmaxf(M, sm_m[w][i]);
    float f[NW];
    float L = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float mw = sm_m[w][i];
      f[w] = (mw == -INFINITY) ? 0.f : fast_exp2(mw - M);  // a wavefront without chunks
      L += f[w] * sm_l[w][i];
    }
    float o[SL];
#pragma unroll
    for (int k = 0; k < SL; ++k) {
      float a = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) a += f[w] * sm_acc[w][wave * SL + k][lane];
      o[k] = a;
    }
    if (i < p.group) {
      const int head = cur.kvh * p.group + i;
      const int d0 = 4 * r * NDT + wave * SL;
      W::template store_q<SL>(reinterpret_cast<char *>(p.out) +
                                  (((int64_t)cur.seq * p.num_heads + head) * D + d0) * 2,
                              o, p.out_scale / L);
    }

    if (!has_next) break;
    cur = nxt;
    armed = next_armed;
    sink_raw = next_sink;
    ++n;
  }
}

}  // namespace fa
