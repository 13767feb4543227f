// Paged-attention decode kernel for gfx950 (MI355X), grid form: the single-pass "loop"
// kernel and the split-context "partition" kernel share this one template.
//
// Work decomposition (upstream: one work-group per (sequence, kv head[, partition]),
// paged_attention_kernel_loop.hpp:602-607, paged_attention_kernel_v2.hpp:562-569;
// the same here so K/V are read once per kv head):
//   grid  = (num_kv_heads, partitions or 1, num_seqs)
//   block = NW wavefronts; wavefront w takes the chunks (32 or 64 tokens) w, w+NW, ... of the
//           token range and keeps its own online-softmax state; states merge once at
//           the end through LDS.  There is no barrier inside the streaming loop.
//
// Upstream drivers restated: loop paged_attention_kernel_loop.hpp:610-636 (sink only in
// the first partition :387-391, final divide :550-586), split
// paged_attention_kernel_v2.hpp:572-587 (empty partitions write nothing :577-579,
// normalised inside the partition :386, (max, sum) to scratch :413-442, tmp_out :525-546).
#pragma once

#include "paged_attention_wave.h"

namespace fa {

// Merge the NW wavefront states of a work-group, normalise and store.
//   loop : out[seq, head, :]            = acc / L * out_scale, rounded to the q dtype
//   split: tmp_out[seq, head, part, :]  = acc / L * out_scale (fp32),
//          max_logits = M (natural-log units), exp_sums = L
// After the merge wavefront w owns the slice idx in [w*SL, (w+1)*SL) of every lane's NR
// consecutive head-dim elements and stores it.
// `lds`: NW * (NR * 64 + 32) floats of LDS the work-group is done with otherwise (unused with NW = 1).
template <bool PART, int NW, typename W>
__device__ __forceinline__ void merge_and_store(W &wa, const PagedAttnParams &p, int lane, int wave,
                                                int seq, int kvh, int part, float *lds) {
  constexpr int NR = W::NR;
  constexpr int NDT = W::NDT;
  constexpr int D = NDT * 16;
  constexpr int SL = NR / NW;
  static_assert(NR % NW == 0 && SL >= 2, "output slice per wavefront must hold >= 2 elements");
  const int r = wa.r, i = wa.i;
  wa.settle();
  wa.l = rows_sum(wa.l);
  float M = wa.m, L = wa.l;
  float o[SL];
  if constexpr (NW == 1) {
#pragma unroll
    for (int k = 0; k < SL; ++k) o[k] = wa.acc_at(k);
  } else {
    float (*sm_acc)[NR][64] = reinterpret_cast<float (*)[NR][64]>(lds);
    float (*sm_m)[16] = reinterpret_cast<float (*)[16]>(lds + NW * NR * 64);
    float (*sm_l)[16] = reinterpret_cast<float (*)[16]>(lds + NW * NR * 64 + NW * 16);
    if (r == 0) {
      sm_m[wave][i] = wa.m;
      sm_l[wave][i] = wa.l;
    }
#pragma unroll
    for (int k = 0; k < NR; ++k) sm_acc[wave][k][lane] = wa.acc_at(k);
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

  if (!wa.col_valid || !wa.keeps_output()) return;
  float out_scale = p.out_scale;
  if constexpr (W::kExt) out_scale = wa.out_mul;
  const float inv = L > 0.f ? out_scale / L : 0.f;  // L = 0: nothing visible (local window, causal rule)
  const int head = kvh * p.group + wa.col_g;
  const int64_t row = W::kExt ? (int64_t)seq * p.query_len + wa.col_q : seq;  // row of query / out / scratch
  const int d0 = wa.out_elem(4 * r * NDT + wave * SL);  // first head-dim element this lane stores
  const int DR = wa.out_row_elems();
  if constexpr (PART) {
    const int64_t slot = (row * p.num_heads + head) * p.max_num_partitions + part;
    W::template store_f32<SL>(reinterpret_cast<float *>(p.out) + slot * DR + d0, o, inv);
    // one lane per column writes the scalars: r = 0, or of the lanes that keep a paired column's
    // output the first (r = 0 for the pair's first head, 2 for its second)
    if ((wa.paired() ? (r & 1) == 0 : r == 0) && wave == 0) {
      p.max_logits[slot] = M * kLn2;  // natural-log units, as upstream stores them
      p.exp_sums[slot] = L;
    }
  } else {
    W::template store_q<SL>(reinterpret_cast<char *>(p.out) + ((row * p.num_heads + head) * DR + d0) * 2, o, inv);
  }
}

// MASKS: the extended instance.  It applies the score modifiers of p.mask_flags (soft-capping,
// local window, ALiBi) and takes p.query_len query tokens per sequence, causal among
// themselves (speculative decoding, chunked prefill): the MFMA columns are then (query token,
// head) pairs; an FP8 cache may bring per-head or per-block scales (p.kv_scale_mode).  Chunks
// that lie wholly before a sequence's window are skipped; a partition of which a column sees
// nothing stores an empty partial for it (max -inf, sum 0, zeros).
template <int D, typename QT, int KVF, bool PART, int NW, int OCC, int TPC, bool MASKS = false, bool KROW = true>
__global__ void __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(OCC)))
paged_attn_kernel(const PagedAttnParams p) {
  using W = WaveAttn<D, QT, KVF, TPC, PART ? Pipeline<(KVF != 0)>::stream_loads_split : Pipeline<(KVF != 0)>::stream_loads_loop, MASKS, KROW>;
  using Chunk = typename W::Chunk;
  using Ids = typename W::Ids;
  constexpr int CT = W::CT;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int kvh = blockIdx.x;
  const int part = blockIdx.y;
  const int seq = blockIdx.z;

  W wa(p, lane);
  const int tok_begin = PART ? part * p.partition_size : 0;
  const int c_begin = tok_begin / CT;
  const int32_t *table = p.block_tables + (int64_t)seq * p.max_blocks_per_seq;

  // Ids of this wavefront's first chunk.  When the pool size is known any column of the
  // table row is safe to read, so the ids are requested together with the context length
  // instead of after it.
  const bool pool_known = p.max_block_id != INT32_MAX;
  Ids ids0 = {};
  if (pool_known) ids0 = wa.fetch_ids(table, c_begin + wave, p.max_blocks_per_seq - 1);

  // a length the block table cannot hold is cut to what it holds
  const int ctx = min(p.context_lens[seq], p.max_blocks_per_seq << p.block_shift);
  const int tok_end = PART ? min(ctx, tok_begin + p.partition_size) : ctx;
  if (tok_begin >= tok_end) return;  // empty partition / empty sequence: nothing is written

  const int c_end = (tok_end + CT - 1) / CT;
  // highest block-table column that may be read
  const int last_blk = pool_known ? p.max_blocks_per_seq - 1 : (ctx - 1) >> p.block_shift;

  wa.load_q(seq, kvh);
  wa.reset(wa.load_sink(kvh, wave == 0 && (!PART || part == 0)));
  int c_lo = c_begin;  // first chunk that holds a visible token
  typename W::ItemExt ext = {};
  if constexpr (MASKS) {
    ext = wa.fetch_item_ext(kvh, table);
    wa.set_item(ext, ctx);
    c_lo = wa.first_visible_chunk(ctx, c_begin);  // the earliest query token's window decides
  }

  // ---- streaming loop ------------------------------------------------------------------
  // The last chunk of a wavefront is computed outside the issuing path, so no wait on the
  // loads of the current chunk ever has to cover a path on which nothing more was issued.
  // Only that last chunk can reach past the end of the token range.
  int ci = c_lo + wave;
  if (ci < c_end) {
    if (!pool_known || c_lo != c_begin) ids0 = wa.fetch_ids(table, ci, last_blk);
    // One register set.  K of chunk n+1 is requested as soon as the score MFMAs of
    // chunk n have read K, V of chunk n+1 as soon as the P.V MFMAs have read V: about
    // half a chunk is in flight per wavefront at any time.  (Two register sets with the
    // whole next chunk in flight were measured too: same bandwidth, a third fewer
    // wavefronts resident.)
    Chunk R;
    wa.issue_k(R, kvh, ci, ids0);
    wa.issue_v(R, kvh, ci, ids0);
    typename W::TileScales ts = {}, nts = {};  // extended instances only
    if constexpr (MASKS) ts = wa.fetch_scales(ids0, kvh, ext);
    Ids nids = wa.fetch_ids(table, ci + NW, last_blk);
    while (ci + NW < c_end) {
      const int cn = ci + NW;
      const auto s = wa.qk(R);
      wa.issue_k(R, kvh, cn, nids);
      if constexpr (MASKS) nts = wa.fetch_scales(nids, kvh, ext);
      const auto pb = wa.template soft<false, MASKS>(R, s, ci, tok_end, &ts);
      wa.pv(R, pb);
      wa.issue_v(R, kvh, cn, nids);
      nids = wa.fetch_ids(table, cn + NW, last_blk);
      ts = nts;
      ci = cn;
    }
    const auto s = wa.qk(R);
    wa.pv(R, wa.template soft<true, MASKS>(R, s, ci, tok_end, &ts));
  }

  __shared__ float merge_lds[NW > 1 ? NW * (W::NR * 64 + 32) : 1];
  merge_and_store<PART, NW>(wa, p, lane, wave, seq, kvh, part, merge_lds);
}

}  // namespace fa
