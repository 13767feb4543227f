// Single-pass decode for query groups of ONE head without the matrix cores: the scores are lane
// products (v_dot2_f32_f16) summed over the lanes of a token row with DPP moves, and P.V is fp32
// multiply-adds in the VALU (v_fma_mix_f32 straight from the 16-bit values).
//
// Why it exists: with one query head per kv head the MFMA path (paged_attention_wave.h) fills one
// of its sixteen columns, and a dot-product path is the textbook alternative.  WaveDot below is one
// wavefront's share of that alternative; two kernels are built from it, as from WaveAttn:
//   paged_attn_valu_kernel             grid form, one work-group per (sequence, head) (upstream's
//                                      decomposition, paged_attention_kernel_loop.hpp:602-607)
//   paged_attn_valu_persistent_kernel  resident work-groups that walk the items, the schedule of
//                                      paged_attention_loop_persistent_kernel.h
// Head size 128, fp16 queries, 16-bit or FP8 caches, plain decode (no score modifiers).
//
// Layout.  A token row of K or V is ROWB bytes; LPR = ROWB / 16 lanes take 16 bytes of it each, so a
// load instruction covers RPI = 64 / LPR whole rows, every line whole.  A lane keeps the query and the
// output for the head-dim elements of its 16 bytes only.  The lanes of a row all get the row's
// score (a butterfly of DPP adds), so the probabilities need no further exchange: each lane
// multiplies its own V elements.  The RPI rows of a load instruction are independent streams with
// a softmax state each; they merge when the wavefront is through with an item.  Same software
// pipeline as the MFMA kernels: one register set, K of chunk n+1 requested when the scores of chunk
// n are out, V of chunk n+1 after P.V.
//
// Arithmetic follows upstream's (scores paged_attention_kernel_loop.hpp:227-348, softmax :353-444,
// P.V :455-546) except that the probabilities stay fp32 (upstream and the MFMA path round them to
// the query type before P.V).
#pragma once

#include "paged_attention_items.h"
#include "paged_attention_loop_persistent_kernel.h"

namespace fa {

typedef _Float16 f16pair __attribute__((ext_vector_type(2)));

// x + (x of the lane that CTRL names), within rows of 16 lanes
template <int CTRL>
__device__ __forceinline__ float dpp_add(float x) {
  return x + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}

template <int KVF, bool STREAM>
struct WaveDot {
  static constexpr int D = 128;
  static constexpr bool KV8 = KVF != kKv16;
  static constexpr int ROWB = D * (KV8 ? 1 : 2);  // bytes per token row
  static constexpr int LPR = ROWB / 16;           // lanes per token row
  static constexpr int RPI = 64 / LPR;            // token rows per load instruction = streams per wavefront
  static constexpr int CT = 32;                   // tokens per chunk
  static constexpr int NL = CT / RPI;             // load instructions per chunk and operand
  static constexpr int EPL = KV8 ? 16 : 8;        // head-dim elements per lane
  static constexpr int QD = EPL / 2;              // dwords of fp16 pairs per lane
  static_assert(kTileTokens % RPI == 0, "the rows of a load instruction lie in one block");
  static constexpr uint32_t kNoSink = 0xffffffffu;

  struct Ids { uint32_t v[2]; };               // physical blocks of a chunk's two 16-token tiles
  struct Chunk { uint32_t k[NL][4], v[NL][4]; };

  const PagedAttnParams &p;
  const int sub, rowi;  // which 16 bytes of a row, which row of a load instruction
  const int blk_mask;
  uint32_t q[QD];       // the query elements of this lane's 16 bytes of a row, as fp16 pairs
  float m, l, acc[EPL];  // this lane's stream: maximum in base-2 units, sum, un-normalised output

  __device__ __forceinline__ WaveDot(const PagedAttnParams &p_, int lane)
      : p(p_), sub(lane % LPR), rowi(lane / LPR), blk_mask((1 << p_.block_shift) - 1) {}

  __device__ __forceinline__ Ids fetch_ids(const int32_t *table, int ci, int col_max) const {
    Ids ids;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int col = min((ci * CT + t * kTileTokens) >> p.block_shift, col_max);
      ids.v[t] = min((uint32_t)load_uniform_i32(table + col), (uint32_t)p.max_block_id);
    }
    return ids;
  }
  __device__ __forceinline__ void load_q(int seq, int head) {
    const char *src = reinterpret_cast<const char *>(p.query) + (((int64_t)seq * p.num_heads + head) * D + sub * EPL) * 2;
#pragma unroll
    for (int d = 0; d < QD; d += 4) {
      const u32x4 t = *reinterpret_cast<const u32x4 *>(src + d * 4);
      q[d] = t[0]; q[d + 1] = t[1]; q[d + 2] = t[2]; q[d + 3] = t[3];
    }
  }
  // the sink is one more logit with a zero value row: it joins ONE stream of one wavefront
  __device__ __forceinline__ uint32_t load_sink(int head, bool with_sink) const {
    uint32_t raw = kNoSink;
    if (with_sink && rowi == 0 && p.sinks != nullptr) raw = reinterpret_cast<const uint16_t *>(p.sinks)[head];
    return raw;
  }
  __device__ __forceinline__ void reset(uint32_t sink_raw) {
    m = -INFINITY;
    l = 0.f;
    if (sink_raw != kNoSink) {
      const uint16_t h = (uint16_t)sink_raw;
      m = load_scalar16<F16>(&h) * kLog2e;
      l = 1.f;
    }
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[e] = 0.f;
  }
  // where this lane reads in load instruction j of chunk ci, as a byte offset into the pool
  __device__ __forceinline__ int64_t row_offset(int head, int ci, int j, const Ids &ids) const {
    const int tok = ci * CT + j * RPI + rowi;
    return (int64_t)ids.v[(j * RPI) / kTileTokens] * p.kv_block_bytes + (int64_t)head * p.kv_head_bytes +
           (int64_t)(tok & blk_mask) * p.kv_token_bytes + sub * 16;
  }
  __device__ __forceinline__ void issue_k(Chunk &R, int head, int ci, const Ids &ids) const {
#pragma unroll
    for (int j = 0; j < NL; ++j) VLoad<4, STREAM>::ld(R.k[j], p.key_cache + row_offset(head, ci, j, ids));
  }
  __device__ __forceinline__ void issue_v(Chunk &R, int head, int ci, const Ids &ids) const {
#pragma unroll
    for (int j = 0; j < NL; ++j) VLoad<4, STREAM>::ld(R.v[j], p.value_cache + row_offset(head, ci, j, ids));
  }
  // 16 bytes of a row as QD dwords of fp16 pairs
  static __device__ __forceinline__ void pairs_of(const uint32_t (&w)[4], uint32_t (&h)[QD]) {
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      if constexpr (KV8) {
        h[2 * d] = fp8_adjacent_pair<KVF, F16>(w[d], 0);
        h[2 * d + 1] = fp8_adjacent_pair<KVF, F16>(w[d], 1);
      } else {
        h[d] = w[d];
      }
    }
  }
  // scores of the chunk's NL rows of this lane's stream, in base-2 units: every lane of a row gets its row's
  struct Scores { float s[NL]; };
  __device__ __forceinline__ Scores qk(const Chunk &R) const {
    Scores out;
#pragma unroll
    for (int j = 0; j < NL; ++j) {
      uint32_t h[QD];
      pairs_of(R.k[j], h);
      float dot = 0.f;
#pragma unroll
      for (int d = 0; d < QD; ++d)
        dot = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16pair, h[d]), __builtin_bit_cast(f16pair, q[d]), dot, false);
      dot = dpp_add<0xB1>(dot);                            // quad_perm [1,0,3,2]
      dot = dpp_add<0x4E>(dot);                            // quad_perm [2,3,0,1]
      dot = dpp_add<0x141>(dot);                           // row_half_mirror: the other quad of eight lanes
      if constexpr (LPR == 16) dot = dpp_add<0x140>(dot);  // row_mirror: the other eight lanes
      out.s[j] = dot * p.score_scale_log2;
    }
    return out;
  }
  // online softmax and P.V for one chunk; TAIL: tokens at or beyond tok_end are selected away (never
  // multiplied: rows past a context may hold anything)
  template <bool TAIL>
  __device__ __forceinline__ void soft_pv(const Chunk &R, Scores sc, int ci, int tok_end) {
    bool live[NL];
    float mc = -INFINITY;
#pragma unroll
    for (int j = 0; j < NL; ++j) {
      live[j] = !TAIL || ci * CT + j * RPI + rowi < tok_end;
      if constexpr (TAIL) sc.s[j] = live[j] ? sc.s[j] : -INFINITY;
      mc = fmaxf(mc, sc.s[j]);
    }
    const float mn = fmaxf(m, mc);
    if (__any(mn != m)) {
      const float alpha = (m == -INFINITY) ? 0.f : fast_exp2(m - mn);  // (mn > -inf wherever mn != m)
      l *= alpha;
#pragma unroll
      for (int e = 0; e < EPL; ++e) acc[e] *= alpha;
      m = mn;
    }
    const float base = (m == -INFINITY) ? 0.f : m;
#pragma unroll
    for (int j = 0; j < NL; ++j) {
      const float pj = fast_exp2(sc.s[j] - base);
      l += pj;
      uint32_t h[QD];
      pairs_of(R.v[j], h);
#pragma unroll
      for (int d = 0; d < QD; ++d) {
        const f16pair v = __builtin_bit_cast(f16pair, TAIL && !live[j] ? 0u : h[d]);
        acc[2 * d] = fmaf((float)v[0], pj, acc[2 * d]);
        acc[2 * d + 1] = fmaf((float)v[1], pj, acc[2 * d + 1]);
      }
    }
  }
  // the wavefront's streams into one state, which every lane ends up with
  __device__ __forceinline__ void merge_streams() {
#pragma unroll
    for (int off = LPR; off < 64; off <<= 1) {
      const float mb = __shfl_xor(m, off), lb = __shfl_xor(l, off);
      const float M = fmaxf(m, mb);
      const float base = (M == -INFINITY) ? 0.f : M;
      const float fa_ = (m == -INFINITY) ? 0.f : fast_exp2(m - base);
      const float fb = (mb == -INFINITY) ? 0.f : fast_exp2(mb - base);
      l = fa_ * l + fb * lb;
#pragma unroll
      for (int e = 0; e < EPL; ++e) acc[e] = fa_ * acc[e] + fb * __shfl_xor(acc[e], off);
      m = M;
    }
  }
};

// States of the NW wavefronts of a work-group (after merge_streams) into head-dim element d of the
// result: sm_m / sm_l [NW], sm_acc [NW][128].
template <int NW>
__device__ __forceinline__ float merged_output(const float *sm_m, const float *sm_l, const float (*sm_acc)[128], int d,
                                               float out_scale) {
  float M = -INFINITY;
#pragma unroll
  for (int w = 0; w < NW; ++w) M = fmaxf(M, sm_m[w]);
  float L = 0.f, o = 0.f;
#pragma unroll
  for (int w = 0; w < NW; ++w) {
    const float f = (sm_m[w] == -INFINITY) ? 0.f : fast_exp2(sm_m[w] - M);  // a wavefront without chunks
    L += f * sm_l[w];
    o += f * sm_acc[w][d];
  }
  return L > 0.f ? o * (out_scale / L) : 0.f;
}

// ---- grid form ------------------------------------------------------------------------------------
template <int KVF, int NW, bool STREAM>
__global__ void __launch_bounds__(NW * 64) paged_attn_valu_kernel(const PagedAttnParams p) {
  using W = WaveDot<KVF, STREAM>;
  using Ids = typename W::Ids;
  constexpr int CT = W::CT, D = W::D;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int head = blockIdx.x;  // = kv head: groups of one
  const int seq = blockIdx.z;
  const int32_t *table = p.block_tables + (int64_t)seq * p.max_blocks_per_seq;
  const bool pool_known = p.max_block_id != INT32_MAX;

  W wa(p, lane);
  Ids ids0 = {};
  if (pool_known) ids0 = wa.fetch_ids(table, wave, p.max_blocks_per_seq - 1);  // with the length, not after it
  const int ctx = min(p.context_lens[seq], p.max_blocks_per_seq << p.block_shift);
  if (ctx <= 0) return;  // nothing is written for an empty sequence
  const int c_end = (ctx + CT - 1) / CT;
  const int last_blk = pool_known ? p.max_blocks_per_seq - 1 : (ctx - 1) >> p.block_shift;

  wa.load_q(seq, head);
  wa.reset(wa.load_sink(head, wave == 0));
  int ci = wave;
  if (ci < c_end) {
    if (!pool_known) ids0 = wa.fetch_ids(table, ci, last_blk);
    typename W::Chunk R;
    wa.issue_k(R, head, ci, ids0);
    wa.issue_v(R, head, ci, ids0);
    Ids nids = wa.fetch_ids(table, ci + NW, last_blk);
    while (ci + NW < c_end) {  // the last chunk is computed outside the issuing path
      const int cn = ci + NW;
      const auto s = wa.qk(R);
      wa.issue_k(R, head, cn, nids);
      wa.template soft_pv<false>(R, s, ci, ctx);
      wa.issue_v(R, head, cn, nids);
      nids = wa.fetch_ids(table, cn + NW, last_blk);
      ci = cn;
    }
    const auto s = wa.qk(R);
    wa.template soft_pv<true>(R, s, ci, ctx);
  }
  wa.merge_streams();
  __shared__ float sm_m[NW], sm_l[NW], sm_acc[NW][D];
  if (wa.rowi == 0) {
#pragma unroll
    for (int e = 0; e < W::EPL; ++e) sm_acc[wave][wa.sub * W::EPL + e] = wa.acc[e];
    if (wa.sub == 0) {
      sm_m[wave] = wa.m;
      sm_l[wave] = wa.l;
    }
  }
  __syncthreads();
  if (threadIdx.x < D)  // thread d stores head-dim element d
    reinterpret_cast<_Float16 *>(p.out)[((int64_t)seq * p.num_heads + head) * D + threadIdx.x] =
        (_Float16)merged_output<NW>(sm_m, sm_l, sm_acc, threadIdx.x, p.out_scale);
}

// ---- persistent form --------------------------------------------------------------------------------
// The schedule of paged_attn_loop_persistent_kernel with WaveDot in WaveAttn's place: resident
// work-groups walk (sequence, head) items dealt longest first in snake order; a wavefront that is
// through with its chunks of an item has already requested the query and the first K/V chunk of the
// next one, parks its state in LDS and goes on; the states of an item are merged one chunk later
// (publish / finish: see that kernel for why the wait always ends and why a buffer is never
// overwritten while it is read).  Up to 128 sequences, as there.
template <int KVF, int NWG, bool STREAM, int OCC>
__global__ void __launch_bounds__(NWG * 64) __attribute__((amdgpu_waves_per_eu(OCC)))
paged_attn_valu_persistent_kernel(const PagedAttnParams p) {
  constexpr int NW = NWG;
  using W = WaveDot<KVF, STREAM>;
  using Ids = typename W::Ids;
  constexpr int CT = W::CT, D = W::D;
  constexpr int SL = D / NW;  // head-dim elements a wavefront stores of a merged item
  static_assert(SL <= 64 && D % NW == 0, "one lane per stored element");
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int G = gridDim.x;
  const int wg = blockIdx.x;
  const int col_max = p.max_blocks_per_seq - 1;

  using Item = WorkItem;
  LoopItems<2> items;
  items.build(p, lane, wave, G, CT, 1);
  auto item_at = [&](int n, Item &it) -> bool { return items.at(n, G, wg, CT, it); };

  __shared__ float sm_m[2][NW], sm_l[2][NW], sm_acc[2][NW][D];  // item n goes to buffer n & 1
  __shared__ int sm_arrived[2];  // wavefronts that have published into the buffer, ever

  W wa(p, lane);
  typename W::Chunk R;
  int n = 0;
  Item cur;
  if (!item_at(0, cur)) return;  // the same for every wavefront of the work-group
  if (threadIdx.x < 2) sm_arrived[threadIdx.x] = 0;
  __syncthreads();  // the only barrier: wavefronts meet through the counters from here on

  auto publish = [&](int item) {
    const int b = item & 1;
    wa.merge_streams();
    if (wa.rowi == 0) {
#pragma unroll
      for (int e = 0; e < W::EPL; ++e) sm_acc[b][wave][wa.sub * W::EPL + e] = wa.acc[e];
      if (wa.sub == 0) {
        sm_m[b][wave] = wa.m;
        sm_l[b][wave] = wa.l;
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    if (lane == 0) __hip_atomic_fetch_add(&sm_arrived[b], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  };
  auto finish = [&](int item, int seq, int head) {
    const int b = item & 1;
    const int target = NW * ((item >> 1) + 1);
    bool arrived = false;
    for (int spin = 0; spin < p.spin_limit; ++spin) {
      const int seen = __hip_atomic_load(&sm_arrived[b], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      if (__builtin_amdgcn_readfirstlane(seen) >= target) {
        arrived = true;
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    // gave up: the result is wrong; say so in the status word and carry on, so that the grid drains
    if (!arrived && lane == 0) __hip_atomic_store(p.status, kStatusSpinLimit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    if (lane < SL) {
      const int d = wave * SL + lane;
      reinterpret_cast<_Float16 *>(p.out)[((int64_t)seq * p.num_heads + head) * D + d] =
          (_Float16)merged_output<NW>(sm_m[b], sm_l[b], sm_acc[b], d, p.out_scale);
    }
  };

  // A wavefront takes chunks wave, wave + NW, ... of an item.  One that has none (an item of fewer
  // than NW chunks) reads the item's last chunk all the same and selects every token of it away: one
  // path through the loop for all wavefronts, so that no second register set for the chunk in
  // flight is needed where paths would meet.
  auto first_chunk = [&](const Item &it) { return min(wave, it.c_end - 1); };
  auto visible_end = [&](const Item &it) { return wave < it.c_end ? it.ctx : 0; };
  {  // first chunk of the first item
    Ids ids;
#pragma unroll
    for (int t = 0; t < 2; ++t) ids.v[t] = min((uint32_t)items.first_id(t, cur.seq), (uint32_t)p.max_block_id);
    if (wave >= cur.c_end) ids = wa.fetch_ids(p.block_tables + (int64_t)cur.seq * p.max_blocks_per_seq, first_chunk(cur), col_max);
    wa.load_q(cur.seq, cur.kvh);
    wa.issue_k(R, cur.kvh, first_chunk(cur), ids);
    wa.issue_v(R, cur.kvh, first_chunk(cur), ids);
  }
  uint32_t sink_raw = wa.load_sink(cur.kvh, wave == 0);
  Item prev = cur;  // the item whose merge is still owed (from the second item on)

  while (true) {
    Item nxt;
    const bool has_next = item_at(n + 1, nxt);
    Ids nxt_ids = {};
    if (has_next) nxt_ids = wa.fetch_ids(p.block_tables + (int64_t)nxt.seq * p.max_blocks_per_seq, first_chunk(nxt), col_max);

    wa.reset(sink_raw);
    uint32_t next_sink = W::kNoSink;
    bool owed = n > 0;
    const int32_t *table = p.block_tables + (int64_t)cur.seq * p.max_blocks_per_seq;
    const int tok_end = visible_end(cur);
    int ci = first_chunk(cur);
    Ids nids = wa.fetch_ids(table, ci + NW, col_max);
    if (ci + NW < cur.c_end) {
      {  // first chunk of the item, then the merge owed to the previous item
        const int cn = ci + NW;
        const auto s = wa.qk(R);
        wa.issue_k(R, cur.kvh, cn, nids);
        wa.template soft_pv<false>(R, s, ci, tok_end);
        wa.issue_v(R, cur.kvh, cn, nids);
        nids = wa.fetch_ids(table, cn + NW, col_max);
        ci = cn;
      }
      if (owed) {
        finish(n - 1, prev.seq, prev.kvh);
        owed = false;
      }
      while (ci + NW < cur.c_end) {  // steady state: the next chunk belongs to the same item
        const int cn = ci + NW;
        const auto s = wa.qk(R);
        wa.issue_k(R, cur.kvh, cn, nids);
        wa.template soft_pv<false>(R, s, ci, tok_end);
        wa.issue_v(R, cur.kvh, cn, nids);
        nids = wa.fetch_ids(table, cn + NW, col_max);
        ci = cn;
      }
    }
    {  // last chunk of this wavefront in `cur`: what goes out next belongs to `nxt`
      const auto s = wa.qk(R);
      if (has_next) {
        wa.load_q(nxt.seq, nxt.kvh);  // the query registers are free once the last scores are out
        next_sink = wa.load_sink(nxt.kvh, wave == 0);
        wa.issue_k(R, nxt.kvh, first_chunk(nxt), nxt_ids);
      }
      wa.template soft_pv<true>(R, s, ci, tok_end);
      if (has_next) wa.issue_v(R, nxt.kvh, first_chunk(nxt), nxt_ids);
    }
    if (owed) finish(n - 1, prev.seq, prev.kvh);
    publish(n);

    if (!has_next) break;
    prev = cur;
    cur = nxt;
    sink_raw = next_sink;
    ++n;
  }
  finish(n, cur.seq, cur.kvh);
}

}  // namespace fa
