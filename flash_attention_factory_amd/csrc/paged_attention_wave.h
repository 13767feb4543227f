// One wavefront's share of paged-attention decode on gfx950: operand loads, the two
// MFMA products and the online softmax between them.  The grid kernel and the
// persistent kernels are all built from this.
//
// Per chunk of TPC 16-token tiles (the query group's G <= 16 heads are the 16 MFMA columns):
//   S^T[token, head] = K[token, :] . Q^T[:, head]      per tile: D/32 MFMA 16x16x32
//   online softmax over tokens, fp32, base 2            VALU + two cross-row shuffles
//   O^T[d, head]    += V^T[d, token] . P^T[token, head] per 32 tokens: D/16 MFMA 16x16x32
// K rows enter the MFMA "A" operand exactly as they lie in HBM (lane 16r+i loads 16 B
// of token i); V rows are loaded row-wise (16 lanes cover one token row) and
// transposed inside each lane with byte permutes, so neither needs LDS.  The scores
// come out of the first MFMA in the register layout the second MFMA wants for P^T.
//
// Arithmetic follows the upstream kernels (scores paged_attention_kernel_loop.hpp:227-348,
// softmax :353-444, P.V :455-546; FP8 paged_attention_kernel_fp8_loop.hpp:328-333,540-545):
// fp32 scores scaled after the dot, tail tokens masked to -inf, probabilities rounded to
// the query dtype before P.V, fp8_scale folded into the score scale and the final scale.
#pragma once

#include <type_traits>

#include "paged_attention_policy.h"
#include "paged_attention_utils.h"

// K tiles with rows of 128 bytes or more are loaded a whole 128-byte line per eight lanes and put
// into MFMA layout with one exchange between lanes i and i ^ 8 (see WaveAttn::issue_k).
#ifndef FA_K_ROW_LOADS
#define FA_K_ROW_LOADS 1
#endif


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
  int32_t num_seqs;
  int32_t num_heads;
  int32_t num_kv_heads;
  int32_t group;                // query heads per kv head
  int32_t max_blocks_per_seq;
  int32_t max_num_partitions;
  int32_t partition_size;       // tokens; multiple of 64
  int32_t block_shift;          // log2(block_size)
  int32_t max_block_id;         // block ids are clamped into [0, max_block_id]
  int64_t kv_block_bytes;       // strides in BYTES
  int64_t kv_token_bytes;
  int64_t kv_head_bytes;
  // score modifiers, applied only by kernel instances built with MASKS (mask_flags != 0)
  const float *alibi_slopes;    // [H] fp32
  float score_scale;            // sm_scale * fp8_scale (natural-log units)
  float softcap;
  int32_t window_left;
  int32_t mask_flags;           // kMaskAlibi | kMaskSoftcap | kMaskWindow
  int32_t query_len;            // query tokens per sequence (1 = plain decode)
  int32_t query_first;          // of those, the launch at hand covers tokens query_first ..
  int32_t query_count;          // query_first + query_count - 1 (query_count * group <= 16)
  // finer dequantisation scales of an FP8 cache, read only by the extended instances.  With a
  // mode other than kScaleTensor score_scale is the bare softmax scale and out_scale is 1.
  int32_t kv_scale_mode;        // kScaleTensor / kScaleHead / kScaleBlock
  const float *k_scales;        // [Hk] or [pool blocks, Hk] fp32
  const float *v_scales;
  // persistent kernels: polls a wavefront spends on one wait for the other wavefronts of its
  // work-group before it gives up, and the device word in which it says so (see launch_common.h)
  int32_t spin_limit;
  int32_t *status;
  // Paired kv heads (FP8 caches with token rows of 64 bytes whose kv heads lie next to each
  // other): a head-size-128 instance takes two kv heads as one -- num_kv_heads, group and
  // kv_head_bytes describe the pairs -- while query and out rows keep 64 elements.  See
  // WaveAttn::kPairable.
  int32_t pair_heads;
  // what the split path's segment length depends on besides the batch (partitions_per_segment):
  // the compute units of the GPU, and whether the token rows of a kv head lie apart in the pools
  // (upstream's layout [blocks, block, kv_heads, d]) or on end (a block's rows of one kv head
  // contiguous)
  int32_t compute_units;
  int32_t kv_rows_apart;
  int32_t segment_force;  // options->segment_partitions: > 0 partitions per segment as the caller fixed them, -1 even shares
  // Split path, segment form: the call's `out`.  A row whose context fits one segment has one
  // partial, which is its result: the attention kernel rounds it to the query type and stores it
  // here, not into tmp_out (exp_sums and max_logits still get the partial's scalars), and the reduce
  // kernel leaves such rows alone.  NULL: every partial goes to tmp_out.
  void *final_out;
};

constexpr int kMaskAlibi = 1, kMaskSoftcap = 2, kMaskWindow = 4;  // = fa_mask of the C ABI
constexpr int kScaleTensor = 0, kScaleHead = 1, kScaleBlock = 2;  // = fa_kv_scale of the C ABI

// TPC: 16-token tiles per chunk (2 or 4).  One chunk is the unit of the software
// pipeline; 4 tiles give an FP8 cache the same bytes in flight as 2 tiles of fp16.
// KVF: cache format, kKv16 (elements of the query type), kKvE5M2 or kKvE4M3 (bytes).
// EXT: the extended instance -- score modifiers, several query tokens per sequence and
// per-head or per-block scales of an FP8 cache (p.mask_flags, p.query_len, p.kv_scale_mode).
// The MFMA columns then stand for (query token, head) pairs: column i = query token
// p.query_first + i / G, head i % G of the kv head's group; a launch covers the p.query_count
// tokens that fit the 16 columns, the host launches once per such group of tokens.
// KROW: K tiles are loaded a whole 128-byte line per eight lanes (see kRowLoads below).
template <int D, typename QT, int KVF, int TPC, bool STREAM, bool EXT = false, bool KROW = true>
struct WaveAttn {
  static constexpr bool KV8 = KVF != kKv16;
  static constexpr bool kExt = EXT;
  static_assert(TPC == 2 || TPC == 4, "a chunk is one or two 32-token P.V steps");
  static constexpr int ROWB = D * (KV8 ? 1 : 2);  // bytes per token row
  static constexpr int KL = ROWB / 64;            // 16-byte K loads per lane and tile
  static constexpr int KSTEPS = D / 32;           // MFMA k-steps across the head dimension
  static constexpr int NDT = D / 16;  // output d-tiles; lane row i of tile dt is d = i*NDT + dt
  static constexpr int VW = ROWB / 64;            // dwords of V per lane and token
  static constexpr int VB = VW * 4;               // bytes of V per lane and token
  static constexpr int CT = TPC * kTileTokens;    // tokens per chunk
  static constexpr int NP2 = TPC / 2;             // 32-token P.V steps per chunk
  static constexpr int NR = NDT * 4;              // accumulator values per lane
  static constexpr bool kStream = STREAM;  // non-temporal K/V loads
  // K rows of one or two 128-byte lines: a load instruction in MFMA layout (lane 16r+i takes
  // 16 B of row i) would touch half of each of 16 lines, and the memory pipeline pays per line
  // touched -- measured on a plain streaming probe, 3-5 % of the bandwidth.  Instead a load
  // takes one whole line of each of eight rows (lane (r, i): row 8h + (i & 7), bytes
  // 128 L + (i >> 3) * 64 + r * 16 for load c = 2L + h), and k_rows_to_mfma() moves the halves
  // that sit in the wrong lane across with DPP.  The head-dim <-> k-slot map stays what it was.
  static constexpr bool kRowLoads = FA_K_ROW_LOADS != 0 && KROW && ROWB >= 128;
  // Paired kv heads (p.pair_heads).  With token rows of 64 bytes every 128-byte line of a
  // token-major pool belongs to two kv heads; two work-groups would fetch it once each.  Here
  // the two heads' rows are one 128-byte row of a pair: the 2G query heads of both are the MFMA
  // columns, a column's query is zero over the other head's half of the row (so the scores are
  // its own head's), and of the 128 output rows a column keeps the half that belongs to its
  // head: lanes r = 0, 1 hold a pair's dims 0..63 (first head), r = 2, 3 dims 64..127 (second).
  static constexpr bool kPairable = KV8 && D == 128 && !EXT;
  __device__ __forceinline__ bool paired() const { return kPairable && p.pair_heads != 0; }
  // which head of its pair column i belongs to
  __device__ __forceinline__ int col_half() const { return i >= (p.group >> 1) ? 1 : 0; }
  // does this lane hold output elements its column keeps, how long is a row of query / out /
  // tmp_out, and which element of that row is the lane's first (d0: its first of the pair's 128)
  __device__ __forceinline__ bool keeps_output() const { return !paired() || (r >> 1) == col_half(); }
  __device__ __forceinline__ int out_row_elems() const { return paired() ? D / 2 : D; }
  __device__ __forceinline__ int out_elem(int d0) const { return paired() ? d0 - (D / 2) * (r >> 1) : d0; }


  // Register image of one chunk of K and V.
  struct Chunk {
    u32x4 k[TPC][KL];
    uint32_t v[4 * TPC][VW];
  };
  struct Ids { int v[TPC]; };      // physical block id of every tile of a chunk
  struct Scores { f32x4 v[TPC]; };
  // EXT, per-block scales: what the scores of each tile are multiplied with (softmax scale x
  // the tile's K scale) and what its probabilities are multiplied with before P.V (the tile's
  // V scale over the item's reference V scale)
  struct TileScales { float k[TPC], v[TPC]; };
  struct Probs { u32x4 v[NP2]; };

  const PagedAttnParams &p;
  const int r;  // 16-lane row of the wavefront
  const int i;  // position in the row: token (K), head (Q, P, O) or d-row (V)
  const int blk_mask;
  // EXT only: what column i stands for, and the position of its query token
  int col_q = 0, col_g = 0, col_last = 0;
  bool col_valid = false;
  // EXT only, the same in every lane: the keys vis_lo .. vis_hi of the item at hand are seen by
  // every query token of the launch (causal rule and local window)
  int vis_lo = 0, vis_hi = -1;

  // Q^T as the MFMA "B" operand, one dword quad per k-step.  k-slot (r, e) of step c
  // stands for head-dim element qd(c, r) + e; K uses the same map.
  u32x4 qB[KSTEPS];
  // Online softmax state.  mt: running max (base-2 units) of head i, identical in the four
  // rows r.  m: the reference the sums are taken against, exp2(score - m); it follows mt only
  // when it has fallen behind by more than kRescaleSlack, because every change of m costs a
  // pass over the accumulators (with a handful of heads or query tokens in the 16 columns some
  // column sets a new maximum in nearly every chunk, by a small step).  Until then the
  // probabilities may exceed 1, by a factor of at most 2^kRescaleSlack: well inside the range
  // of fp16 and bf16, and sums and accumulators are fp32.  settle() brings m up to mt.
  // l: this lane's share of the running sum (its own tokens).
  // acc[dt][e]: O^T[d = (4r+e)*NDT + dt][head i], un-normalised.
  static constexpr float kRescaleSlack = 8.0f;
  float m, mt, l;
  f32x4 acc[NDT];
  float slope_log2 = 0.f;  // ALiBi slope of head i in base-2 units (MASKS instances only)
  // EXT: what the normalised output of the item at hand is multiplied with (see ItemExt).
  float out_mul = 1.f;

  // `tile`: which 16 columns of the launch's (query token, head) pairs this wavefront holds
  // (kernels with several column tiles per launch; 0 otherwise)
  __device__ __forceinline__ WaveAttn(const PagedAttnParams &prm, int lane, int tile = 0)
      : p(prm), r(lane >> 4), i(lane & 15), blk_mask((1 << prm.block_shift) - 1) {
    if constexpr (EXT) {
      const int q = tile * (16 / prm.group) + i / prm.group;  // query token of the launch
      col_g = i % prm.group;
      col_q = prm.query_first + q;
      col_valid = i < (16 / prm.group) * prm.group && q < prm.query_count;
    } else {
      col_g = i;
      col_valid = i < prm.group;
    }
  }

  // EXT: what an item (sequence, kv head) brings besides its query rows.  fetch_item_ext only
  // requests the values, so that a persistent kernel can ask for the next item's while the
  // current one still streams; set_item makes them the ones soft() works with.
  struct ItemExt {
    float slope;       // ALiBi slope of this lane's head as loaded (set_item converts it: arithmetic on
                       // the value here would make the wavefront wait for the load where it is issued)
    float k_mul;       // raw score -> scaled score: softmax scale x K scale (tensor or head)
    float out_mul;     // what the normalised output is multiplied with: V scale (tensor or
                       // head), or with per-block scales the item's reference V scale
    float inv_v_ref;   // per-block scales: 1 / out_mul
  };

  // `table`: the sequence's row of the block table; its first block's V scale serves as the
  // item's reference with per-block scales.
  __device__ __forceinline__ ItemExt fetch_item_ext(int kvh, const int32_t *table) const {
    ItemExt x;
    x.slope = 0.f;
    if ((p.mask_flags & kMaskAlibi) && col_valid) x.slope = p.alibi_slopes[kvh * p.group + col_g];
    x.k_mul = p.score_scale;
    x.out_mul = p.out_scale;
    x.inv_v_ref = 1.f;
    if constexpr (KV8) {
      if (p.kv_scale_mode == kScaleHead) {
        x.k_mul = p.score_scale * load_uniform_f32(p.k_scales + kvh);
        x.out_mul = load_uniform_f32(p.v_scales + kvh);
      } else if (p.kv_scale_mode == kScaleBlock) {
        const uint32_t b0 = min((uint32_t)load_uniform_i32(table), (uint32_t)p.max_block_id);
        x.out_mul = load_uniform_f32(p.v_scales + (int64_t)b0 * p.num_kv_heads + kvh);
        x.inv_v_ref = 1.0f / x.out_mul;
      }
    }
    return x;
  }

  // Query token q of the item sits at position ctx - query_len + q and sees the keys up to there.
  __device__ __forceinline__ void set_item(const ItemExt &x, int ctx) {
    slope_log2 = x.slope * kLog2e;
    out_mul = x.out_mul;
    col_last = ctx - p.query_len + col_q;
    vis_hi = ctx - p.query_len + p.query_first;  // the launch's earliest query token
    vis_lo = (p.mask_flags & kMaskWindow) ? vis_hi + p.query_count - 1 - p.window_left : 0;
  }

  // First chunk that holds a key some query token of the item sees (local window), at least c_begin.
  __device__ __forceinline__ int first_visible_chunk(int ctx, int c_begin) const {
    if (!(p.mask_flags & kMaskWindow)) return c_begin;
    return max(c_begin, max(0, ctx - p.query_len + p.query_first - p.window_left) / CT);
  }

  // EXT: multipliers of a chunk's tiles (uniform over the item unless the scales are per block).
  __device__ __forceinline__ TileScales fetch_scales(const Ids &ids, int kvh, const ItemExt &x) const {
    TileScales ts;
#pragma unroll
    for (int t = 0; t < TPC; ++t) {
      ts.k[t] = x.k_mul;
      ts.v[t] = 1.0f;
    }
    if constexpr (KV8) {
      if (p.kv_scale_mode == kScaleBlock) {
#pragma unroll
        for (int t = 0; t < TPC; ++t) {
          const int64_t at = (int64_t)ids.v[t] * p.num_kv_heads + kvh;
          ts.k[t] = p.score_scale * load_uniform_f32(p.k_scales + at);
          ts.v[t] = load_uniform_f32(p.v_scales + at) * x.inv_v_ref;
        }
      }
    }
    return ts;
  }

  __device__ __forceinline__ void load_q(int seq, int kvh) {
    const int head = kvh * p.group + col_g;
    const int64_t row = EXT ? (int64_t)seq * p.query_len + col_q : seq;
    const char *qrow = reinterpret_cast<const char *>(p.query) + (row * p.num_heads + head) * (out_row_elems() * 2);
#pragma unroll
    for (int c = 0; c < KSTEPS; ++c) {
      int d0 = KV8 ? ((c >> 1) * 4 + r) * 16 + (c & 1) * 8 : (c * 4 + r) * 8;
      bool live = col_valid;
      if constexpr (kPairable) {
        if (p.pair_heads) {  // k-steps 0, 1 run over the first head's dims, 2, 3 over the second's
          live = live && (c >> 1) == col_half();
          d0 -= (D / 2) * (c >> 1);
        }
      }
      u32x4 z = {0u, 0u, 0u, 0u};
      qB[c] = live ? *reinterpret_cast<const u32x4 *>(qrow + d0 * 2) : z;
    }
  }

  // The sink is one more logit with a zero value row; it belongs to the wavefront that
  // owns the start of the context (paged_attention_kernel_loop.hpp:387-391,
  // paged_attention_kernel_v2.hpp:373-376).  load_sink only requests the 16-bit value
  // (kNoSink if there is none for this lane); reset() decodes it, so that nothing has to
  // wait for the load where it is issued.
  static constexpr uint32_t kNoSink = 0xffffffffu;
  __device__ __forceinline__ uint32_t load_sink(int kvh, bool with_sink) const {
    uint32_t raw = kNoSink;
    if (with_sink && p.sinks != nullptr && col_valid)
      raw = *reinterpret_cast<const uint16_t *>(reinterpret_cast<const char *>(p.sinks) +
                                                (kvh * p.group + col_g) * 2);
    return raw;
  }

  // Fresh softmax state, optionally seeded with a sink logit (weight 1, value row 0).
  __device__ __forceinline__ void reset(uint32_t sink_raw) {
    m = -INFINITY;
    l = 0.f;
    if (sink_raw != kNoSink) {
      const uint16_t h = (uint16_t)sink_raw;
      m = load_scalar16<QT>(&h) * kLog2e;
      l = (r == 0) ? 1.f : 0.f;
    }
    mt = m;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // Sums and accumulators relative to the true maximum: the state every merge, publish and store
  // starts from (m is what max_logits and the merges see).
  __device__ __forceinline__ void settle() {
    if (__any(mt != m)) {
      const float m_sub = (mt == -INFINITY) ? 0.f : mt;
      const float alpha = fast_exp2(m - m_sub);
      l *= alpha;
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) acc[dt] *= alpha;
      m = mt;
    }
  }

  // Physical block id of every 16-token tile of chunk ci of a sequence's table row.
  // Columns are clamped to `col_max` and ids into the pool, so a tile wholly past the
  // context re-reads memory that exists; it is masked later.
  __device__ __forceinline__ Ids fetch_ids(const int32_t *table, int ci, int col_max) const {
    Ids ids;
#pragma unroll
    for (int t = 0; t < TPC; ++t) {
      const int col = min((ci * CT + t * kTileTokens) >> p.block_shift, col_max);
      ids.v[t] = min((uint32_t)load_uniform_i32(table + col), (uint32_t)p.max_block_id);
    }
    return ids;
  }

  __device__ __forceinline__ int64_t tile_offset(int kvh, int ci, int t, const Ids &ids) const {
    return (int64_t)ids.v[t] * p.kv_block_bytes + (int64_t)kvh * p.kv_head_bytes +
           (int64_t)((ci * CT + t * kTileTokens) & blk_mask) * p.kv_token_bytes;
  }

  // K and V of a chunk go out separately so that either half of the register set can be
  // refilled as soon as it has been consumed.  k_tile_at / v_tile_at: where this lane reads in
  // tile t of the chunk, as a byte offset into the pool (an offset, not a pointer: a pointer kept
  // across loop iterations loses its address space and the loads become flat loads);
  // load_k_one / load_v_one: one load instruction from there (KL per tile for K, four token rows
  // per tile for V), for kernels that spread a chunk's loads over the arithmetic of another.
  __device__ __forceinline__ int64_t k_tile_at(int kvh, int ci, int t, const Ids &ids) const {
    if constexpr (kRowLoads) {
      // load c brings line c >> 1 of the rows 8 (c & 1) .. 8 (c & 1) + 7 whole: the lanes (r, i)
      // and (r, i ^ 8) share a row
      return tile_offset(kvh, ci, t, ids) + (int64_t)(i & 7) * p.kv_token_bytes + (i >> 3) * 64 + r * 16;
    } else {
      return tile_offset(kvh, ci, t, ids) + (int64_t)i * p.kv_token_bytes + r * 16;
    }
  }
  __device__ __forceinline__ void load_k_one(Chunk &R, int t, int c, int64_t at) const {
    const char *kp = p.key_cache + at;
    if constexpr (kRowLoads) {
      R.k[t][c] = kv_load<kStream>(reinterpret_cast<const u32x4 *>(kp + (int64_t)(8 * (c & 1)) * p.kv_token_bytes + (c >> 1) * 128));
    } else {
      R.k[t][c] = kv_load<kStream>(reinterpret_cast<const u32x4 *>(kp + c * 64));
    }
  }
  __device__ __forceinline__ int64_t v_tile_at(int kvh, int ci, int t, const Ids &ids) const {
    return tile_offset(kvh, ci, t, ids) + (int64_t)(4 * r) * p.kv_token_bytes + i * VB;
  }
  __device__ __forceinline__ void load_v_one(Chunk &R, int t, int e, int64_t at) const {
    VLoad<VW, kStream>::ld(R.v[t * 4 + e], p.value_cache + at + e * p.kv_token_bytes);
  }
  __device__ __forceinline__ void issue_k(Chunk &R, int kvh, int ci, const Ids &ids) const {
#pragma unroll
    for (int t = 0; t < TPC; ++t) {
      const int64_t at = k_tile_at(kvh, ci, t, ids);
#pragma unroll
      for (int c = 0; c < KL; ++c) load_k_one(R, t, c, at);
    }
  }
  __device__ __forceinline__ void issue_v(Chunk &R, int kvh, int ci, const Ids &ids) const {
#pragma unroll
    for (int t = 0; t < TPC; ++t) {
      const int64_t at = v_tile_at(kvh, ci, t, ids);
#pragma unroll
      for (int e = 0; e < 4; ++e) load_v_one(R, t, e, at);
    }
  }

  // Row loads -> MFMA layout.  After the loads lane (r, i) holds x = bytes (i>>3)*64 + r*16 .. of
  // row i & 7 and y = the same bytes of row 8 + (i & 7); it needs bytes r*16 .. and 64 + r*16 .. of
  // row i.  Lanes i < 8 keep x and take x of lane i + 8; lanes i >= 8 keep y and take y of lane
  // i - 8: one rotation by eight within each row of 16 lanes, written to half of the lanes.
  static __device__ __forceinline__ void k_rows_to_mfma(u32x4 &x, u32x4 &y) {
    constexpr int kRowRor8 = 0x128;  // DPP control: rotate right by 8 within a row of 16 lanes
    u32x4 a0, a1;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      // bank mask 0xC: lanes 8..15 of each row are written, 0x3: lanes 0..7; the others keep `old`
      a0[w] = __builtin_amdgcn_update_dpp(x[w], y[w], kRowRor8, 0xF, 0xC, false);
      a1[w] = __builtin_amdgcn_update_dpp(y[w], x[w], kRowRor8, 0xF, 0x3, false);
    }
    x = a0;
    y = a1;
  }

  // K "A" operand of k-step c for one tile: row i = token, 8 head-dim elements.
  __device__ __forceinline__ u32x4 k_operand(const Chunk &R, int tile, int c) const {
    if constexpr (!KV8) {
      return R.k[tile][c];
    } else {
      const u32x4 src = R.k[tile][c >> 1];
      const int h = c & 1;
      u32x4 o;
      o[0] = fp8_adjacent_pair<KVF, QT>(src[2 * h], 0);
      o[1] = fp8_adjacent_pair<KVF, QT>(src[2 * h], 1);
      o[2] = fp8_adjacent_pair<KVF, QT>(src[2 * h + 1], 0);
      o[3] = fp8_adjacent_pair<KVF, QT>(src[2 * h + 1], 1);
      return o;
    }
  }

  // V^T "A" operand of d-tile dt for the 32-token step `pr` of the chunk: row i = d-row,
  // k-slots = this lane row's 8 tokens of the step.  In-lane transpose: R.v[e] holds
  // token e's NDT consecutive head-dim elements.
  __device__ __forceinline__ u32x4 v_operand(const Chunk &R, int pr, int dt) const {
    u32x4 o;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int e0 = pr * 8 + 2 * c;
      if constexpr (!KV8) {
        const uint32_t y = R.v[e0][dt >> 1], x = R.v[e0 + 1][dt >> 1];
        o[c] = (dt & 1) ? ((y >> 16) | (x & 0xffff0000u)) : ((y & 0xffffu) | (x << 16));
      } else {
        o[c] = fp8_pair_at<KVF, QT>(R.v[e0][dt >> 2], R.v[e0 + 1][dt >> 2], dt & 3);
      }
    }
    return o;
  }

  // scores: S^T tile rows are tokens 4r+e of the tile, column i is the head
  __device__ __forceinline__ Scores qk(Chunk &R) const {
    Scores s;
    if constexpr (kRowLoads) {
#pragma unroll
      for (int t = 0; t < TPC; ++t)
#pragma unroll
        for (int c = 0; c < KL; c += 2) k_rows_to_mfma(R.k[t][c], R.k[t][c + 1]);
    }
#pragma unroll
    for (int t = 0; t < TPC; ++t) s.v[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < KSTEPS; ++c)
#pragma unroll
      for (int t = 0; t < TPC; ++t) s.v[t] = mfma_16x16x32<QT>(k_operand(R, t, c), qB[c], s.v[t]);
    return s;
  }

  // Online softmax step over the chunk's tokens; returns the P^T "B" operands.
  // check_tail: whether this chunk can reach past tok_end (a compile-time false drops
  // the masking code from the steady-state loop).
  // MASKS (EXT instances): apply the score modifiers p.mask_flags names -- soft-capping, local
  // window, ALiBi, in that order (upstream test_paged.py:92-110) -- and the causal rule, all
  // relative to the position col_last of this column's query token.
  // ACC_IN_AGPRS: the kernel holds more than 256 registers and its accumulators live in AGPRs.
  // The rarely taken rescale branch then reads them with v_accvgpr_read_b32 spelled out and pins the
  // results to AGPRs again; left to itself the compiler copies every accumulator to a VGPR in front
  // of the branch, in every chunk, for the branch's benefit.
  template <bool CHECK_TAIL, bool MASKS = false, bool ACC_IN_AGPRS = false>
  __device__ __forceinline__ Probs soft(Chunk &R, const Scores &s, int ci, int tok_end,
                                        const TileScales *ts = nullptr) {
    constexpr int NT = 4 * TPC;  // this lane's tokens in the chunk: tile e/4, row 4r + e%4
    float t[NT];
    if (MASKS && !(p.mask_flags & (kMaskSoftcap | kMaskAlibi)) && ci * CT >= vis_lo && ci * CT + CT - 1 <= vis_hi) {
      // no score modifier, and every query token of the launch sees the whole chunk (all but the
      // last chunks of an item): plain scores with the tiles' own scale
      float k2[TPC];
#pragma unroll
      for (int tl = 0; tl < TPC; ++tl) k2[tl] = ts->k[tl] * kLog2e;
#pragma unroll
      for (int e = 0; e < NT; ++e) t[e] = s.v[e >> 2][e & 3] * k2[e >> 2];
    } else if constexpr (MASKS) {
      const bool cap = p.mask_flags & kMaskSoftcap;
      const float inv_cap2 = 2.0f * kLog2e / p.softcap;  // exp(2x/cap) = exp2(x * inv_cap2)
      const int first_visible = (p.mask_flags & kMaskWindow) ? col_last - p.window_left : 0;
#pragma unroll
      for (int e = 0; e < NT; ++e) t[e] = s.v[e >> 2][e & 3] * ts->k[e >> 2];
      if (cap) {  // cap * tanh(x / cap), tanh(z) = 1 - 2 / (exp(2z) + 1); a loop of its own: stays a branch
#pragma unroll
        for (int e = 0; e < NT; ++e) {
          const float e2 = fast_exp2(t[e] * inv_cap2);
          t[e] = p.softcap * (1.0f - 2.0f * __builtin_amdgcn_rcpf(e2 + 1.0f));
        }
      }
#pragma unroll
      for (int e = 0; e < NT; ++e) {
        const int tok = ci * CT + (e >> 2) * kTileTokens + 4 * r + (e & 3);
        const float x = t[e] * kLog2e + slope_log2 * (float)(tok - col_last);
        t[e] = (tok < first_visible || tok > col_last) ? -INFINITY : x;
      }
    } else {
#pragma unroll
      for (int e = 0; e < NT; ++e) t[e] = s.v[e >> 2][e & 3] * p.score_scale_log2;
    }
    if constexpr (CHECK_TAIL) {
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
    mt = fmaxf(mt, mx);
    // the reference follows when some column's has fallen too far behind (on the first chunk: has
    // none yet, inf > slack; a column that has seen nothing so far: -inf - -inf = NaN, no)
    // (per-block V scales ride on the probabilities and may be large: no slack to spare there)
    const float slack = (MASKS && KV8 && p.kv_scale_mode == kScaleBlock) ? 0.f : kRescaleSlack;
    // (unlikely: where the accumulators live in AGPRs the copies to and from VGPRs that this
    // block needs are then placed inside it, not in front of the branch)
    if (__builtin_expect(__any(mt - m > slack), 0)) {
      // MASKS: a column may see nothing of a chunk (a query token before the chunk's keys)
      // and nothing before it either; subtract 0 then, so that -inf stays -inf, not NaN
      if (__any(m != -INFINITY)) {  // on an item's first chunk (without sinks) sums and accumulators are still zero
        const float m_to = (MASKS && mt == -INFINITY) ? 0.f : mt;
        const float alpha = fast_exp2(m - m_to);  // exp2(-inf) = 0 for a column that has seen nothing so far
        l *= alpha;
        if constexpr (ACC_IN_AGPRS) {
#pragma unroll
          for (int dt = 0; dt < NDT; ++dt) {
            f32x4 t;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              // Read where it is used: a plain read is hoisted in front of the branch.  (The MFMAs that
              // wrote these registers, P.V of the chunk before, lie a whole score pass back: no MFMA
              // result is still on its way.)
              float x;
              asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(x) : "a"(acc[dt][e]));
              t[e] = x * alpha;
            }
            acc[dt] = t;
            asm volatile("" : "+a"(acc[dt]));
          }
        } else {
#pragma unroll
          for (int dt = 0; dt < NDT; ++dt) acc[dt] *= alpha;
        }
      }
      m = mt;
    }
    const float m_sub = (MASKS && m == -INFINITY) ? 0.f : m;
    float ps = 0.f;
#pragma unroll
    for (int e = 0; e < NT; ++e) {
      t[e] = fast_exp2(t[e] - m_sub);
      ps += t[e];
    }
    l += ps;
    // k-slots (r, e) of step pr = this lane's eight tokens of the step, rounded to the q
    // dtype (paged_attention_kernel_loop.hpp:404-407)
    if constexpr (MASKS && KV8) {  // per-block V scales ride on the probabilities
      if (p.kv_scale_mode == kScaleBlock) {
        // by select: a tile past the context takes its block id from a clamped or unused table
        // column, and the scale of a block nobody wrote may be anything, NaN included
#pragma unroll
        for (int e = 0; e < NT; ++e) t[e] = t[e] == 0.f ? 0.f : t[e] * ts->v[e >> 2];
      }
    }
    Probs pb;
#pragma unroll
    for (int pr = 0; pr < NP2; ++pr)
#pragma unroll
      for (int c = 0; c < 4; ++c) pb.v[pr][c] = pack2<QT>(t[pr * 8 + 2 * c], t[pr * 8 + 2 * c + 1]);
    return pb;
  }

  __device__ __forceinline__ void pv(const Chunk &R, const Probs &pb) {
#pragma unroll
    for (int pr = 0; pr < NP2; ++pr)
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt)
        acc[dt] = mfma_16x16x32<QT>(v_operand(R, pr, dt), pb.v[pr], acc[dt]);
  }

  // Two column tiles held by ONE wavefront (a and b: the same chunk, different 16 columns) share
  // the K and V operands: every operand is built once and feeds both tiles' MFMAs.
  // `between(slot)` is called after the MFMAs of every (k-step, tile) pair, slot = c * TPC + t, and
  // after those of every d-tile, slot = pr * NDT + dt: where a kernel places the loads of other chunks.
  template <typename F>
  static __device__ __forceinline__ void qk_two(const WaveAttn &a, const WaveAttn &b, Chunk &R, Scores &sa, Scores &sb,
                                                F &&between) {
    if constexpr (kRowLoads) {
#pragma unroll
      for (int t = 0; t < TPC; ++t)
#pragma unroll
        for (int c = 0; c < KL; c += 2) k_rows_to_mfma(R.k[t][c], R.k[t][c + 1]);
    }
#pragma unroll
    for (int t = 0; t < TPC; ++t) sa.v[t] = sb.v[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < KSTEPS; ++c)
#pragma unroll
      for (int t = 0; t < TPC; ++t) {
        const u32x4 ko = a.k_operand(R, t, c);
        sa.v[t] = mfma_16x16x32<QT>(ko, a.qB[c], sa.v[t]);
        sb.v[t] = mfma_16x16x32<QT>(ko, b.qB[c], sb.v[t]);
        between(c * TPC + t);
      }
  }
  template <typename F>
  static __device__ __forceinline__ void pv_two(WaveAttn &a, WaveAttn &b, const Chunk &R, const Probs &pa, const Probs &pb,
                                                F &&between) {
#pragma unroll
    for (int pr = 0; pr < NP2; ++pr)
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) {
        const u32x4 vo = a.v_operand(R, pr, dt);
        a.acc[dt] = mfma_16x16x32<QT>(vo, pa.v[pr], a.acc[dt]);
        b.acc[dt] = mfma_16x16x32<QT>(vo, pb.v[pr], b.acc[dt]);
        between(pr * NDT + dt);
      }
  }
  static __device__ __forceinline__ void qk_two(const WaveAttn &a, const WaveAttn &b, Chunk &R, Scores &sa, Scores &sb) {
    qk_two(a, b, R, sa, sb, [](int) {});
  }
  static __device__ __forceinline__ void pv_two(WaveAttn &a, WaveAttn &b, const Chunk &R, const Probs &pa, const Probs &pb) {
    pv_two(a, b, R, pa, pb, [](int) {});
  }

  // A lane's NR accumulator values are NR consecutive head-dim elements of head i:
  // d = 4r*NDT + idx with idx = e*NDT + dt.
  __device__ __forceinline__ float acc_at(int idx) const { return acc[idx % NDT][idx / NDT]; }

  // Store `n` normalised fp32 values starting at head-dim element d0 of one tmp_out row.
  template <int N>
  static __device__ __forceinline__ void store_f32(float *dst, const float (&o)[N], float inv) {
    if constexpr (N % 4 == 0) {
#pragma unroll
      for (int k = 0; k < N; k += 4) {
        f32x4 v = {o[k] * inv, o[k + 1] * inv, o[k + 2] * inv, o[k + 3] * inv};
        *reinterpret_cast<f32x4 *>(dst + k) = v;
      }
    } else {
#pragma unroll
      for (int k = 0; k < N; ++k) dst[k] = o[k] * inv;
    }
  }

  // Store `n` normalised values rounded to the q dtype.
  template <int N>
  static __device__ __forceinline__ void store_q(char *dst, const float (&o)[N], float inv) {
    uint32_t w2[N / 2];
#pragma unroll
    for (int k = 0; k < N / 2; ++k) w2[k] = pack2<QT>(o[2 * k] * inv, o[2 * k + 1] * inv);
    if constexpr (N % 8 == 0) {
#pragma unroll
      for (int k = 0; k < N / 2; k += 4) {
        u32x4 v = {w2[k], w2[k + 1], w2[k + 2], w2[k + 3]};
        *reinterpret_cast<u32x4 *>(dst + k * 4) = v;
      }
    } else if constexpr (N % 4 == 0) {
#pragma unroll
      for (int k = 0; k < N / 2; k += 2) {
        u32x2 v = {w2[k], w2[k + 1]};
        *reinterpret_cast<u32x2 *>(dst + k * 4) = v;
      }
    } else {
#pragma unroll
      for (int k = 0; k < N / 2; ++k) *reinterpret_cast<uint32_t *>(dst + k * 4) = w2[k];
    }
  }
};

}  // namespace fa
