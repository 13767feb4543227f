/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the paged-attention decode path.
 *
 * This file is the checker, never the product: only tests/, the smoke check and
 * the bench's cpu_baseline leg may build, load or call it.  The shipped path is
 * the HIP library; nothing in the package falls back to this code.
 *
 * Two groups of functions live here.
 *
 * (1) oracle_attention_ref  -- a restatement of the PyTorch reference the
 *     upstream tests compare their kernels with
 *     (reference test_paged.py:79-123,165-168 `attention_ref`, the paged gather of
 *     test_paged.py:170-194 `_generate_block_kvcache`, and the fp8 form
 *     test_paged_fp8cache.py:80-81 which dequantises the cache before the same
 *     maths).  It works per (sequence, kv head) straight from the paged pool, so
 *     no padded [S, max_ctx, H, D] tensor is ever built.
 *
 * (2) oracle_kernel_loop / oracle_kernel_partition / oracle_kernel_reduce -- a
 *     restatement of the arithmetic of the upstream device kernels, including
 *     their rounding points:
 *       loop kernel      paged_attention_loop/paged_attention_kernel_loop.hpp:610-636
 *                        (scores :227-348, online softmax :353-444, PV :455-546,
 *                        final divide :550-586)
 *       partition kernel paged_attention_reduce/paged_attention_kernel_v2.hpp:572-587
 *                        (softmax normalised inside the partition :342-447,
 *                        tmp_out :452-547)
 *       reduce kernel    paged_attention_reduce/paged_attention_kernel_v2.hpp:957-969
 *                        (rescale_exp_sums :736-764, compute_out :771-864)
 *       fp8 deltas       paged_attention_fp8_loop/paged_attention_kernel_fp8_loop.hpp:328-333,540-545
 *     tmp_out is kept in fp32 here (the upstream stores it in the query dtype).
 *
 * Pinning status (what fixes each function beyond its own formula):
 *   oracle_attention_ref     pinned by tests/test_oracle_*.py against
 *                            torch.nn.functional.scaled_dot_product_attention, a
 *                            float64 brute force, closed forms and invariants.
 *   oracle_kernel_*          pinned against oracle_attention_ref through the
 *                            split-invariance of log-sum-exp and by closed forms.
 *   e5m2 / e4m3 decode       pinned on all 256 codes against torch.float8_e5m2 /
 *                            torch.float8_e4m3fn.
 *   oracle_attention_ref_masked  soft-capping, local window and ALiBi: pinned against SDPA
 *                            with an additive bias / mask and against plain torch ops for
 *                            the tanh cap (tests/test_oracle_masks.py).  Upstream's KERNELS
 *                            do not implement these (the code is commented out there).
 *   oracle_attention_ref_scaled  per-head / per-block K and V scales of an FP8 cache:
 *                            PARITY UNPINNED against upstream, which has nothing of the
 *                            kind; the reading K^ = dequant(K)*k_scale, V^ = dequant(V)*v_scale
 *                            is pinned against SDPA over tensors dequantised, scaled and
 *                            gathered with torch indexing (tests/test_oracle_kv_scales.py).
 *   fp8_scale != 1           PARITY UNPINNED: the upstream tests only ever pass
 *                            1.0 (test_paged_fp8cache.py:489,510); the reading
 *                            implemented is K^ = dequant(K)*s, V^ = dequant(V)*s.
 *
 * The upstream kernels cannot be compiled here (SYCL-ESIMD + XeTLA, Intel only), so
 * there is no oracle/_ref build for this path.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))
#define CLONES __attribute__((target_clones("avx2", "default")))

enum { ORACLE_Q_F16 = 0, ORACLE_Q_BF16 = 1 };
enum { ORACLE_KV_SAME_AS_Q = 0, ORACLE_KV_E5M2 = 1, ORACLE_KV_E4M3 = 2 };

/* ------------------------------------------------------------------ */
/* 16-bit and 8-bit float formats, bit exact, round-to-nearest-even     */
/* ------------------------------------------------------------------ */

static inline float bits_to_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static inline uint32_t f32_to_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}

ORACLE_API float oracle_f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu;
  uint32_t man = h & 0x3FFu;
  if (exp == 0) {
    if (man == 0) return bits_to_f32(sign);
    /* subnormal: value = man * 2^-24 */
    float v = (float)man * 5.9604644775390625e-08f;
    return sign ? -v : v;
  }
  if (exp == 31) return bits_to_f32(sign | 0x7F800000u | (man << 13));
  return bits_to_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

ORACLE_API uint16_t oracle_f32_to_f16(float f) {
  uint32_t x = f32_to_bits(f);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t ax = x & 0x7FFFFFFFu;
  if (ax >= 0x7F800000u) { /* inf / nan */
    if (ax > 0x7F800000u) return (uint16_t)(sign | 0x7E00u);
    return (uint16_t)(sign | 0x7C00u);
  }
  if (ax >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u); /* rounds to inf */
  if (ax < 0x33000001u) return (uint16_t)sign;             /* rounds to zero (<= 2^-25) */
  int32_t e = (int32_t)(ax >> 23) - 127;
  uint32_t m = (ax & 0x7FFFFFu) | 0x800000u; /* 24-bit significand */
  uint32_t shift, half_exp;
  if (e < -14) { /* subnormal result */
    shift = (uint32_t)(13 + (-14 - e));
    half_exp = 0;
  } else {
    shift = 13;
    half_exp = (uint32_t)(e + 15);
  }
  uint32_t q = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (q & 1u))) q++;
  uint32_t out;
  if (half_exp == 0) {
    out = q; /* may carry into exponent 1: correct by construction */
  } else {
    out = ((half_exp - 1u) << 10) + q; /* q carries the implicit 1 at bit 10 */
  }
  return (uint16_t)(sign | out);
}

ORACLE_API float oracle_bf16_to_f32(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }

ORACLE_API uint16_t oracle_f32_to_bf16(float f) {
  uint32_t x = f32_to_bits(f);
  if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((x >> 16) | 0x0040u);
  uint32_t lsb = (x >> 16) & 1u;
  x += 0x7FFFu + lsb;
  return (uint16_t)(x >> 16);
}

/* E5M2 is binary16 cut down to its top byte, so decoding is a byte shift. */
ORACLE_API float oracle_e5m2_to_f32(uint8_t b) { return oracle_f16_to_f32((uint16_t)((uint16_t)b << 8)); }

/* E4M3 ("fn": finite numbers and NaN only): 1 sign, 4 exponent bits with bias 7, 3 mantissa
 * bits; exponent 15 with mantissa 7 is NaN, everything else is a number (largest 448);
 * exponent 0 holds the subnormals m * 2^-9.  The format upstream's FP8 kernels carry as a
 * template parameter next to E5M2 (paged_attention_kernel_fp8_loop.hpp:42). */
ORACLE_API float oracle_e4m3_to_f32(uint8_t b) {
  const int sign = b >> 7, e = (b >> 3) & 15, m = b & 7;
  float v;
  if (e == 15 && m == 7) return bits_to_f32(sign ? 0xFFC00000u : 0x7FC00000u);
  if (e == 0) v = (float)m * 0.001953125f; /* m * 2^-9 */
  else v = ldexpf((float)(8 + m), e - 10); /* (1 + m/8) * 2^(e-7) */
  return sign ? -v : v;
}

static inline float load16(const uint16_t *p, int q_dtype) {
  return q_dtype == ORACLE_Q_BF16 ? oracle_bf16_to_f32(*p) : oracle_f16_to_f32(*p);
}
static inline uint16_t round16(float f, int q_dtype) {
  return q_dtype == ORACLE_Q_BF16 ? oracle_f32_to_bf16(f) : oracle_f32_to_f16(f);
}
static inline float roundtrip16(float f, int q_dtype) {
  uint16_t h = round16(f, q_dtype);
  return q_dtype == ORACLE_Q_BF16 ? oracle_bf16_to_f32(h) : oracle_f16_to_f32(h);
}

/* ------------------------------------------------------------------ */
/* Problem description shared by every entry point                      */
/* ------------------------------------------------------------------ */

typedef struct {
  int32_t num_seqs, num_heads, num_kv_heads, head_size, block_size;
  int32_t max_blocks_per_seq;
  int64_t kv_block_stride, kv_token_stride, kv_head_stride; /* in elements */
  int32_t q_dtype;  /* ORACLE_Q_*  */
  int32_t kv_dtype; /* ORACLE_KV_* */
  float scale;      /* softmax scale applied to q.k */
  float fp8_scale;  /* per-tensor dequant scale, 1.0 for 16-bit caches */
} oracle_problem;

/* Gather one (sequence, kv head)'s first n tokens of a cache into dense fp32
 * rows [n][D] (reference test_paged.py:184-193 does the same with fancy
 * indexing on the whole pool). */
/* `scales` NULL: every row is multiplied by p->fp8_scale.  Otherwise by
 * scales[blk * scale_block_pitch + kv_head]: per-head scales with pitch 0, per physical
 * block and kv head with pitch num_kv_heads (FP8 caches only). */
CLONES static void gather_rows_scaled(float *dst, const void *cache, const int32_t *table, int n,
                                      int kv_head, const oracle_problem *p, const float *scales,
                                      int scale_block_pitch) {
  const int D = p->head_size, B = p->block_size;
  for (int t = 0; t < n; ++t) {
    int64_t blk = table[t / B];
    const float mul = scales ? scales[blk * scale_block_pitch + kv_head] : p->fp8_scale;
    int64_t off = blk * p->kv_block_stride + (int64_t)(t % B) * p->kv_token_stride +
                  (int64_t)kv_head * p->kv_head_stride;
    float *row = dst + (size_t)t * D;
    if (p->kv_dtype == ORACLE_KV_E5M2) {
      const uint8_t *src = (const uint8_t *)cache + off;
      for (int d = 0; d < D; ++d) row[d] = oracle_e5m2_to_f32(src[d]) * mul;
    } else if (p->kv_dtype == ORACLE_KV_E4M3) {
      const uint8_t *src = (const uint8_t *)cache + off;
      for (int d = 0; d < D; ++d) row[d] = oracle_e4m3_to_f32(src[d]) * mul;
    } else {
      const uint16_t *src = (const uint16_t *)cache + off;
      if (p->q_dtype == ORACLE_Q_BF16)
        for (int d = 0; d < D; ++d) row[d] = oracle_bf16_to_f32(src[d]);
      else
        for (int d = 0; d < D; ++d) row[d] = oracle_f16_to_f32(src[d]);
    }
  }
}

static void gather_rows(float *dst, const void *cache, const int32_t *table, int n, int kv_head,
                        const oracle_problem *p) {
  gather_rows_scaled(dst, cache, table, n, kv_head, p, NULL, 0);
}

CLONES static float dot_f32(const float *a, const float *b, int n) {
  float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  int i = 0;
  for (; i + 8 <= n; i += 8)
    for (int j = 0; j < 8; ++j) acc[j] += a[i + j] * b[i + j];
  float s = ((acc[0] + acc[4]) + (acc[1] + acc[5])) + ((acc[2] + acc[6]) + (acc[3] + acc[7]));
  for (; i < n; ++i) s += a[i] * b[i];
  return s;
}

CLONES static void axpy_f32(float *y, float a, const float *x, int n) {
  for (int i = 0; i < n; ++i) y[i] += a * x[i];
}

/* ------------------------------------------------------------------ */
/* (1) The tests' PyTorch reference                                     */
/* ------------------------------------------------------------------ */

/*
 * out[S,H,D] (16-bit, q dtype) and optionally out_f32[S,H,D] (before the final
 * cast) = softmax((q*scale) . K^T  [+ sink column]) . V over the first
 * context_lens[s] tokens of each sequence.
 *   scores      test_paged.py:89   (q scaled in fp32 BEFORE the dot)
 *   length mask test_paged.py:96-97
 *   softmax     test_paged.py:112-123 (sink only enters max and denominator)
 *   output      test_paged.py:165,168
 * sinks may be NULL; its entries are in the q dtype.
 * Returns 0, or -1 on allocation failure.
 */
/* The score modifiers of the upstream reference that its kernels leave out (commented-out
 * code, paged_attention_kernel_loop.hpp:329-342) but its attention_ref defines
 * (test_paged.py:92-110): soft-capping cap*tanh(s/cap) of the scaled scores, then the local
 * window -- a decode query at position n-1 sees keys n-1-window_left .. n-1 -- then the
 * ALiBi bias -slope_h * (n-1-t).  softcap <= 0, window_left < 0 and a NULL slope array each
 * switch their modifier off. */
typedef struct {
  const float *alibi_slopes; /* [num_heads] or NULL */
  float softcap;
  int32_t window_left;
  int32_t query_len; /* query tokens per sequence (speculative decoding, chunked prefill):
                        query and out are [num_seqs, query_len, num_heads, head_size]; the
                        query tokens are the LAST query_len positions of the context (their
                        K/V rows are in the cache) and each sees the keys up to its own
                        position -- upstream's causal rule, key j visible to query i iff
                        j <= i + seqlen_k - seqlen_q (test_paged.py:79-80 with the local mask
                        of :98-109).  1 = plain decode. */
  /* Finer dequantisation scales of an FP8 cache (upstream has the one scalar fp8_scale):
   * K^ = dequant(K) * k_scales[..], V^ = dequant(V) * v_scales[..], indexed
   * [blk * scale_block_pitch + kv_head].  NULL = p->fp8_scale. */
  const float *k_scales;
  const float *v_scales;
  int32_t scale_block_pitch;
} oracle_masks;

static int attention_ref_core(uint16_t *out, float *out_f32, const uint16_t *query,
                              const void *key_cache, const void *value_cache,
                              const int32_t *block_tables, const int32_t *context_lens,
                              const uint16_t *sinks, const oracle_problem *p, const oracle_masks *mk) {
  const int S = p->num_seqs, H = p->num_heads, Hk = p->num_kv_heads, D = p->head_size;
  const int G = H / Hk;
  int failed = 0;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
  for (int s = 0; s < S; ++s) {
    for (int kh = 0; kh < Hk; ++kh) {
      const int n_all = context_lens[s];
      const int QL = mk && mk->query_len > 1 ? mk->query_len : 1;
      if (n_all <= 0) continue;
      float *K = (float *)malloc((size_t)n_all * D * sizeof(float));
      float *V = (float *)malloc((size_t)n_all * D * sizeof(float));
      float *sc = (float *)malloc((size_t)n_all * sizeof(float));
      float *qf = (float *)malloc((size_t)D * sizeof(float));
      float *acc = (float *)malloc((size_t)D * sizeof(float));
      if (!K || !V || !sc || !qf || !acc) {
        failed = 1;
      } else {
        const int32_t *table = block_tables + (size_t)s * p->max_blocks_per_seq;
        gather_rows_scaled(K, key_cache, table, n_all, kh, p, mk ? mk->k_scales : NULL,
                           mk ? mk->scale_block_pitch : 0);
        gather_rows_scaled(V, value_cache, table, n_all, kh, p, mk ? mk->v_scales : NULL,
                           mk ? mk->scale_block_pitch : 0);
        for (int qg = 0; qg < QL * G; ++qg) {
          const int qt = qg / G, g = qg % G;
          const int n = n_all - QL + qt + 1; /* keys this query token sees */
          if (n <= 0) continue;
          const int h = kh * G + g;
          const uint16_t *qrow = query + (((size_t)s * QL + qt) * H + h) * D;
          for (int d = 0; d < D; ++d) qf[d] = load16(qrow + d, p->q_dtype) * p->scale;
          float m = -INFINITY;
          for (int t = 0; t < n; ++t) {
            float x = dot_f32(qf, K + (size_t)t * D, D);
            if (mk && mk->softcap > 0.f) x = mk->softcap * tanhf(x / mk->softcap);
            if (mk && mk->window_left >= 0 && t < n - 1 - mk->window_left) x = -INFINITY;
            if (mk && mk->alibi_slopes) x -= mk->alibi_slopes[h] * (float)(n - 1 - t);
            sc[t] = x;
            if (sc[t] > m) m = sc[t];
          }
          float sink_term = 0.f;
          if (sinks) {
            float sk = load16(sinks + h, p->q_dtype);
            if (sk > m) m = sk;
            sink_term = expf(sk - m);
          }
          float denom = 0.f;
          for (int t = 0; t < n; ++t) {
            sc[t] = expf(sc[t] - m);
            denom += sc[t];
          }
          denom += sink_term;
          for (int d = 0; d < D; ++d) acc[d] = 0.f;
          for (int t = 0; t < n; ++t) axpy_f32(acc, sc[t] / denom, V + (size_t)t * D, D);
          size_t o = (((size_t)s * QL + qt) * H + h) * D;
          for (int d = 0; d < D; ++d) {
            if (out_f32) out_f32[o + d] = acc[d];
            if (out) out[o + d] = round16(acc[d], p->q_dtype);
          }
        }
      }
      free(K); free(V); free(sc); free(qf); free(acc);
    }
  }
  return failed ? -1 : 0;
}

ORACLE_API int oracle_attention_ref(uint16_t *out, float *out_f32, const uint16_t *query,
                                    const void *key_cache, const void *value_cache,
                                    const int32_t *block_tables, const int32_t *context_lens,
                                    const uint16_t *sinks, const oracle_problem *p) {
  return attention_ref_core(out, out_f32, query, key_cache, value_cache, block_tables, context_lens,
                            sinks, p, NULL);
}

ORACLE_API int oracle_attention_ref_masked(uint16_t *out, float *out_f32, const uint16_t *query,
                                           const void *key_cache, const void *value_cache,
                                           const int32_t *block_tables, const int32_t *context_lens,
                                           const uint16_t *sinks, const float *alibi_slopes,
                                           float softcap, int32_t window_left, int32_t query_len,
                                           const oracle_problem *p) {
  oracle_masks mk = {alibi_slopes, softcap, window_left, query_len, NULL, NULL, 0};
  return attention_ref_core(out, out_f32, query, key_cache, value_cache, block_tables, context_lens,
                            sinks, p, &mk);
}

/* The same with per-head (scale_block_pitch 0) or per-block (scale_block_pitch num_kv_heads)
 * K and V scales of an FP8 cache in place of p->fp8_scale. */
ORACLE_API int oracle_attention_ref_scaled(uint16_t *out, float *out_f32, const uint16_t *query,
                                           const void *key_cache, const void *value_cache,
                                           const int32_t *block_tables, const int32_t *context_lens,
                                           const uint16_t *sinks, const float *alibi_slopes,
                                           float softcap, int32_t window_left, int32_t query_len,
                                           const float *k_scales, const float *v_scales,
                                           int32_t scale_block_pitch, const oracle_problem *p) {
  oracle_masks mk = {alibi_slopes, softcap, window_left, query_len, k_scales, v_scales, scale_block_pitch};
  return attention_ref_core(out, out_f32, query, key_cache, value_cache, block_tables, context_lens,
                            sinks, p, &mk);
}

/* ------------------------------------------------------------------ */
/* (2) The device kernels' arithmetic                                   */
/* ------------------------------------------------------------------ */

/* Scores of one partition: fp32 dot of the raw 16-bit inputs, THEN the scale
 * (paged_attention_kernel_loop.hpp:309-321; the fp8 kernel multiplies by
 * sm_scale*fp8_scale at paged_attention_kernel_fp8_loop.hpp:333).  Rows here
 * hold the dequantised values WITHOUT fp8_scale. */
static void partition_scores(float *sc, const float *qf, const float *K, int t0, int t1, int D,
                             float scale) {
  for (int t = t0; t < t1; ++t) sc[t - t0] = dot_f32(qf, K + (size_t)t * D, D) * scale;
}

/*
 * Single-pass loop kernel: serial walk over partitions of `partition_size`
 * tokens with an online softmax (paged_attention_kernel_loop.hpp:620-636).
 * Probabilities are rounded to the q dtype before the PV product (:404-407),
 * the running sum uses the unrounded values (:397-401), the sink joins only
 * partition 0 (:387-391) and the result is acc * (1/l) (:559-566 via
 * paged_attention_utils.hpp:834-835).
 */
ORACLE_API int oracle_kernel_loop(uint16_t *out, float *out_f32, const uint16_t *query,
                                  const void *key_cache, const void *value_cache,
                                  const int32_t *block_tables, const int32_t *context_lens,
                                  const uint16_t *sinks, int partition_size,
                                  const oracle_problem *p) {
  const int S = p->num_seqs, H = p->num_heads, Hk = p->num_kv_heads, D = p->head_size;
  const int G = H / Hk;
  oracle_problem raw = *p;
  raw.fp8_scale = 1.0f; /* rows without the scale; folded in after the dots */
  const float kscale = p->kv_dtype != ORACLE_KV_SAME_AS_Q ? p->scale * p->fp8_scale : p->scale;
  const float vscale = p->kv_dtype != ORACLE_KV_SAME_AS_Q ? p->fp8_scale : 1.0f;
  int failed = 0;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
  for (int s = 0; s < S; ++s) {
    for (int kh = 0; kh < Hk; ++kh) {
      const int n = context_lens[s];
      if (n <= 0) continue;
      float *K = (float *)malloc((size_t)n * D * sizeof(float));
      float *V = (float *)malloc((size_t)n * D * sizeof(float));
      float *sc = (float *)malloc((size_t)partition_size * sizeof(float));
      float *qf = (float *)malloc((size_t)D * sizeof(float));
      float *acc = (float *)malloc((size_t)D * sizeof(float));
      float *cur = (float *)malloc((size_t)D * sizeof(float));
      if (!K || !V || !sc || !qf || !acc || !cur) {
        failed = 1;
      } else {
        const int32_t *table = block_tables + (size_t)s * p->max_blocks_per_seq;
        gather_rows(K, key_cache, table, n, kh, &raw);
        gather_rows(V, value_cache, table, n, kh, &raw);
        for (int g = 0; g < G; ++g) {
          const int h = kh * G + g;
          const uint16_t *qrow = query + ((size_t)s * H + h) * D;
          for (int d = 0; d < D; ++d) qf[d] = load16(qrow + d, p->q_dtype);
          const float sink = sinks ? load16(sinks + h, p->q_dtype) : -INFINITY;
          float m_old = -INFINITY, l_old = 0.f;
          for (int d = 0; d < D; ++d) acc[d] = 0.f;
          const int nparts = (n + partition_size - 1) / partition_size;
          for (int pi = 0; pi < nparts; ++pi) {
            const int t0 = pi * partition_size;
            const int t1 = t0 + partition_size < n ? t0 + partition_size : n;
            partition_scores(sc, qf, K, t0, t1, D, kscale);
            float m = -INFINITY;
            for (int t = 0; t < t1 - t0; ++t)
              if (sc[t] > m) m = sc[t];
            const float sk = pi == 0 ? sink : -INFINITY;
            if (sk > m) m = sk;
            const float m_new = m_old > m ? m_old : m;
            float l = 0.f;
            for (int d = 0; d < D; ++d) cur[d] = 0.f;
            for (int t = 0; t < t1 - t0; ++t) {
              float e = expf(sc[t] - m_new);
              l += e;
              axpy_f32(cur, roundtrip16(e, p->q_dtype), V + (size_t)(t0 + t) * D, D);
            }
            l += expf(sk - m_new); /* exp(-inf) = 0 when there is no sink */
            const float r = expf(m_old - m_new);
            l_old = r * l_old + l;
            m_old = m_new;
            for (int d = 0; d < D; ++d) acc[d] = acc[d] * r + cur[d] * vscale;
          }
          const float inv = 1.0f / l_old;
          size_t o = ((size_t)s * H + h) * D;
          for (int d = 0; d < D; ++d) {
            float v = acc[d] * inv;
            if (out_f32) out_f32[o + d] = v;
            if (out) out[o + d] = round16(v, p->q_dtype);
          }
        }
      }
      free(K); free(V); free(sc); free(qf); free(acc); free(cur);
    }
  }
  return failed ? -1 : 0;
}

/*
 * Split-context attention kernel: one independent softmax per partition
 * (paged_attention_kernel_v2.hpp:572-587).  For partition pi of sequence s and
 * head h it stores
 *   max_logits[s,h,pi] = m   = max(scores, sink if pi == 0)          (:373-376,432)
 *   exp_sums[s,h,pi]   = l   = sum exp(score - m) + exp(sink - m)    (:381-385,441)
 *   tmp_out[s,h,pi,:]  = sum_t round16(exp(score_t - m) / l) * V[t]  (:386-397,498-546)
 * Partitions at or beyond ceil(ctx/partition_size) are left untouched (:577-579).
 * Scratch arrays have `max_num_partitions` slots per (s,h).
 */
ORACLE_API int oracle_kernel_partition(float *exp_sums, float *max_logits, float *tmp_out,
                                       const uint16_t *query, const void *key_cache,
                                       const void *value_cache, const int32_t *block_tables,
                                       const int32_t *context_lens, const uint16_t *sinks,
                                       int partition_size, int max_num_partitions,
                                       const oracle_problem *p) {
  const int S = p->num_seqs, H = p->num_heads, Hk = p->num_kv_heads, D = p->head_size;
  const int G = H / Hk;
  oracle_problem raw = *p;
  raw.fp8_scale = 1.0f;
  const float kscale = p->kv_dtype != ORACLE_KV_SAME_AS_Q ? p->scale * p->fp8_scale : p->scale;
  const float vscale = p->kv_dtype != ORACLE_KV_SAME_AS_Q ? p->fp8_scale : 1.0f;
  int failed = 0;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
  for (int s = 0; s < S; ++s) {
    for (int kh = 0; kh < Hk; ++kh) {
      const int n = context_lens[s];
      if (n <= 0) continue;
      float *K = (float *)malloc((size_t)n * D * sizeof(float));
      float *V = (float *)malloc((size_t)n * D * sizeof(float));
      float *sc = (float *)malloc((size_t)partition_size * sizeof(float));
      float *qf = (float *)malloc((size_t)D * sizeof(float));
      float *cur = (float *)malloc((size_t)D * sizeof(float));
      if (!K || !V || !sc || !qf || !cur) {
        failed = 1;
      } else {
        const int32_t *table = block_tables + (size_t)s * p->max_blocks_per_seq;
        gather_rows(K, key_cache, table, n, kh, &raw);
        gather_rows(V, value_cache, table, n, kh, &raw);
        int nparts = (n + partition_size - 1) / partition_size;
        if (nparts > max_num_partitions) nparts = max_num_partitions;
        for (int g = 0; g < G; ++g) {
          const int h = kh * G + g;
          const uint16_t *qrow = query + ((size_t)s * H + h) * D;
          for (int d = 0; d < D; ++d) qf[d] = load16(qrow + d, p->q_dtype);
          const float sink = sinks ? load16(sinks + h, p->q_dtype) : -INFINITY;
          for (int pi = 0; pi < nparts; ++pi) {
            const int t0 = pi * partition_size;
            const int t1 = t0 + partition_size < n ? t0 + partition_size : n;
            partition_scores(sc, qf, K, t0, t1, D, kscale);
            float m = -INFINITY;
            for (int t = 0; t < t1 - t0; ++t)
              if (sc[t] > m) m = sc[t];
            const float sk = pi == 0 ? sink : -INFINITY;
            if (sk > m) m = sk;
            float l = 0.f;
            for (int t = 0; t < t1 - t0; ++t) {
              sc[t] = expf(sc[t] - m);
              l += sc[t];
            }
            l += expf(sk - m);
            for (int d = 0; d < D; ++d) cur[d] = 0.f;
            for (int t = 0; t < t1 - t0; ++t)
              axpy_f32(cur, roundtrip16(sc[t] / l, p->q_dtype), V + (size_t)(t0 + t) * D, D);
            size_t slot = ((size_t)s * H + h) * max_num_partitions + pi;
            max_logits[slot] = m;
            exp_sums[slot] = l;
            for (int d = 0; d < D; ++d) tmp_out[slot * D + d] = cur[d] * vscale;
          }
        }
      }
      free(K); free(V); free(sc); free(qf); free(cur);
    }
  }
  return failed ? -1 : 0;
}

/*
 * Reduce kernel (paged_attention_kernel_v2.hpp:957-969): over the
 * ceil(ctx/partition_size) live partitions of (s,h)
 *   M = max_p m_p;  w_p = l_p * exp(m_p - M)   (:736-764)
 *   out = sum_p (w_p / sum_q w_q) * tmp_out_p  (:816-861), cast to the q dtype (:930-932)
 */
ORACLE_API int oracle_kernel_reduce(uint16_t *out, float *out_f32, const float *exp_sums,
                                    const float *max_logits, const float *tmp_out,
                                    const int32_t *context_lens, int partition_size,
                                    int max_num_partitions, const oracle_problem *p) {
  const int S = p->num_seqs, H = p->num_heads, D = p->head_size;
#pragma omp parallel for collapse(2) schedule(static)
  for (int s = 0; s < S; ++s) {
    for (int h = 0; h < H; ++h) {
      const int n = context_lens[s];
      if (n <= 0) continue;
      int nparts = (n + partition_size - 1) / partition_size;
      if (nparts > max_num_partitions) nparts = max_num_partitions;
      const size_t base = ((size_t)s * H + h) * max_num_partitions;
      float M = -INFINITY;
      for (int pi = 0; pi < nparts; ++pi)
        if (max_logits[base + pi] > M) M = max_logits[base + pi];
      float W = 0.f;
      for (int pi = 0; pi < nparts; ++pi) W += exp_sums[base + pi] * expf(max_logits[base + pi] - M);
      const float inv = 1.0f / W;
      size_t o = ((size_t)s * H + h) * D;
      for (int d = 0; d < D; ++d) {
        float a = 0.f;
        for (int pi = 0; pi < nparts; ++pi) {
          float w = exp_sums[base + pi] * expf(max_logits[base + pi] - M) * inv;
          a += w * tmp_out[(base + pi) * D + d];
        }
        if (out_f32) out_f32[o + d] = a;
        if (out) out[o + d] = round16(a, p->q_dtype);
      }
    }
  }
  return 0;
}

ORACLE_API int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

ORACLE_API void oracle_set_num_threads(int n) {
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
#else
  (void)n;
#endif
}
