/*
 * C ABI of the MI355X paged-attention decode library (libfa_paged_attention.so).
 *
 * Four entry points, one per upstream host launcher.  Each replaces the pybind11
 * `run` function of one upstream extension module together with the dispatcher and
 * launcher underneath it:
 *
 *   fa_paged_attention_loop        paged_attention_loop/paged_attention_loop.cpp:21-84
 *                                  paged_attention_loop/launch_kernels_loop.h:16-173
 *   fa_paged_attention_reduce      paged_attention_reduce/paged_attention_reduce.cpp:21-84
 *                                  paged_attention_reduce/launch_kernels_reduce.h:18-197
 *   fa_paged_attention_fp8_loop    paged_attention_fp8_loop/paged_attention_fp8_loop.cpp:21-86
 *                                  paged_attention_fp8_loop/launch_kernels_fp8_loop.h:17-175
 *   fa_paged_attention_fp8_reduce  paged_attention_fp8_reduce/paged_attention_fp8_reduce.cpp:21-86
 *                                  paged_attention_fp8_reduce/launch_kernels_fp8_reduce.h:16-196
 *
 * All pointers except those in fa_paged_attention_options are DEVICE pointers owned
 * by the caller for the duration of the call; nothing is retained.  No exception
 * crosses this boundary: every function returns an fa_status and the text of the
 * last failure on the calling thread is available from fa_last_error().
 *
 * Tensor shapes (row-major, innermost dimension contiguous):
 *   out, query      [num_seqs, num_heads, head_size]            q_dtype (fp16 / bf16);
 *                   [num_seqs, query_len, num_heads, head_size] with options->query_len > 1
 *   key_cache,      a pool of blocks addressed with explicit element strides
 *   value_cache       element(block b, token t, kv head h, dim d) =
 *                       base[b*kv_block_stride + t*kv_token_stride + h*kv_head_stride + d]
 *                     16-bit caches hold q_dtype values, FP8 caches hold E5M2 bytes (as
 *                     upstream) or E4M3 bytes (options->kv_fp8_format).
 *                     upstream layout [blocks, block_size, kv_heads, head_size]
 *                       -> strides (block_size*kv_heads*head_size, kv_heads*head_size, head_size)
 *                     head-major layout [blocks, kv_heads, block_size, head_size]
 *                       -> strides (kv_heads*block_size*head_size, head_size, block_size*head_size)
 *   block_tables    [num_seqs, max_blocks_per_seq]              int32
 *   context_lens    [num_seqs]                                  int32
 *   exp_sums,       [num_seqs, num_heads, max_num_partitions]   fp32
 *   max_logits
 *   tmp_out         [num_seqs, num_heads, max_num_partitions, head_size]   fp32
 *                   (the upstream keeps tmp_out in the query dtype,
 *                    launch_kernels_reduce.h:20-21; fp32 drops one rounding step)
 *
 * Semantics follow the upstream kernels: query head h reads kv head
 * h / (num_heads / num_kv_heads); tokens at or beyond context_lens[s] never
 * contribute; an optional per-head sink logit joins the softmax denominator only;
 * alibi_slopes and softcap are accepted and ignored exactly as upstream
 * (paged_attention_kernel_loop.hpp:175-178,329-342 are commented out there) unless
 * options->mask_flags asks for them (see fa_mask below).
 * A sequence with context_lens[s] <= 0 leaves its rows of `out` untouched; a
 * context length above max_blocks_per_seq * block_size is cut to that bound, so the
 * kernels never read past a row of block_tables.
 *
 * Versioned structs.  fa_paged_attention_shape, fa_paged_attention_options and
 * fa_kv_cache_write_shape begin with `struct_size`, which the caller sets to sizeof of the
 * struct AS ITS HEADER DECLARES IT (the *_INIT macros do).  The library reads that many bytes and
 * takes every later field as zero, its default, so a caller built against an older revision of
 * this header keeps working when fields are appended; a size of 0, one that is not a multiple of
 * 4, one smaller than the fields a struct cannot do without (the shapes: all fields of revision 8;
 * the options: struct_size alone) or one larger than the library knows is FA_ERR_BAD_SHAPE.
 */
#ifndef FA_PAGED_ATTENTION_H_
#define FA_PAGED_ATTENTION_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum fa_status {
  FA_OK = 0,
  FA_ERR_NULL_POINTER = 1,
  /* upstream: std::runtime_error("Unsupported head size or block size"),
   * launch_kernels_loop.h:170-172 */
  FA_ERR_UNSUPPORTED_HEAD_OR_BLOCK_SIZE = 2,
  /* upstream: std::runtime_error("Unsupported number of queries per token"),
   * launch_kernels_loop.h:114-115 */
  FA_ERR_UNSUPPORTED_GROUP = 3,
  FA_ERR_UNSUPPORTED_DTYPE = 4,
  FA_ERR_PARTITION_OVERFLOW = 5, /* max_context_len needs more than max_num_partitions */
  FA_ERR_BAD_SHAPE = 6,          /* non-positive sizes, misaligned strides or pointers */
  FA_ERR_RUNTIME = 7,            /* a HIP call failed; see fa_last_error() */
  FA_ERR_SCRATCH_TOO_SMALL = 8   /* fa_paged_attention_reduce_static_scratch: the call needs more
                                    scratch than FA_STATIC_SCRATCH_BYTES */
} fa_status;

typedef enum fa_dtype { FA_DTYPE_F16 = 0, FA_DTYPE_BF16 = 1 } fa_dtype;

/* Byte format of an FP8 cache.  Upstream's FP8 kernels carry the format as a template
 * parameter (paged_attention_kernel_fp8_loop.hpp:42) and its entry points fix E5M2
 * (paged_attention_fp8_loop.cpp:43); E4M3 is the "fn" variant: bias 7, largest number 448,
 * no infinities, 0x7f / 0xff NaN. */
typedef enum fa_fp8_format { FA_FP8_E5M2 = 0, FA_FP8_E4M3 = 1 } fa_fp8_format;

/* Score modifiers upstream's kernels leave out (their code is commented out,
 * paged_attention_kernel_loop.hpp:329-342) but upstream's test reference defines
 * (test_paged.py:92-110), applied in its order: soft-capping softcap * tanh(s / softcap) of the
 * scaled scores, the local window, then the ALiBi bias -alibi_slopes[h] * (distance to the
 * query).  Opt-in: with mask_flags = 0 the entry points behave as upstream does. */
typedef enum fa_mask { FA_MASK_ALIBI = 1, FA_MASK_SOFTCAP = 2, FA_MASK_WINDOW = 4 } fa_mask;

/* Granularity of the dequantisation scales of an FP8 cache.  Upstream has one scalar for both
 * caches (fp8_scale, paged_attention_kernel_fp8_loop.hpp:328-333,540-545): FA_KV_SCALE_TENSOR.
 * The finer forms take separate K and V scales from device arrays:
 *   FA_KV_SCALE_HEAD   k_scales, v_scales [num_kv_heads] fp32
 *   FA_KV_SCALE_BLOCK  k_scales, v_scales [num_pool_blocks, num_kv_heads] fp32, one scale per
 *                      physical block and kv head (num_pool_blocks must be given)
 * K^ = dequant(K) * k_scale, V^ = dequant(V) * v_scale.  Scales must be finite and positive. */
/* How the work is laid over the GPU.  FA_SCHEDULE_AUTO picks the fastest form for the batch: for
 * batches of up to a few hundred sequences resident work-groups that walk the (sequence, kv head)
 * items -- and, in the split path, write one partial per SEGMENT of several partitions.
 * FA_SCHEDULE_GRID is upstream's own decomposition, one work-group per (sequence, kv head) and,
 * in the split path, per partition (paged_attention_kernel_loop.hpp:602-607,
 * paged_attention_kernel_v2.hpp:562-569): every live slot of exp_sums / max_logits / tmp_out then
 * holds exactly what upstream stores there.  FA_SCHEDULE_GRID_LDS is the grid form with K and V
 * staged through LDS by direct-to-LDS loads (FP8 entries, head size 128, no score modifiers;
 * anything else falls back to FA_SCHEDULE_GRID).  FA_SCHEDULE_SPLIT is FA_SCHEDULE_AUTO except that a
 * reduce entry always runs its two kernels, also where rows are so short that FA_SCHEDULE_AUTO runs the
 * single-pass kernel instead (fa_paged_attention_reduce_plan); loop entries take it as FA_SCHEDULE_AUTO.
 * FA_SCHEDULE_GRID_VALU and FA_SCHEDULE_VALU are the loop entries without the matrix cores: lane dot
 * products and fp32 multiply-adds, for query groups of ONE head (head size 128, fp16 queries, no score
 * modifiers or query tokens; anything else, and the reduce entries, run as FA_SCHEDULE_GRID) -- the first
 * in the grid form, the second as resident work-groups like FA_SCHEDULE_AUTO.  They are there to be
 * measured beside the matrix-core kernels, which the other schedules use for every group size and
 * which are as fast or faster in the resident form.
 * `out` is the same under all of them, to the tolerance of the path. */
typedef enum fa_schedule {
  FA_SCHEDULE_AUTO = 0, FA_SCHEDULE_GRID = 1, FA_SCHEDULE_GRID_LDS = 2, FA_SCHEDULE_SPLIT = 3,
  FA_SCHEDULE_GRID_VALU = 4, FA_SCHEDULE_VALU = 5
} fa_schedule;

typedef enum fa_kv_scale { FA_KV_SCALE_TENSOR = 0, FA_KV_SCALE_HEAD = 1, FA_KV_SCALE_BLOCK = 2 } fa_kv_scale;

/* Shapes and strides that upstream reads off the torch tensors
 * (paged_attention_loop.cpp:60-65) or fixes at compile time. */
typedef struct fa_paged_attention_shape {
  uint32_t struct_size;       /* sizeof(fa_paged_attention_shape) in the caller's header */
  int32_t num_seqs;
  int32_t num_heads;
  int32_t num_kv_heads;
  int32_t head_size;          /* 64 or 128 */
  int32_t block_size;         /* power of two, >= 16 */
  int32_t max_blocks_per_seq; /* row pitch of block_tables */
  int32_t max_num_partitions; /* slots per (seq, head) in the scratch arrays; loop entries ignore it */
  int32_t partition_size;     /* tokens per partition; 0 = upstream policy (512 for head 128,
                                 256 for head 64, include/paged_attention_policy_v2.hpp:28,50) */
  int64_t kv_block_stride;    /* in elements */
  int64_t kv_token_stride;
  int64_t kv_head_stride;
  int32_t q_dtype;            /* fa_dtype of query, out, sinks and of a 16-bit cache */
  int32_t num_pool_blocks;    /* blocks in each cache pool, or 0 if unknown.  When given, block ids
                                 read from block_tables are clamped into [0, num_pool_blocks) so a
                                 corrupt table cannot make the kernel touch memory outside the pool
                                 (upstream has no such guard) */
} fa_paged_attention_shape;
#define FA_PAGED_ATTENTION_SHAPE_INIT {(uint32_t)sizeof(fa_paged_attention_shape)}

/* Everything upstream's `run` takes beyond the result-affecting list, plus stream
 * and timing control.  A NULL options pointer means all defaults. */
typedef struct fa_paged_attention_options {
  uint32_t struct_size;       /* sizeof(fa_paged_attention_options) in the caller's header */
  const void *sinks;          /* device, [num_heads] in q_dtype, or NULL */
  const float *alibi_slopes;  /* device, [num_heads] fp32; ignored unless FA_MASK_ALIBI */
  float softcap;              /* ignored unless FA_MASK_SOFTCAP (then > 0) */
  float fp8_scale;            /* FP8 entries only: K^ = dequant(K)*s, V^ = dequant(V)*s; 0 means 1.0 */
  void *stream;               /* hipStream_t; NULL = the null stream */
  float *elapsed_us;          /* HOST pointer or NULL.  Non-NULL: the call synchronises and writes
                                 kernel times in microseconds, 1 float for loop entries,
                                 2 floats (attention, reduce) for reduce entries -- what the
                                 upstream `run` returns (launch_kernels_loop.h:53,
                                 launch_kernels_reduce.h:76-77).  NULL: asynchronous, no timing. */
  int32_t validate_only;      /* non-zero: check arguments, launch nothing */
  int32_t kv_fp8_format;      /* FP8 entries only: fa_fp8_format of the caches; 0 = E5M2 as upstream */
  int32_t mask_flags;         /* bit set of fa_mask: which score modifiers to APPLY.  0, the default,
                                 is upstream's behaviour: alibi_slopes and softcap are taken and
                                 ignored */
  int32_t window_left;        /* FA_MASK_WINDOW: the query (position context_len - 1) sees the keys
                                 at positions context_len - 1 - window_left .. context_len - 1 */
  int32_t query_len;          /* query tokens per sequence; 0 or 1 = decode.  With n > 1 (speculative
                                 decoding, chunked prefill) query and out are
                                 [num_seqs, n, num_heads, head_size], the scratch arrays have
                                 num_seqs * n rows, the n tokens are the last n positions of the
                                 context (their K/V rows already in the caches, context_lens counting
                                 them) and token j sees the keys up to its own position -- upstream's
                                 causal rule, test_paged.py:79-80.  At most 64.  K and V are read
                                 once per group of 2 * (16 / (num_heads / num_kv_heads)) query
                                 tokens */
  int32_t kv_scale_mode;      /* FP8 entries and the KV-cache writer: fa_kv_scale.  0 = the scalar
                                 fp8_scale as upstream; otherwise fp8_scale is ignored and the two
                                 arrays below are read */
  const float *k_scales;      /* device, fp32, shaped as kv_scale_mode says; NULL with mode 0 */
  const float *v_scales;
  int32_t schedule;           /* fa_schedule; 0 = the library chooses */
  int32_t spin_limit;         /* persistent kernels: polls a wavefront spends on one wait for the other
                                 wavefronts of its work-group before it gives up (and the call's result is
                                 void, see fa_paged_attention_kernel_status).  0 = the library's bound,
                                 which no correct run reaches; negative = do not wait at all, which makes
                                 the give-up path run for a test while every kernel still ends normally */
  int32_t segment_partitions; /* reduce entries, FA_SCHEDULE_AUTO: how rows are cut into partials where the
                                 library would choose that itself (see fa_paged_attention_reduce): 0 = the
                                 library chooses; n >= 1 = every n partitions (at most 64); -1 = even shares,
                                 one contiguous run of partitions per work-group; -2 = segments of the length
                                 the library's rule gives, never even shares.  A tuning and test knob:
                                 `out` does not depend on it beyond the order of fp32 sums */
} fa_paged_attention_options;
#define FA_PAGED_ATTENTION_OPTIONS_INIT {(uint32_t)sizeof(fa_paged_attention_options)}

/* Single-pass kernel: no scratch.  One launch for a decode batch of up to 128 sequences; larger
 * batches and query blocks of more than 32 (token, head) columns per kv head take several. */
int32_t fa_paged_attention_loop(void *out, const void *query, const void *key_cache,
                                const void *value_cache, const int32_t *block_tables,
                                const int32_t *context_lens, float scale, int32_t max_context_len,
                                const fa_paged_attention_shape *shape,
                                const fa_paged_attention_options *options);

/* Split-context kernel followed by the reduce kernel.  exp_sums, max_logits and tmp_out are
 * scratch the two kernels hand partial softmax states through; every slot either holds what
 * upstream stores there for its partition -- or nothing: for batches with many
 * (sequence, kv head) pairs one partial covers several consecutive partitions and sits in
 * the slot of the first; the slots of max_logits in between hold a mark by which the reduce
 * kernel tells them from partials (a NaN no maximum can be), those of exp_sums and tmp_out stay
 * untouched; a row whose whole context lies in one partial gets that partial straight into `out`,
 * as its result -- its scalars are in exp_sums and max_logits, its tmp_out row stays untouched; and
 * where the rows are provably too short for splitting to pay the call runs the single-pass kernel
 * and leaves all three arrays alone (fa_paged_attention_reduce_plan).  Only `out` is a result;
 * FA_SCHEDULE_GRID is the schedule under which the arrays hold upstream's per-partition contents. */
int32_t fa_paged_attention_reduce(void *out, const void *query, const void *key_cache,
                                  const void *value_cache, const int32_t *block_tables,
                                  const int32_t *context_lens, float scale,
                                  int32_t max_context_len, float *exp_sums, float *max_logits,
                                  float *tmp_out, const fa_paged_attention_shape *shape,
                                  const fa_paged_attention_options *options);

/* fa_paged_attention_reduce for callers that cannot allocate: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart upstream (there
 * the caller allocates max_logits, exp_sums and tem_output, test_paged.py:449-457).  Same kernels,
 * same arguments and same `out` as fa_paged_attention_reduce, but exp_sums, max_logits and tmp_out
 * live in a fixed array of FA_STATIC_SCRATCH_BYTES that the library holds in device memory on
 * every GPU it runs on until the process ends.  The call allocates nothing, on the host or on the
 * device, and frees nothing.
 * The array is part of the library's code object: every process that loads the library holds
 * FA_STATIC_SCRATCH_BYTES of device memory on every GPU it touches, whether or not this entry point
 * is ever called.  Under HIP graph capture: fa_paged_attention_init() and one eager call of the same
 * shape first (see there).
 *   needs  2 * align256(4 * slots) + 4 * slots * head_size bytes,
 *          slots = num_seqs * max(query_len, 1) * num_heads * max_num_partitions;
 *          more than FA_STATIC_SCRATCH_BYTES -> FA_ERR_SCRATCH_TOO_SMALL, nothing is launched
 *   options->elapsed_us must be NULL (timing creates events): the call is always asynchronous
 * Every call a process makes on a GPU uses that GPU's one array and finds the last call's
 * contents in it: calls whose kernels may overlap on one GPU (two streams, two threads) race --
 * order them on one stream or with events.  Nothing in the array has to start at zero: every
 * slot the reduce kernel reads was written by the attention kernel of the same call. */
#define FA_STATIC_SCRATCH_BYTES (64u << 20)
int32_t fa_paged_attention_reduce_static_scratch(void *out, const void *query, const void *key_cache,
                                                 const void *value_cache, const int32_t *block_tables,
                                                 const int32_t *context_lens, float scale,
                                                 int32_t max_context_len,
                                                 const fa_paged_attention_shape *shape,
                                                 const fa_paged_attention_options *options);

/* FP8 KV-cache variants: caches are bytes (E5M2 as upstream, or E4M3), dequantised in registers. */
int32_t fa_paged_attention_fp8_loop(void *out, const void *query, const void *key_cache,
                                    const void *value_cache, const int32_t *block_tables,
                                    const int32_t *context_lens, float scale,
                                    int32_t max_context_len,
                                    const fa_paged_attention_shape *shape,
                                    const fa_paged_attention_options *options);

int32_t fa_paged_attention_fp8_reduce(void *out, const void *query, const void *key_cache,
                                      const void *value_cache, const int32_t *block_tables,
                                      const int32_t *context_lens, float scale,
                                      int32_t max_context_len, float *exp_sums,
                                      float *max_logits, float *tmp_out,
                                      const fa_paged_attention_shape *shape,
                                      const fa_paged_attention_options *options);

/* Everything the library sets up once per GPU, done now on the current device instead of inside the
 * first call there: the device addresses of its two static device arrays (the status word of
 * fa_paged_attention_kernel_status and the scratch of fa_paged_attention_reduce_static_scratch, both
 * through hipGetSymbolAddress, which may load the code object) and the device's compute-unit count.
 * A caller that records calls into a HIP graph calls this first, outside the capture, and makes one
 * eager call of each shape it will record (the first launch of a kernel instance asks the occupancy
 * calculator how many of its work-groups stay resident).  No counterpart upstream. */
int32_t fa_paged_attention_init(void);

/* Text of the last failure on the calling thread ("" if none). */
const char *fa_last_error(void);

/* Which kernels fa_paged_attention_reduce / fa_paged_attention_fp8_reduce (kv_fp8 non-zero) run for a
 * call of this shape, options and max_context_len -- decided on the host, from these arguments alone:
 *   FA_SPLIT_FORM_GRID     upstream's decomposition: one work-group and one partial per (sequence, kv
 *                          head, partition), then the reduce kernel (launch_kernels_reduce.h:18-78)
 *   FA_SPLIT_FORM_SEGMENT  resident work-groups, one partial per segment of several partitions, then
 *                          the reduce kernel
 *   FA_SPLIT_FORM_LOOP     the rows are too short for splitting to pay -- at most 1024 keys, or at most
 *                          2048 with a (sequence, kv head) row for every compute unit, by what
 *                          max_context_len (0 = unknown), the block table's width and the scratch
 *                          arrays' capacity say: the call is the single-pass kernel, one launch; the
 *                          scratch arrays stay untouched and the second kernel time is 0
 * compute_units > 0: of the GPU in question; the plan is then made without a device and work_groups
 * stays 0.  compute_units = 0: the current device's, and work_groups is filled in.  Launches nothing.
 * No counterpart upstream, whose launcher has one form. */
typedef enum fa_split_form { FA_SPLIT_FORM_GRID = 0, FA_SPLIT_FORM_SEGMENT = 1, FA_SPLIT_FORM_LOOP = 2 } fa_split_form;
typedef struct fa_split_plan {
  uint32_t struct_size;      /* sizeof(fa_split_plan) in the caller's header */
  int32_t form;              /* fa_split_form */
  int32_t compute_units;     /* as given, or of the current device */
  int32_t work_groups;       /* FA_SPLIT_FORM_SEGMENT, made with a device: work-groups of the attention
                                launch (the first, if the batch takes several); else 0 */
  int32_t kv_heads_per_item; /* FA_SPLIT_FORM_SEGMENT, made with a device: kv heads that one work item of the
                                attention kernel covers -- 2 where adjacent heads are taken as pairs or by
                                teams of wavefronts, else 1; 0 when not filled in */
} fa_split_plan;
#define FA_SPLIT_PLAN_INIT {(uint32_t)sizeof(fa_split_plan)}
int32_t fa_paged_attention_reduce_plan(const fa_paged_attention_shape *shape,
                                       const fa_paged_attention_options *options, int32_t max_context_len,
                                       int32_t kv_fp8, int32_t compute_units, fa_split_plan *plan);

/* Did a persistent kernel of the current GPU give up a wait for the wavefronts of its work-group
 * (options->spin_limit) since the word was last cleared?  Then the output of that call is not
 * valid.  Timed calls (elapsed_us) look by themselves and return FA_ERR_RUNTIME; asynchronous
 * calls cannot, so their caller asks here at a synchronisation point of its own: the function
 * waits for `stream` (a hipStream_t; NULL = the null stream), reads the word and, with `clear`
 * non-zero, resets it.  Returns FA_OK (nothing happened) or FA_ERR_RUNTIME with the reason in
 * fa_last_error().  One word per GPU: it does not say which call it was.  No counterpart upstream
 * (whose work-groups meet at barriers, paged_attention_kernel_loop.hpp:345-347). */
int32_t fa_paged_attention_kernel_status(void *stream, int32_t clear);

/* ABI revision of this header: 8 (structs begin with struct_size). */
int32_t fa_paged_attention_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* FA_PAGED_ATTENTION_H_ */
