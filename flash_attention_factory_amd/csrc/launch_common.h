// Host-side pieces shared by the four launchers: error text, argument checks,
// kernel-parameter assembly and event timing.
//
// Upstream has no counterpart for the checks (paged_attention_loop.cpp:44-65 reads
// pointers and sizes without looking at them) and reports errors by throwing
// std::runtime_error from the dispatchers (launch_kernels_loop.h:114-115,170-172);
// here the same conditions become status codes because nothing may throw across a C ABI.
#pragma once

#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <mutex>

#include "../../include/fa_paged_attention.h"
#include "paged_attention_kernel.h"
#include "paged_attention_lds_kernel.h"
#include "paged_attention_loop_persistent_kernel.h"
#include "paged_attention_loop_two_tile_kernel.h"
#include "paged_attention_policy.h"
#include "paged_attention_reduce_kernel.h"
#include "paged_attention_segment_kernel.h"
#include "paged_attention_valu_kernel.h"

namespace fa {

constexpr int kAbiRevision = 8;  // fa_paged_attention_abi_version()

inline char *error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

inline fa_status fail(fa_status code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

#define FA_HIP_CHECK(expr)                                                                  \
  do {                                                                                      \
    hipError_t e_ = (expr);                                                                 \
    if (e_ != hipSuccess)                                                                   \
      return ::fa::fail(FA_ERR_RUNTIME, "%s failed: %s", #expr, hipGetErrorString(e_));     \
  } while (0)

// The status word of the persistent kernels: a wavefront that exhausts its spin limit while it
// waits for the other wavefronts of its work-group stores kStatusSpinLimit here and goes on (so
// the grid drains) with a result that is wrong.  One word per GPU, in device memory; as with any
// __device__ variable the name is only a handle on the host, the address on the current device
// comes from hipGetSymbolAddress, once per device.
static __device__ int32_t kernel_status_word;

inline fa_status kernel_status_of_current_device(int32_t **word) {
  constexpr int kMaxDevices = 64;
  static std::mutex mutex;
  static int32_t *address[kMaxDevices];  // nullptr until the device's first launch
  int dev = 0;
  FA_HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices)
    return fail(FA_ERR_RUNTIME, "device %d is beyond the %d devices this library serves", dev, kMaxDevices);
  std::lock_guard<std::mutex> guard(mutex);
  if (address[dev] == nullptr) {
    void *a = nullptr;
    FA_HIP_CHECK(hipGetSymbolAddress(&a, HIP_SYMBOL(kernel_status_word)));
    address[dev] = static_cast<int32_t *>(a);
  }
  *word = address[dev];
  return FA_OK;
}

// The spin limit of a call's persistent kernels (fa_paged_attention_options::spin_limit): 0 = the
// library's bound, negative = no polls at all, so that every wait gives up at once -- the way to see
// the give-up path run while every kernel still ends normally.
inline int32_t spin_limit_of(const fa_paged_attention_options *o) {
  if (!o || o->spin_limit == 0) return kLoopPersistentSpinLimit;
  return o->spin_limit < 0 ? 0 : o->spin_limit;
}

// A versioned struct as the library works with it: the `struct_size` bytes the caller's header
// knows, every later field zero.  `least`: bytes of the fields the struct cannot do without.
template <typename T>
inline fa_status read_versioned(const T *in, T *out, size_t least, const char *name) {
  const size_t size = in->struct_size;
  if (size < least || size > sizeof(T) || size % 4)
    return fail(FA_ERR_BAD_SHAPE, "%s.struct_size is %zu: it must be sizeof of the struct in the caller's header, "
                                  "%zu to %zu bytes for this library (ABI revision %d)",
                name, size, least, sizeof(T), kAbiRevision);
  memset(reinterpret_cast<char *>(out), 0, sizeof(T));
  memcpy(reinterpret_cast<char *>(out), reinterpret_cast<const char *>(in), size);
  out->struct_size = (uint32_t)sizeof(T);
  return FA_OK;
}

// Shape and options of a decode entry point, copied out of the caller's structs.  options() is
// NULL when the caller passed none.
struct CallStructs {
  fa_paged_attention_shape shape;
  fa_paged_attention_options options_storage;
  bool has_options = false;
  const fa_paged_attention_options *options() const { return has_options ? &options_storage : nullptr; }
};

inline fa_status read_options(const fa_paged_attention_options *options, CallStructs *c) {
  c->has_options = options != nullptr;
  if (!options) return FA_OK;
  return read_versioned(options, &c->options_storage, sizeof(uint32_t), "options");
}

inline fa_status read_call_structs(const fa_paged_attention_shape *shape, const fa_paged_attention_options *options,
                                   CallStructs *c) {
  error_buffer()[0] = 0;
  if (!shape) return fail(FA_ERR_NULL_POINTER, "shape is NULL");
  // every field of revision 8 is needed: the struct ends with num_pool_blocks
  constexpr size_t kShapeLeast = offsetof(fa_paged_attention_shape, num_pool_blocks) + sizeof(int32_t);
  const fa_status st = read_versioned(shape, &c->shape, kShapeLeast, "shape");
  if (st != FA_OK) return st;
  return read_options(options, c);
}

inline bool is_pow2(int64_t v) { return v > 0 && (v & (v - 1)) == 0; }
inline int ilog2(int32_t v) {
  int s = 0;
  while ((1 << s) < v) ++s;
  return s;
}

// Query tokens per sequence an extended call may bring.  The 16 MFMA columns hold
// 16 / (heads per kv head) of them at a time; a call with more runs as several launches, each
// reading K and V once.
constexpr int kMaxQueryLen = 64;

struct Resolved {
  int32_t group;
  int32_t partition_size;
  int32_t kv_elem_bytes;
  float fp8_scale;
  bool e4m3;  // FP8 entries: the caches hold E4M3 bytes, not E5M2
  int32_t mask_flags;  // fa_mask bits to apply
  const float *alibi_slopes;
  float softcap;
  int32_t window_left;
  int32_t query_len;  // query tokens per sequence, >= 1
  int32_t kv_scale_mode;  // fa_kv_scale; with a mode other than 0 fp8_scale is 1
  const float *k_scales;
  const float *v_scales;
  int32_t schedule;  // fa_schedule (FA_SCHEDULE_SPLIT: FA_SCHEDULE_AUTO with keep_split)
  bool keep_split;   // a reduce entry runs its two kernels however short the rows
  int32_t segment_partitions;  // > 0: partitions per partial of the segment form, fixed by the caller; -1: even shares
  bool pair_heads;   // two adjacent kv heads with 64-byte token rows run as one (WaveAttn::kPairable)
  int32_t *status;   // status word of the current device (nullptr with validate_only)
  int32_t spin_limit;
  hipStream_t stream;
  float *elapsed_us;
  bool validate_only;
  const void *sinks;
  fa_split_plan *plan;  // non-NULL: the split launcher fills this in where it would launch, and launches nothing
};

// Checks every argument the kernels rely on.  `kv8` selects byte caches, `split`
// the presence of the scratch arrays.
inline fa_status validate_and_resolve(const void *out, const void *query, const void *key_cache,
                                      const void *value_cache, const int32_t *block_tables,
                                      const int32_t *context_lens, int32_t max_context_len,
                                      const float *exp_sums, const float *max_logits,
                                      const float *tmp_out, const fa_paged_attention_shape *s,
                                      const fa_paged_attention_options *o, bool kv8, bool split,
                                      Resolved *r) {
  error_buffer()[0] = 0;
  if (!s) return fail(FA_ERR_NULL_POINTER, "shape is NULL");
  if (!out || !query || !key_cache || !value_cache || !block_tables || !context_lens)
    return fail(FA_ERR_NULL_POINTER, "out, query, key_cache, value_cache, block_tables and "
                                     "context_lens must all be non-NULL");
  if (split && (!exp_sums || !max_logits || !tmp_out))
    return fail(FA_ERR_NULL_POINTER, "exp_sums, max_logits and tmp_out must be non-NULL");
  if (s->q_dtype != FA_DTYPE_F16 && s->q_dtype != FA_DTYPE_BF16)
    return fail(FA_ERR_UNSUPPORTED_DTYPE, "q_dtype %d is neither fp16 (0) nor bf16 (1)", s->q_dtype);
  if ((s->head_size != 64 && s->head_size != 128) || s->block_size < 16 || !is_pow2(s->block_size))
    return fail(FA_ERR_UNSUPPORTED_HEAD_OR_BLOCK_SIZE,
                "Unsupported head size or block size (head_size %d must be 64 or 128, block_size "
                "%d a power of two >= 16)", s->head_size, s->block_size);
  if (s->num_seqs <= 0 || s->num_heads <= 0 || s->num_kv_heads <= 0 || s->max_blocks_per_seq <= 0)
    return fail(FA_ERR_BAD_SHAPE, "num_seqs, num_heads, num_kv_heads and max_blocks_per_seq must be positive");
  if (s->num_pool_blocks < 0) return fail(FA_ERR_BAD_SHAPE, "num_pool_blocks must be >= 0");
  if (s->num_heads % s->num_kv_heads != 0)
    return fail(FA_ERR_UNSUPPORTED_GROUP, "Unsupported number of queries per token: num_heads %d is "
                                          "not a multiple of num_kv_heads %d", s->num_heads, s->num_kv_heads);
  r->group = s->num_heads / s->num_kv_heads;
  if (r->group > kMaxGroup)
    return fail(FA_ERR_UNSUPPORTED_GROUP, "Unsupported number of queries per token: %d (at most %d)",
                r->group, kMaxGroup);
  r->kv_elem_bytes = kv8 ? 1 : 2;
  const int64_t eb = r->kv_elem_bytes;
  if (s->kv_block_stride <= 0 || s->kv_token_stride <= 0 || s->kv_head_stride <= 0)
    return fail(FA_ERR_BAD_SHAPE, "kv strides must be positive");
  if ((s->kv_block_stride * eb) % 16 || (s->kv_token_stride * eb) % 16 || (s->kv_head_stride * eb) % 16)
    return fail(FA_ERR_BAD_SHAPE, "kv strides must be multiples of 16 bytes");
  if (s->kv_token_stride < s->head_size || s->kv_head_stride < s->head_size)
    return fail(FA_ERR_BAD_SHAPE, "kv_token_stride and kv_head_stride must each cover one head_size row");
  if (((uintptr_t)key_cache | (uintptr_t)value_cache | (uintptr_t)query | (uintptr_t)out) % 16)
    return fail(FA_ERR_BAD_SHAPE, "out, query, key_cache and value_cache must be 16-byte aligned");
  r->partition_size = s->partition_size > 0 ? s->partition_size : default_partition_size(s->head_size);
  if (split) {
    if (r->partition_size % kMaxChunkTokens)
      return fail(FA_ERR_BAD_SHAPE, "partition_size %d must be a multiple of %d", r->partition_size, kMaxChunkTokens);
    if (s->max_num_partitions <= 0 || s->max_num_partitions > 65535)
      return fail(FA_ERR_BAD_SHAPE, "max_num_partitions %d must be in [1, 65535]", s->max_num_partitions);
    if (max_context_len > 0 &&
        (int64_t)s->max_num_partitions * r->partition_size < (int64_t)max_context_len)
      return fail(FA_ERR_PARTITION_OVERFLOW, "max_context_len %d needs %d partitions of %d tokens, scratch has %d",
                  max_context_len, (max_context_len + r->partition_size - 1) / r->partition_size,
                  r->partition_size, s->max_num_partitions);
    if ((uintptr_t)tmp_out % 16) return fail(FA_ERR_BAD_SHAPE, "tmp_out must be 16-byte aligned");
  }
  if (max_context_len > 0 &&
      (int64_t)s->max_blocks_per_seq * s->block_size < (int64_t)max_context_len)
    return fail(FA_ERR_BAD_SHAPE, "max_context_len %d does not fit %d blocks of %d tokens", max_context_len,
                s->max_blocks_per_seq, s->block_size);
  if (kv8 && o && o->kv_fp8_format != FA_FP8_E5M2 && o->kv_fp8_format != FA_FP8_E4M3)
    return fail(FA_ERR_UNSUPPORTED_DTYPE, "kv_fp8_format %d is neither E5M2 (0) nor E4M3 (1)", o->kv_fp8_format);
  r->e4m3 = kv8 && o && o->kv_fp8_format == FA_FP8_E4M3;
  r->mask_flags = o ? o->mask_flags : 0;
  if (r->mask_flags & ~(FA_MASK_ALIBI | FA_MASK_SOFTCAP | FA_MASK_WINDOW))
    return fail(FA_ERR_BAD_SHAPE, "mask_flags 0x%x has bits that mean nothing", r->mask_flags);
  if ((r->mask_flags & FA_MASK_ALIBI) && !o->alibi_slopes)
    return fail(FA_ERR_NULL_POINTER, "FA_MASK_ALIBI needs alibi_slopes");
  if ((r->mask_flags & FA_MASK_SOFTCAP) && !(o->softcap > 0.f))
    return fail(FA_ERR_BAD_SHAPE, "FA_MASK_SOFTCAP needs softcap > 0");
  if ((r->mask_flags & FA_MASK_WINDOW) && o->window_left < 0)
    return fail(FA_ERR_BAD_SHAPE, "FA_MASK_WINDOW needs window_left >= 0");
  r->query_len = (o && o->query_len > 1) ? o->query_len : 1;
  if (o && o->query_len < 0) return fail(FA_ERR_BAD_SHAPE, "query_len must be >= 0");
  if (r->query_len > kMaxQueryLen)
    return fail(FA_ERR_BAD_SHAPE, "query_len %d exceeds %d", r->query_len, kMaxQueryLen);
  if ((int64_t)s->num_seqs * r->query_len * s->num_heads > 0x7fffffffLL)
    return fail(FA_ERR_BAD_SHAPE, "num_seqs x query_len x num_heads %lld exceeds the grid limit 2^31 - 1",
                (long long)s->num_seqs * r->query_len * s->num_heads);
  r->alibi_slopes = o ? o->alibi_slopes : nullptr;
  r->softcap = o ? o->softcap : 0.f;
  r->window_left = o ? o->window_left : 0;
  r->fp8_scale = (kv8 && o && o->fp8_scale != 0.f) ? o->fp8_scale : 1.0f;
  r->kv_scale_mode = (kv8 && o) ? o->kv_scale_mode : FA_KV_SCALE_TENSOR;
  r->k_scales = r->v_scales = nullptr;
  if (r->kv_scale_mode != FA_KV_SCALE_TENSOR) {
    if (r->kv_scale_mode != FA_KV_SCALE_HEAD && r->kv_scale_mode != FA_KV_SCALE_BLOCK)
      return fail(FA_ERR_BAD_SHAPE, "kv_scale_mode %d is none of tensor (0), head (1), block (2)", r->kv_scale_mode);
    if (!o->k_scales || !o->v_scales)
      return fail(FA_ERR_NULL_POINTER, "kv_scale_mode %d needs k_scales and v_scales", r->kv_scale_mode);
    if (((uintptr_t)o->k_scales | (uintptr_t)o->v_scales) % 4)
      return fail(FA_ERR_BAD_SHAPE, "k_scales and v_scales must be 4-byte aligned");
    if (r->kv_scale_mode == FA_KV_SCALE_BLOCK && s->num_pool_blocks <= 0)
      return fail(FA_ERR_BAD_SHAPE, "per-block scales need num_pool_blocks");
    r->k_scales = o->k_scales;
    r->v_scales = o->v_scales;
    r->fp8_scale = 1.0f;
  }
  r->schedule = o ? o->schedule : FA_SCHEDULE_AUTO;
  if (r->schedule != FA_SCHEDULE_AUTO && r->schedule != FA_SCHEDULE_GRID && r->schedule != FA_SCHEDULE_GRID_LDS &&
      r->schedule != FA_SCHEDULE_SPLIT && r->schedule != FA_SCHEDULE_GRID_VALU && r->schedule != FA_SCHEDULE_VALU)
    return fail(FA_ERR_BAD_SHAPE,
                "schedule %d is none of auto (0), grid (1), grid with LDS staging (2), split (3), without matrix cores: grid (4), persistent (5)",
                r->schedule);
  r->keep_split = r->schedule == FA_SCHEDULE_SPLIT;  // otherwise the library's own choice
  if (r->keep_split) r->schedule = FA_SCHEDULE_AUTO;
  r->segment_partitions = o ? o->segment_partitions : 0;
  if (r->segment_partitions < -2)
    return fail(FA_ERR_BAD_SHAPE, "segment_partitions must be -2 (segments of the library's length), -1 (even shares), "
                                  "0 (the library chooses) or a count");
  r->pair_heads = kPairHeads && kv8 && s->head_size == 64 && s->kv_head_stride == s->head_size &&
                  s->num_kv_heads % 2 == 0 && 2 * r->group <= kMaxGroup && r->mask_flags == 0 &&
                  r->query_len == 1 && r->kv_scale_mode == FA_KV_SCALE_TENSOR;
  r->stream = o ? reinterpret_cast<hipStream_t>(o->stream) : nullptr;
  r->elapsed_us = o ? o->elapsed_us : nullptr;
  r->validate_only = o && o->validate_only != 0;
  r->sinks = o ? o->sinks : nullptr;
  r->plan = nullptr;
  r->status = nullptr;
  r->spin_limit = spin_limit_of(o);
  if (!r->validate_only) return kernel_status_of_current_device(&r->status);
  return FA_OK;
}

// Did a kernel of the current GPU give up a wait since the status word was last cleared?  Waits for
// `stream`, reads the word, clears it on request, and turns a set word into FA_ERR_RUNTIME.
inline fa_status read_kernel_status(hipStream_t stream, bool clear, int32_t spin_limit) {
  int32_t *word = nullptr;
  const fa_status st = kernel_status_of_current_device(&word);
  if (st != FA_OK) return st;
  // read through one pinned word per thread (a copy into pageable memory costs ten times as much);
  // allocated on the first look, like the timing events
  static thread_local int32_t *pinned = nullptr;
  if (pinned == nullptr) FA_HIP_CHECK(hipHostMalloc(reinterpret_cast<void **>(&pinned), sizeof(int32_t), hipHostMallocDefault));
  FA_HIP_CHECK(hipMemcpyAsync(pinned, word, sizeof(int32_t), hipMemcpyDeviceToHost, stream));
  FA_HIP_CHECK(hipStreamSynchronize(stream));
  const int32_t seen = *pinned;
  if (seen == 0) return FA_OK;
  if (clear) {
    const int32_t zero = 0;
    FA_HIP_CHECK(hipMemcpyAsync(word, &zero, sizeof(zero), hipMemcpyHostToDevice, stream));
    FA_HIP_CHECK(hipStreamSynchronize(stream));
  }
  if (spin_limit > 0)
    return fail(FA_ERR_RUNTIME, "a wavefront gave up waiting for the other wavefronts of its work-group (spin limit %d, "
                                "status %d): the output of this or an earlier call on this GPU is not valid",
                spin_limit, seen);
  return fail(FA_ERR_RUNTIME, "a wavefront gave up waiting for the other wavefronts of its work-group (status %d): the "
                              "output of this or an earlier call on this GPU is not valid", seen);
}

// After a timed call (which has synchronised anyway): report and clear the status word.
// Asynchronous calls do not look: the word stays set until the next timed call on the device, or
// fa_paged_attention_kernel_status, reports it.
inline fa_status report_kernel_status(const Resolved &r) {
  if (!r.elapsed_us || !r.status) return FA_OK;
  return read_kernel_status(r.stream, true, r.spin_limit);
}

inline PagedAttnParams make_params(void *out, float *exp_sums, float *max_logits, const void *query,
                                   const void *key_cache, const void *value_cache,
                                   const int32_t *block_tables, const int32_t *context_lens,
                                   float scale, const fa_paged_attention_shape &s, const Resolved &r) {
  PagedAttnParams p;
  p.out = out;
  p.exp_sums = exp_sums;
  p.max_logits = max_logits;
  p.query = query;
  p.key_cache = reinterpret_cast<const char *>(key_cache);
  p.value_cache = reinterpret_cast<const char *>(value_cache);
  p.block_tables = block_tables;
  p.context_lens = context_lens;
  p.sinks = r.sinks;
  p.score_scale_log2 = scale * r.fp8_scale * kLog2e;
  p.score_scale = scale * r.fp8_scale;
  p.mask_flags = r.mask_flags;
  p.alibi_slopes = r.alibi_slopes;
  p.softcap = r.softcap;
  p.window_left = r.window_left;
  p.query_len = r.query_len;
  p.query_first = 0;
  p.query_count = std::min(r.query_len, kMaxGroup / r.group);
  p.out_scale = r.fp8_scale;
  p.kv_scale_mode = r.kv_scale_mode;
  p.k_scales = r.k_scales;
  p.v_scales = r.v_scales;
  p.num_seqs = s.num_seqs;
  p.num_heads = s.num_heads;
  p.num_kv_heads = s.num_kv_heads;
  p.group = r.group;
  p.max_blocks_per_seq = s.max_blocks_per_seq;
  p.max_num_partitions = s.max_num_partitions;
  p.partition_size = r.partition_size;
  p.block_shift = ilog2(s.block_size);
  p.max_block_id = s.num_pool_blocks > 0 ? s.num_pool_blocks - 1 : INT32_MAX;
  p.spin_limit = r.spin_limit;
  p.status = r.status;
  p.kv_block_bytes = s.kv_block_stride * r.kv_elem_bytes;
  p.kv_token_bytes = s.kv_token_stride * r.kv_elem_bytes;
  p.kv_head_bytes = s.kv_head_stride * r.kv_elem_bytes;
  p.compute_units = 0;  // the split path's launcher fills it in
  p.final_out = nullptr;  // (and this, in the segment form)
  p.kv_rows_apart = s.kv_token_stride != s.head_size;
  p.segment_force = r.segment_partitions;
  p.pair_heads = 0;
  if (r.pair_heads) {  // the kernel sees pairs of kv heads: half as many, twice the group, rows of two heads
    p.pair_heads = 1;
    p.num_kv_heads /= 2;
    p.group *= 2;
    p.kv_head_bytes *= 2;
  }
  return p;
}

// Compute units of the current device (asked once per thread and device).
inline hipError_t compute_units_of_current_device(int *cus_out) {
  static thread_local int cached_dev = -1, cached_cus = 0;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev != cached_dev) {
    int cus = 0;
    e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return e;
    cached_dev = dev;
    cached_cus = cus;
  }
  *cus_out = cached_cus;
  return hipSuccess;
}

// How many work-groups of `threads` threads of a kernel the current device keeps resident
// (compute units x work-groups per compute unit).  Asked once per (kernel, device); all
// kernels here share one function-pointer type, so the cache is keyed by the pointer value.
// cus_out, if given: the compute units of the device.
inline hipError_t resident_groups(void (*kernel)(PagedAttnParams), int threads, int *out, int *cus_out = nullptr) {
  struct Entry { const void *fn; int dev; int groups; int cus; };
  constexpr int kSlots = 64;
  static thread_local Entry cache[kSlots];
  static thread_local int used = 0;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const void *fn = reinterpret_cast<const void *>(kernel);
  for (int k = 0; k < used; ++k)
    if (cache[k].fn == fn && cache[k].dev == dev) {
      *out = cache[k].groups;
      if (cus_out) *cus_out = cache[k].cus;
      return hipSuccess;
    }
  int cus = 0, per_cu = 0;
  e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e != hipSuccess) return e;
  e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, 0);
  if (e != hipSuccess) return e;
  const int groups = cus * (per_cu > 0 ? per_cu : 1);
  if (used < kSlots) cache[used++] = Entry{fn, dev, groups, cus};
  *out = groups;
  if (cus_out) *cus_out = cus;
  return hipSuccess;
}

// Kernel-only time -- the counterpart of upstream's get_exe_time
// (launch_kernels_loop.h:6-12), which reads the start/end stamps of the kernel's own
// SYCL event.  hipExtLaunchKernelGGL attaches a start and a stop event to the dispatch
// itself, so the pair brackets the kernel and nothing else (events recorded with
// separate hipEventRecord calls also count the gap between the record and the
// dispatch).  Events are created once per thread and device and reused.
class KernelTimer {
 public:
  KernelTimer(bool enabled, hipStream_t stream) : enabled_(enabled), stream_(stream) {}

  // Launch `kernel` on the stream; with timing on, events 2*slot / 2*slot+1 bracket it.
  template <typename Params>
  hipError_t launch(void (*kernel)(Params), dim3 grid, dim3 block, int slot, const Params &prm) {
    if (!enabled_) {  // plain launch: nothing but the kernel goes on the stream, so a
                      // caller may record it into a HIP graph
      hipLaunchKernelGGL(kernel, grid, block, 0, stream_, prm);
      return hipGetLastError();
    }
    hipError_t e = ensure();
    if (e != hipSuccess) return e;
    hipExtLaunchKernelGGL(kernel, grid, block, 0, stream_, events()[2 * slot], events()[2 * slot + 1], 0, prm);
    return hipGetLastError();
  }

  // Time of the launch last made in `slot`, ADDED to *us: a call that makes several launches
  // in a slot reads after each of them.
  hipError_t accumulate(int slot, float *us) {
    float one = 0.f;
    const hipError_t e = read(slot, &one);
    *us += one;
    return e;
  }

  hipError_t read(int slot, float *us) {
    if (!enabled_) return hipSuccess;
    hipError_t e = hipEventSynchronize(events()[2 * slot + 1]);
    if (e != hipSuccess) return e;
    float ms = 0.f;
    e = hipEventElapsedTime(&ms, events()[2 * slot], events()[2 * slot + 1]);
    *us = ms * 1000.f;
    return e;
  }

 private:
  static hipEvent_t *events() {
    static thread_local hipEvent_t ev[4] = {nullptr, nullptr, nullptr, nullptr};
    return ev;
  }
  static hipError_t ensure() {
    static thread_local int device_of_events = -1;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (device_of_events == dev) return hipSuccess;
    for (int k = 0; k < 4; ++k) {
      if (events()[k]) (void)hipEventDestroy(events()[k]);
      e = hipEventCreate(&events()[k]);
      if (e != hipSuccess) return e;
    }
    device_of_events = dev;
    return hipSuccess;
  }
  bool enabled_;
  hipStream_t stream_;
};

}  // namespace fa
