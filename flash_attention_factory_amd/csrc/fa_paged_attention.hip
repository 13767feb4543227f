// extern "C" surface of libfa_paged_attention.so: four decode entry points, one per host
// launcher, declared in include/fa_paged_attention.h, and the KV-cache writer declared in
// include/fa_kv_cache.h.
#include <mutex>

#include "../../include/fa_kv_cache.h"
#include "../../include/fa_paged_attention.h"

#include "launch_kernels_fp8_loop.h"
#include "launch_kernels_fp8_reduce.h"
#include "launch_kernels_loop.h"
#include "launch_kernels_reduce.h"
#include "launch_kv_cache_write.h"

#define FA_EXPORT extern "C" __attribute__((visibility("default")))

FA_EXPORT int32_t fa_paged_attention_loop(void *out, const void *query, const void *key_cache,
                                          const void *value_cache, const int32_t *block_tables,
                                          const int32_t *context_lens, float scale,
                                          int32_t max_context_len,
                                          const fa_paged_attention_shape *shape,
                                          const fa_paged_attention_options *options) {
  fa::CallStructs c;
  const fa_status st = fa::read_call_structs(shape, options, &c);
  if (st != FA_OK) return st;
  return fa::dispatch_paged_attention_loop(out, query, key_cache, value_cache, block_tables,
                                           context_lens, scale, max_context_len, &c.shape, c.options());
}

FA_EXPORT int32_t fa_paged_attention_reduce(void *out, const void *query, const void *key_cache,
                                            const void *value_cache, const int32_t *block_tables,
                                            const int32_t *context_lens, float scale,
                                            int32_t max_context_len, float *exp_sums,
                                            float *max_logits, float *tmp_out,
                                            const fa_paged_attention_shape *shape,
                                            const fa_paged_attention_options *options) {
  fa::CallStructs c;
  const fa_status st = fa::read_call_structs(shape, options, &c);
  if (st != FA_OK) return st;
  return fa::dispatch_paged_attention(out, query, key_cache, value_cache, block_tables,
                                      context_lens, scale, max_context_len, exp_sums, max_logits,
                                      tmp_out, &c.shape, c.options());
}

// ---- the entry point that allocates nothing ---------------------------------------------
// Scratch of the split path (exp_sums, max_logits, tmp_out) in a fixed device array.  In host
// code the name `scratch` is only a handle for hipGetSymbolAddress: each GPU holds its own copy
// of the array at its own address, asked for once per device and kept in scratch_address.
static __device__ __align__(256) unsigned char scratch[FA_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kScratchMaxDevices = 64;
std::mutex scratch_mutex;
void *scratch_address[kScratchMaxDevices];  // nullptr until the device's first call

// Device address of `scratch` on the current device.
fa_status static_scratch_of_current_device(unsigned char **base) {
  int dev = 0;
  FA_HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kScratchMaxDevices)
    return fa::fail(FA_ERR_RUNTIME, "device %d is beyond the %d devices the static scratch serves", dev,
                    kScratchMaxDevices);
  std::lock_guard<std::mutex> guard(scratch_mutex);
  if (scratch_address[dev] == nullptr) {
    void *address = nullptr;
    FA_HIP_CHECK(hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)));
    if (address == nullptr) return fa::fail(FA_ERR_RUNTIME, "hipGetSymbolAddress gave no address for the static scratch");
    scratch_address[dev] = address;
  }
  *base = static_cast<unsigned char *>(scratch_address[dev]);
  return FA_OK;
}

}  // namespace

FA_EXPORT int32_t fa_paged_attention_reduce_static_scratch(void *out, const void *query, const void *key_cache,
                                                           const void *value_cache, const int32_t *block_tables,
                                                           const int32_t *context_lens, float scale,
                                                           int32_t max_context_len,
                                                           const fa_paged_attention_shape *shape,
                                                           const fa_paged_attention_options *options) {
  fa::CallStructs c;
  const fa_status read = fa::read_call_structs(shape, options, &c);
  if (read != FA_OK) return read;
  shape = &c.shape;
  options = c.options();
  if (options && options->elapsed_us)
    return fa::fail(FA_ERR_BAD_SHAPE, "fa_paged_attention_reduce_static_scratch allocates nothing, events included: "
                                      "elapsed_us must be NULL (time the call with fa_paged_attention_reduce)");
  if (shape->num_seqs <= 0 || shape->num_heads <= 0 || shape->max_num_partitions <= 0 || shape->head_size <= 0)
    return fa::fail(FA_ERR_BAD_SHAPE, "num_seqs, num_heads, max_num_partitions and head_size must be positive");
  const int64_t query_len = (options && options->query_len > 1) ? options->query_len : 1;
  const int64_t slots = (int64_t)shape->num_seqs * query_len * shape->num_heads * shape->max_num_partitions;
  const int64_t scalars = (slots * 4 + 255) / 256 * 256;  // bytes of exp_sums, and of max_logits
  const int64_t need = 2 * scalars + slots * shape->head_size * 4;
  if (need > (int64_t)FA_STATIC_SCRATCH_BYTES)
    return fa::fail(FA_ERR_SCRATCH_TOO_SMALL,
                    "%lld scratch slots of head size %d need %lld bytes, the static scratch holds %lld: "
                    "lower max_num_partitions or use fa_paged_attention_reduce with scratch of your own",
                    (long long)slots, shape->head_size, (long long)need, (long long)FA_STATIC_SCRATCH_BYTES);
  // validate_only launches nothing and must work without a GPU: any non-NULL aligned address will do
  static float placeholder[4] __attribute__((aligned(16)));
  unsigned char *base = reinterpret_cast<unsigned char *>(placeholder);
  int64_t off_ml = 0, off_tmp = 0;
  if (!(options && options->validate_only)) {
    const fa_status st = static_scratch_of_current_device(&base);
    if (st != FA_OK) return st;
    off_ml = scalars;
    off_tmp = 2 * scalars;
  }
  return fa::dispatch_paged_attention(out, query, key_cache, value_cache, block_tables, context_lens, scale,
                                      max_context_len, reinterpret_cast<float *>(base),
                                      reinterpret_cast<float *>(base + off_ml),
                                      reinterpret_cast<float *>(base + off_tmp), shape, options);
}

FA_EXPORT int32_t fa_paged_attention_fp8_loop(void *out, const void *query, const void *key_cache,
                                              const void *value_cache,
                                              const int32_t *block_tables,
                                              const int32_t *context_lens, float scale,
                                              int32_t max_context_len,
                                              const fa_paged_attention_shape *shape,
                                              const fa_paged_attention_options *options) {
  fa::CallStructs c;
  const fa_status st = fa::read_call_structs(shape, options, &c);
  if (st != FA_OK) return st;
  return fa::dispatch_paged_attention_fp8_loop(out, query, key_cache, value_cache, block_tables,
                                               context_lens, scale, max_context_len, &c.shape,
                                               c.options());
}

FA_EXPORT int32_t fa_paged_attention_fp8_reduce(void *out, const void *query,
                                                const void *key_cache, const void *value_cache,
                                                const int32_t *block_tables,
                                                const int32_t *context_lens, float scale,
                                                int32_t max_context_len, float *exp_sums,
                                                float *max_logits, float *tmp_out,
                                                const fa_paged_attention_shape *shape,
                                                const fa_paged_attention_options *options) {
  fa::CallStructs c;
  const fa_status st = fa::read_call_structs(shape, options, &c);
  if (st != FA_OK) return st;
  return fa::dispatch_paged_attention_fp8(out, query, key_cache, value_cache, block_tables,
                                          context_lens, scale, max_context_len, exp_sums,
                                          max_logits, tmp_out, &c.shape, c.options());
}

FA_EXPORT int32_t fa_kv_cache_write(const void *key, const void *value, void *key_cache,
                                    void *value_cache, const int64_t *slot_mapping,
                                    const fa_kv_cache_write_shape *shape,
                                    const fa_paged_attention_options *options) {
  fa::error_buffer()[0] = 0;
  if (!shape) return fa::fail(FA_ERR_NULL_POINTER, "shape is NULL");
  fa_kv_cache_write_shape sh;
  fa::CallStructs c;
  constexpr size_t kLeast = offsetof(fa_kv_cache_write_shape, num_pool_blocks) + sizeof(int64_t);
  fa_status st = fa::read_versioned(shape, &sh, kLeast, "shape");
  if (st == FA_OK) st = fa::read_options(options, &c);
  if (st != FA_OK) return st;
  return fa::launch_kv_cache_write(key, value, key_cache, value_cache, slot_mapping, &sh, c.options());
}

FA_EXPORT int32_t fa_paged_attention_init(void) {
  fa::error_buffer()[0] = 0;
  int32_t *word = nullptr;
  fa_status st = fa::kernel_status_of_current_device(&word);
  if (st != FA_OK) return st;
  unsigned char *base = nullptr;
  st = static_scratch_of_current_device(&base);
  if (st != FA_OK) return st;
  int cus = 0;
  FA_HIP_CHECK(fa::compute_units_of_current_device(&cus));
  return FA_OK;
}

FA_EXPORT int32_t fa_paged_attention_reduce_plan(const fa_paged_attention_shape *shape,
                                                 const fa_paged_attention_options *options, int32_t max_context_len,
                                                 int32_t kv_fp8, int32_t compute_units, fa_split_plan *plan) {
  fa::CallStructs c;
  fa_status st = fa::read_call_structs(shape, options, &c);
  if (st != FA_OK) return st;
  if (!plan) return fa::fail(FA_ERR_NULL_POINTER, "plan is NULL");
  if (plan->struct_size != sizeof(fa_split_plan))
    return fa::fail(FA_ERR_BAD_SHAPE, "plan.struct_size is %u, this library's fa_split_plan has %zu bytes",
                    plan->struct_size, sizeof(fa_split_plan));
  // the checks of a call, made on placeholders: nothing is launched and no pointer is followed
  static float placeholder[4] __attribute__((aligned(16)));
  fa_paged_attention_options op = c.has_options ? c.options_storage : fa_paged_attention_options{};
  op.struct_size = sizeof(op);
  op.elapsed_us = nullptr;
  void *any = placeholder;
  const int32_t *ints = reinterpret_cast<const int32_t *>(placeholder);
  plan->form = plan->work_groups = plan->kv_heads_per_item = 0;
  plan->compute_units = compute_units;
  if (compute_units > 0) {  // without a device: the form alone
    op.validate_only = 1;
    fa::Resolved r;
    st = fa::validate_and_resolve(any, any, any, any, ints, ints, max_context_len, placeholder, placeholder, placeholder,
                                  &c.shape, &op, kv_fp8 != 0, /*split=*/true, &r);
    if (st != FA_OK) return st;
    plan->form = fa::split_form_of(c.shape, r, kv_fp8 != 0, max_context_len, compute_units);
    return FA_OK;
  }
  // with the current device: the launchers themselves, told to fill in the plan where they would launch
  op.validate_only = 0;
  if (kv_fp8)
    return fa::dispatch_paged_attention_fp8(any, any, any, any, ints, ints, 1.f, max_context_len, placeholder, placeholder,
                                            placeholder, &c.shape, &op, plan);
  return fa::dispatch_paged_attention(any, any, any, any, ints, ints, 1.f, max_context_len, placeholder, placeholder,
                                      placeholder, &c.shape, &op, plan);
}

FA_EXPORT int32_t fa_paged_attention_kernel_status(void *stream, int32_t clear) {
  fa::error_buffer()[0] = 0;
  return fa::read_kernel_status(reinterpret_cast<hipStream_t>(stream), clear != 0, 0);
}

#ifdef FA_TIMELINE
// Debug builds only (-DFA_TIMELINE): the in-kernel timeline of the current device, copied to the host
// (kTimelineWaves x kTimelineSlots 64-bit words), and cleared on request.
FA_EXPORT int32_t fa_debug_timeline(void *dst, size_t bytes, int32_t clear) {
  const size_t all = sizeof(unsigned long long) * fa::kTimelineWaves * fa::kTimelineSlots;
  FA_HIP_CHECK(hipDeviceSynchronize());
  FA_HIP_CHECK(hipMemcpyFromSymbol(dst, HIP_SYMBOL(fa::timeline_words), bytes < all ? bytes : all));
  if (clear) {
    void *address = nullptr;
    FA_HIP_CHECK(hipGetSymbolAddress(&address, HIP_SYMBOL(fa::timeline_words)));
    FA_HIP_CHECK(hipMemset(address, 0, all));
  }
  return FA_OK;
}
#endif

FA_EXPORT const char *fa_last_error(void) { return fa::error_buffer(); }

FA_EXPORT int32_t fa_paged_attention_abi_version(void) { return fa::kAbiRevision; }
