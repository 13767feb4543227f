"""``paged_attention_fp8_reduce.run``: the split-context + reduce kernels over an FP8-E5M2 KV cache.

Drop-in for the upstream extension module of the same name
(paged_attention_fp8_reduce/paged_attention_fp8_reduce.cpp:21-39,84-86): same positional arguments, same return value
(a list of kernel times in microseconds).  ``timed=False`` (keyword only, not in
upstream) launches asynchronously on the current stream and returns ``[]``;
``partition_size`` (keyword only) overrides the upstream policy value (512 tokens for
head size 128, 256 for head size 64); ``segment_partitions`` (keyword only) fixes how many partitions one
partial covers where the library would choose that number itself (0: it chooses).  ``apply_alibi``, ``apply_softcap`` and
``window_left`` (keyword only) switch on the score modifiers upstream's kernels take and
ignore (paged_attention_kernel_loop.hpp:329-342); ``k_scales`` / ``v_scales`` (keyword only;
fp32 device tensors ``[kv_heads]`` or ``[blocks, kv_heads]``) replace the scalar
``fp8_scale`` by per-head or per-block scales.
"""
from ._run import run_impl


def run(max_logits, exp_sums, tem_output, output, debug_output, query, key_cache, value_cache,
        block_tables, context_lens, num_queries_per_tokens, sm_scale, fp8_scale, block_size, max_context_len,
        alibi_slopes, sinks, softcap, *, timed=True, partition_size=0, apply_alibi=False, apply_softcap=False, window_left=None, schedule=0,
        k_scales=None, v_scales=None, spin_limit=0, segment_partitions=0):
    return run_impl("fa_paged_attention_fp8_reduce", True, True, max_logits, exp_sums, tem_output, output,
                    debug_output, query, key_cache, value_cache, block_tables, context_lens,
                    num_queries_per_tokens, sm_scale, fp8_scale, block_size, max_context_len,
                    alibi_slopes, sinks, softcap, timed=timed, partition_size=partition_size, apply_alibi=apply_alibi,
                    apply_softcap=apply_softcap, window_left=window_left, schedule=schedule, k_scales=k_scales, v_scales=v_scales, spin_limit=spin_limit, segment_partitions=segment_partitions)
