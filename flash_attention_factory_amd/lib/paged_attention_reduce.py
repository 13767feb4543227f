"""``paged_attention_reduce.run``: the split-context kernel followed by the reduce kernel.

Drop-in for the upstream extension module of the same name
(paged_attention_reduce/paged_attention_reduce.cpp:21-38,82-84): same positional arguments, same return value
(a list of kernel times in microseconds).  ``timed=False`` (keyword only, not in
upstream) launches asynchronously on the current stream and returns ``[]``;
``partition_size`` (keyword only) overrides the upstream policy value (512 tokens for
head size 128, 256 for head size 64); ``segment_partitions`` (keyword only) fixes how many partitions one
partial covers where the library would choose that number itself (0: it chooses).
"""
from ._run import run_impl


def run(max_logits, exp_sums, tem_output, output, debug_output, query, key_cache, value_cache,
        block_tables, context_lens, num_queries_per_tokens, sm_scale, block_size, max_context_len,
        alibi_slopes, sinks, softcap, *, timed=True, partition_size=0, apply_alibi=False, apply_softcap=False, window_left=None, schedule=0, spin_limit=0, segment_partitions=0):
    return run_impl("fa_paged_attention_reduce", True, False, max_logits, exp_sums, tem_output, output,
                    debug_output, query, key_cache, value_cache, block_tables, context_lens,
                    num_queries_per_tokens, sm_scale, 1.0, block_size, max_context_len,
                    alibi_slopes, sinks, softcap, timed=timed, partition_size=partition_size, apply_alibi=apply_alibi,
                    apply_softcap=apply_softcap, window_left=window_left, schedule=schedule, spin_limit=spin_limit, segment_partitions=segment_partitions)


def run_static_scratch(output, query, key_cache, value_cache, block_tables, context_lens, num_queries_per_tokens,
                       sm_scale, block_size, max_context_len, max_num_partitions, sinks=None, *, partition_size=0):
    """``run`` for callers that cannot allocate (no upstream counterpart): the C entry point
    ``fa_paged_attention_reduce_static_scratch`` keeps max_logits, exp_sums and tem_output in a fixed
    device array of the library (``_cabi.FA_STATIC_SCRATCH_BYTES``), allocates nothing and is always
    asynchronous on the current stream.  Calls that may overlap on one GPU race for that array."""
    return run_impl("fa_paged_attention_reduce_static_scratch", True, False, None, None, None, output, None, query,
                    key_cache, value_cache, block_tables, context_lens, num_queries_per_tokens, sm_scale, 1.0,
                    block_size, max_context_len, None, sinks, 0.0, timed=False, partition_size=partition_size,
                    static_scratch_partitions=max_num_partitions)
