"""``paged_attention_loop.run``: the single-pass kernel.

Drop-in for the upstream extension module of the same name
(paged_attention_loop/paged_attention_loop.cpp:21-38,82-84): same positional arguments, same return value
(a list of kernel times in microseconds).  ``timed=False`` (keyword only, not in
upstream) launches asynchronously on the current stream and returns ``[]``.
``apply_alibi``, ``apply_softcap`` and ``window_left`` (keyword only) switch on the score
modifiers upstream's kernels take and ignore (paged_attention_kernel_loop.hpp:329-342).
"""
from ._run import run_impl


def run(max_logits, exp_sums, tem_output, output, debug_output, query, key_cache, value_cache,
        block_tables, context_lens, num_queries_per_tokens, sm_scale, block_size, max_context_len,
        alibi_slopes, sinks, softcap, *, timed=True, apply_alibi=False, apply_softcap=False, window_left=None, schedule=0, spin_limit=0):
    return run_impl("fa_paged_attention_loop", False, False, max_logits, exp_sums, tem_output, output,
                    debug_output, query, key_cache, value_cache, block_tables, context_lens,
                    num_queries_per_tokens, sm_scale, 1.0, block_size, max_context_len,
                    alibi_slopes, sinks, softcap, timed=timed, apply_alibi=apply_alibi, apply_softcap=apply_softcap,
                    window_left=window_left, schedule=schedule, spin_limit=spin_limit)
