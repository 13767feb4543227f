"""Upstream's tests import the four operators as ``from lib import paged_attention_loop``
(test_paged.py:2-3, test_paged_fp8cache.py:2-3) and call ``run`` positionally with 17 arguments
(18 with ``fp8_scale``: test_paged.py:465-483, test_paged_fp8cache.py:476-516)."""
import importlib
import inspect


def _positional(fn):
    kinds = (inspect.Parameter.POSITIONAL_ONLY, inspect.Parameter.POSITIONAL_OR_KEYWORD)
    return [p.name for p in inspect.signature(fn).parameters.values() if p.kind in kinds]


def test_upstream_import_lines_resolve():
    from lib import paged_attention_loop, paged_attention_reduce        # test_paged.py:2-3
    from lib import paged_attention_fp8_loop, paged_attention_fp8_reduce  # test_paged_fp8cache.py:2-3
    import flash_attention_factory_amd.lib as inner
    assert paged_attention_loop is inner.paged_attention_loop
    assert importlib.import_module("lib.paged_attention_reduce") is inner.paged_attention_reduce
    upstream = ["max_logits", "exp_sums", "tem_output", "output", "debug_output", "query", "key_cache", "value_cache",
                "block_tables", "context_lens", "num_queries_per_tokens", "sm_scale", "block_size", "max_context_len",
                "alibi_slopes", "sinks", "softcap"]  # paged_attention_loop.cpp:21-38
    for mod in (paged_attention_loop, paged_attention_reduce):
        assert _positional(mod.run) == upstream and len(upstream) == 17
    fp8 = upstream[:12] + ["fp8_scale"] + upstream[12:]  # paged_attention_fp8_loop.cpp:33-34
    for mod in (paged_attention_fp8_loop, paged_attention_fp8_reduce):
        assert _positional(mod.run) == fp8 and len(fp8) == 18
    # everything this build adds is keyword-only, so upstream's positional calls mean what they meant
    for mod in (paged_attention_loop, paged_attention_reduce, paged_attention_fp8_loop, paged_attention_fp8_reduce):
        extra = [p for p in inspect.signature(mod.run).parameters.values() if p.name not in fp8]
        assert extra and all(p.kind is inspect.Parameter.KEYWORD_ONLY and p.default is not inspect.Parameter.empty
                             for p in extra)
