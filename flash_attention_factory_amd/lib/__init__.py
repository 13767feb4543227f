"""The four modules the upstream tests import (``from lib import paged_attention_loop``,
test_paged.py:2-3, test_paged_fp8cache.py:2-3), each exposing ``run(...)``, and
``kv_cache_write`` -- the step upstream has only as test code
(test_paged_fp8cache.py:171-203) that fills the pools those four read."""
from . import (kv_cache_write, paged_attention_fp8_loop, paged_attention_fp8_reduce, paged_attention_loop,
               paged_attention_reduce)

__all__ = ["paged_attention_loop", "paged_attention_reduce", "paged_attention_fp8_loop",
           "paged_attention_fp8_reduce", "kv_cache_write"]
