"""The import name upstream's tests use: ``from lib import paged_attention_loop`` (test_paged.py:2-3,
test_paged_fp8cache.py:2-3; upstream's build installs its four extension modules into a folder of
that name, CMakeLists.txt:74-78).  The modules are those of ``flash_attention_factory_amd.lib``."""
import sys as _sys

from flash_attention_factory_amd.lib import (kv_cache_write, paged_attention_fp8_loop, paged_attention_fp8_reduce,
                                             paged_attention_loop, paged_attention_reduce)

__all__ = ["paged_attention_loop", "paged_attention_reduce", "paged_attention_fp8_loop",
           "paged_attention_fp8_reduce", "kv_cache_write"]
for _name in __all__:  # `import lib.paged_attention_loop` finds the same module objects
    _sys.modules[f"{__name__}.{_name}"] = globals()[_name]
