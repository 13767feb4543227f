"""The torch.library operators register without a GPU, have no CPU implementation to fall
back on, and trace through their fake kernels."""
import pytest
import torch

from flash_attention_factory_amd import torch_ops  # noqa: F401


def test_operators_are_registered():
    for name in ("paged_attention_loop", "paged_attention_reduce", "paged_attention_fp8_loop",
                 "paged_attention_fp8_reduce", "kv_cache_write"):
        assert hasattr(torch.ops.fa_amd, name), name


def test_no_cpu_fallback():
    q = torch.zeros((1, 2, 64), dtype=torch.float16)
    pool = torch.zeros((2, 16, 2, 64), dtype=torch.float16)
    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops.fa_amd.paged_attention_loop(torch.zeros_like(q), q, pool, pool, torch.zeros((1, 2), dtype=torch.int32),
                                              torch.ones(1, dtype=torch.int32), 0.125, None)
    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops.fa_amd.kv_cache_write(torch.zeros((1, 2, 64), dtype=torch.float16), torch.zeros((1, 2, 64), dtype=torch.float16),
                                        pool, pool.clone(), torch.zeros(1, dtype=torch.int64), 1.0)


def test_fake_kernels_trace_on_meta_tensors():
    q = torch.zeros((1, 2, 64), dtype=torch.float16, device="meta")
    pool = torch.zeros((2, 16, 2, 64), dtype=torch.float16, device="meta")
    out = torch.zeros_like(q)
    assert torch.ops.fa_amd.paged_attention_loop(out, q, pool, pool, torch.zeros((1, 2), dtype=torch.int32, device="meta"),
                                                 torch.ones(1, dtype=torch.int32, device="meta"), 0.125, None) is None
