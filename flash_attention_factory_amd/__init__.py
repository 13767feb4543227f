"""MI355X-native paged-attention decode kernels (loop, split-context + reduce and
their FP8-E5M2 KV-cache variants) behind a C ABI, with ``lib.paged_attention_*``
modules that present the upstream ``run(...)`` call."""

__all__ = ["lib", "workloads"]
