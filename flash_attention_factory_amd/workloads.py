"""Synthetic paged-KV decode workloads.

Two families:

* ``make_config(i)`` -- the five measured configurations (shapes, length
  distributions, pool sizes and cache dtypes as the benchmark contract names
  them).  Draw order on one seeded generator: query, K pool, V pool, block
  permutation, context lengths.
* ``make_test_shaped(...)`` -- inputs shaped like the upstream test grid
  (reference test_paged.py:211-256 parametrisation, generator call order of
  test_paged.py:291-341: query, K pool, V pool, ``randperm`` block table, the
  unused ``cache_seqlens`` draw, then the var-len lengths), token-major cache
  layout ``[num_blocks, block_size, num_kv_heads, head_size]`` and block size 64.

Everything is drawn on the CPU generator so the same seed gives the same bits
on any machine; tensors are then moved to the requested device.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Optional

import torch

HEAD_MAJOR = "head_major"    # [num_blocks, num_kv_heads, block_size, head_size]
TOKEN_MAJOR = "token_major"  # [num_blocks, block_size, num_kv_heads, head_size]


@dataclass
class Workload:
    name: str
    query: torch.Tensor            # [S, H, D] fp16 / bf16
    key_cache: torch.Tensor        # 4-D pool, 16-bit, float8_e5m2 or float8_e4m3fn
    value_cache: torch.Tensor
    block_tables: torch.Tensor     # [S, MB] int32
    context_lens: torch.Tensor     # [S] int32
    scale: float
    block_size: int
    num_kv_heads: int
    layout: str
    partition_size: int
    sinks: Optional[torch.Tensor] = None  # [H] in the query dtype
    fp8_scale: float = 1.0
    meta: dict = field(default_factory=dict)

    @property
    def is_fp8(self) -> bool:
        return self.key_cache.dtype in (torch.float8_e5m2, torch.float8_e4m3fn)

    @property
    def num_seqs(self) -> int:
        return self.query.shape[0]

    @property
    def num_heads(self) -> int:
        return self.query.shape[1]

    @property
    def head_size(self) -> int:
        return self.query.shape[2]

    @property
    def max_num_partitions(self) -> int:
        return max(1, math.ceil(int(self.context_lens.max()) / self.partition_size))

    def kv_strides(self):
        """(block, token, head) strides of the caches in elements."""
        st = self.key_cache.stride()
        if self.layout == HEAD_MAJOR:
            return (st[0], st[2], st[1])
        return (st[0], st[1], st[2])

    def algorithmic_bytes(self) -> int:
        """K and V once per kv head and token, q read, out written, the block-table
        entries and context lengths a call has to read."""
        lens = self.context_lens.to(torch.int64).cpu()
        kv_b = self.key_cache.element_size()
        q_b = self.query.element_size()
        S, H, D = self.query.shape
        kv = int(lens.sum()) * self.num_kv_heads * D * 2 * kv_b
        qo = 2 * S * H * D * q_b
        bt = int(((lens + self.block_size - 1) // self.block_size).sum()) * 4
        return kv + qo + bt + S * 4

    def scratch_bytes(self) -> int:
        """exp_sums/max_logits/tmp_out bytes written by the partition pass and read
        back by the reduce pass (2x this crosses HBM)."""
        lens = self.context_lens.to(torch.int64).cpu()
        S, H, D = self.query.shape
        parts = int(((lens + self.partition_size - 1) // self.partition_size).sum())
        return parts * H * (D + 2) * 4

    def algorithmic_flops(self) -> int:
        lens = self.context_lens.to(torch.int64).cpu()
        S, H, D = self.query.shape
        return int(lens.sum()) * H * D * 4

    def to(self, device) -> "Workload":
        def mv(t):
            return None if t is None else t.to(device)
        return Workload(self.name, mv(self.query), mv(self.key_cache), mv(self.value_cache),
                        mv(self.block_tables), mv(self.context_lens), self.scale, self.block_size,
                        self.num_kv_heads, self.layout, self.partition_size, mv(self.sinks),
                        self.fp8_scale, dict(self.meta))


def _randn16(shape, gen, dtype):
    # fp32 draw then cast: identical bits to drawing in fp16 would not be guaranteed
    # across torch versions, while this form is.
    n = 1
    for s in shape:
        n *= s
    out = torch.empty(shape, dtype=dtype)
    flat = out.view(-1)
    step = 1 << 26
    for lo in range(0, n, step):
        hi = min(n, lo + step)
        flat[lo:hi] = torch.randn(hi - lo, generator=gen, dtype=torch.float32).to(dtype)
    return out


def _deal_block_tables(lens, block_size, perm):
    """Deal a random permutation of the pool's block ids to the sequences without
    replacement; unused table slots hold 0."""
    need = [(int(n) + block_size - 1) // block_size for n in lens]
    total = sum(need)
    if total > perm.numel():
        raise ValueError(f"workload needs {total} blocks, pool has {perm.numel()}")
    mb = max(1, max(need))
    tables = torch.zeros((len(need), mb), dtype=torch.int32)
    off = 0
    for s, nb in enumerate(need):
        tables[s, :nb] = perm[off:off + nb]
        off += nb
    return tables


_CONFIGS = {
    0: dict(S=4, H=8, Hk=8, D=64, B=16, NB=128, lens=("uniform", 1, 256), q=torch.float16, fp8=False),
    1: dict(S=32, H=32, Hk=32, D=128, B=16, NB=4096, lens=("uniform", 512, 2048), q=torch.float16, fp8=False),
    2: dict(S=8, H=32, Hk=8, D=128, B=16, NB=16384, lens=("uniform", 8192, 32768), q=torch.float16, fp8=False),
    3: dict(S=32, H=32, Hk=32, D=128, B=16, NB=4096, lens=("uniform", 512, 2048), q=torch.float16, fp8=True),
    4: dict(S=128, H=64, Hk=8, D=128, B=16, NB=65536, lens=("lognormal", 4096, 0.75, 64, 32768),
            q=torch.bfloat16, fp8=True),
}
CONFIG_KERNEL = {0: "loop", 1: "loop", 2: "reduce", 3: "fp8_loop", 4: "fp8_reduce"}


def config_names():
    return {i: f"config{i}_{CONFIG_KERNEL[i]}" for i in _CONFIGS}


def _draw_lens(spec, S, gen):
    if spec[0] == "uniform":
        return torch.randint(spec[1], spec[2] + 1, (S,), generator=gen, dtype=torch.int64).to(torch.int32)
    _, median, sigma, lo, hi = spec
    z = torch.randn(S, generator=gen, dtype=torch.float64)
    lens = torch.exp(math.log(median) + sigma * z).round().clamp(lo, hi)
    return lens.to(torch.int32)


def _randn16_on(shape, device, seed, dtype):
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    return torch.randn(shape, generator=gen, device=device, dtype=torch.float16).to(dtype)


def make_config(index: int, *, seed: int = 0, layout: str = HEAD_MAJOR, num_seqs: Optional[int] = None,
                pool_blocks: Optional[int] = None, device="cpu", pools_on_device: bool = False,
                lens=None, fp8_dtype=torch.float8_e5m2) -> Workload:
    """One of the five measured configurations.  ``num_seqs``/``pool_blocks`` shrink
    a configuration for CPU-sized parity runs without changing anything else.
    ``pools_on_device`` draws the two KV pools with the target device's own generator
    (same distribution, different bits) -- for throughput runs, where drawing a
    gigabyte of normals on the host would dominate the run.  ``lens`` replaces the
    drawn context lengths (the block tables are dealt for the lengths in force).
    ``fp8_dtype`` is the byte format of an FP8 configuration's pools: E5M2 as upstream,
    or ``torch.float8_e4m3fn``."""
    c = _CONFIGS[index]
    S = num_seqs or c["S"]
    H, Hk, D, B = c["H"], c["Hk"], c["D"], c["B"]
    NB = pool_blocks or c["NB"]
    qd = c["q"]
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed)
    query = _randn16((S, H, D), gen, qd)
    shape = (NB, Hk, B, D) if layout == HEAD_MAJOR else (NB, B, Hk, D)
    kv16 = torch.float16 if c["fp8"] else qd
    if pools_on_device:
        k = _randn16_on(shape, device, seed + 1, kv16)
        v = _randn16_on(shape, device, seed + 2, kv16)
    else:
        k = _randn16(shape, gen, kv16)
        v = _randn16(shape, gen, kv16)
    if c["fp8"]:
        # cast of fp16 N(0,1) samples, as test_paged_fp8cache.py:201-203 does
        k = k.to(fp8_dtype)
        v = v.to(fp8_dtype)
    perm = torch.randperm(NB, generator=gen, dtype=torch.int64).to(torch.int32)
    drawn = _draw_lens(c["lens"], S, gen)
    lens = drawn if lens is None else torch.as_tensor(lens, dtype=torch.int32)
    assert lens.numel() == S
    tables = _deal_block_tables(lens, B, perm)
    w = Workload(
        name=config_names()[index], query=query, key_cache=k, value_cache=v, block_tables=tables,
        context_lens=lens, scale=1.0 / math.sqrt(D), block_size=B, num_kv_heads=Hk, layout=layout,
        partition_size=512, sinks=None, fp8_scale=1.0,
        meta=dict(config=index, kernel=CONFIG_KERNEL[index], seed=seed, pool_blocks=NB))
    return w.to(device) if str(device) != "cpu" else w


def make_test_shaped(*, batch_size: int, nheads: int, nheads_k: int, d: int, seqlen_k: int,
                     varlen: bool, has_sinks: bool, fp8: bool = False, block_size: int = 64,
                     seed: int = 0, dtype=torch.float16, layout: str = TOKEN_MAJOR,
                     device="cpu", fp8_dtype=torch.float8_e5m2) -> Workload:
    """Inputs shaped like one case of the upstream test grid."""
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed)
    query = _randn16((batch_size, nheads, d), gen, dtype)  # seqlen_q == 1 folded away
    nblk_seq = math.ceil(seqlen_k / block_size)
    NB = nblk_seq * batch_size
    shape = (NB, block_size, nheads_k, d) if layout == TOKEN_MAJOR else (NB, nheads_k, block_size, d)
    k = _randn16(shape, gen, dtype)
    v = _randn16(shape, gen, dtype)
    tables = torch.randperm(NB, generator=gen, dtype=torch.int64).to(torch.int32).view(batch_size, nblk_seq)
    _ = torch.randint(1, seqlen_k + 1, (batch_size,), generator=gen)  # cache_seqlens: drawn, unused
    if varlen:
        lens = torch.randint(max(1, seqlen_k - 20), seqlen_k + 1, (batch_size,), generator=gen).to(torch.int32)
    else:
        lens = torch.full((batch_size,), seqlen_k, dtype=torch.int32)
    if fp8:
        k = k.to(fp8_dtype)
        v = v.to(fp8_dtype)
    sinks = torch.full((nheads,), 10.0, dtype=dtype) if has_sinks else None
    # upstream partition size: (head_size / 16) sub-groups x block_size tokens
    partition_size = (d // 16) * block_size if block_size == 64 else 512
    w = Workload(
        name=f"grid_b{batch_size}_h{nheads}x{nheads_k}_d{d}_s{seqlen_k}_{'var' if varlen else 'full'}"
             f"{'_sink' if has_sinks else ''}{'_fp8' if fp8 else ''}",
        query=query, key_cache=k, value_cache=v, block_tables=tables.contiguous(), context_lens=lens,
        scale=1.0 / math.sqrt(d), block_size=block_size, num_kv_heads=nheads_k, layout=layout,
        partition_size=partition_size, sinks=sinks, fp8_scale=1.0,
        meta=dict(seed=seed, pool_blocks=NB))
    return w.to(device) if str(device) != "cpu" else w
