"""The order in which the persistent loop kernels list a sequence's kv heads (csrc/paged_attention_utils.h:
stack_affine_shift, stack_affine_head), restated on the host: whatever the pool, every head is listed exactly
once, and where the map applies the q-th item's chunk lies in the 4 KiB units that go to memory stack q mod 8."""
import pytest


def stack_affine_shift(head_chunk_bytes: int, heads: int) -> int:
    if head_chunk_bytes < 1024 or head_chunk_bytes > 4096 or head_chunk_bytes & (head_chunk_bytes - 1):
        return -1
    shift = {4096: 0, 2048: 1, 1024: 2}[head_chunk_bytes]
    return shift if heads % (8 << shift) == 0 else -1


def stack_affine_head(q: int, shift: int) -> int:
    if shift < 0:
        return q
    k, a = q & 7, q >> 3
    return ((a >> shift) << (shift + 3)) | (k << shift) | (a & ((1 << shift) - 1))


@pytest.mark.parametrize("chunk", [128, 256, 512, 1024, 2048, 3072, 4096, 8192])
@pytest.mark.parametrize("heads", [1, 2, 3, 4, 8, 12, 16, 24, 32, 40, 64, 128])
def test_every_head_once_and_on_its_stack(chunk, heads):
    shift = stack_affine_shift(chunk, heads)
    listed = [stack_affine_head(q, shift) for q in range(heads)]
    assert sorted(listed) == list(range(heads))
    if shift >= 0:
        assert all(((h * chunk) >> 12) & 7 == q & 7 for q, h in enumerate(listed))
    else:
        assert listed == list(range(heads))


def test_where_the_map_applies():
    assert stack_affine_shift(4096, 32) == 0    # 16-bit cache, head size 128, blocks of 16: plain order is the map
    assert [stack_affine_head(q, 0) for q in range(32)] == list(range(32))
    assert stack_affine_shift(2048, 32) == 1    # byte cache, same shape
    assert [stack_affine_head(q, 1) for q in range(16)] == [0, 2, 4, 6, 8, 10, 12, 14, 1, 3, 5, 7, 9, 11, 13, 15]
    assert stack_affine_shift(2048, 8) == -1    # too few heads to give every stack one
    assert stack_affine_shift(256, 32) == -1    # upstream's layout: a head's share of a block is one token row at a time
