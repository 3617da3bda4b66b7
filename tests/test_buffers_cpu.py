"""The four behaviours that the reference's own buffer tests hold (lrqk_attention_test.py:10-66), asked of
lrqk_amd.buffers.AutoIncreaseTensor itself: length after random appends along dim 0, indexing while the buffer grows
from a small and from a large first capacity, and growth along dim 2 with 4-D data.  The reference's second test runs
on its GPU; its twin here carries the gpu marker, the others need no GPU.  Beyond the reference's asserts: the capacity
policy (first allocation, x1.5 growth) and the zero tail that the decode step relies on, compared with the oracle's
buffer after every append."""
import random

import pytest
import torch

from lrqk_amd.buffers import AutoIncreaseTensor, AutoIncreaseTensorSharedKV


def test_append_length_dim0():                     # lrqk_attention_test.py:10-19
    rnd = random.Random(0)
    ait = AutoIncreaseTensor(capacity=16, dim=0)
    total = 0
    for _ in range(10):
        s = rnd.randint(1, 16)
        total += s
        ait.append(torch.randn(s, 128))
        assert len(ait) == total
        assert ait.capacity > len(ait) and ait.data.shape[0] == ait.capacity


def _getitem_while_growing(capacity, device, seed):
    rnd = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    ait = AutoIncreaseTensor(capacity=capacity, dim=0, device=device)
    target = torch.randn(512, 128, generator=g)
    ll = 0
    while ll < 512:
        s = rnd.randint(1, 16)
        rr = min(ll + s, 512)
        ait.append(target[ll:rr])
        ll = rr
        if rr < 2:
            continue
        s = rnd.randint(1, rr - 1)
        assert torch.equal(ait[:s].cpu(), target[:s])
        assert torch.equal(ait[:s, 0].cpu(), target[:s, 0])
        assert torch.equal(ait[s].cpu(), target[s])
        assert ait[s].device == ait.data.device
    assert len(ait) == 512
    return ait


def test_getitem_small_first_capacity():           # lrqk_attention_test.py:21-38 (there on cuda:0)
    ait = _getitem_while_growing(16, None, 1)
    assert ait.capacity > 512 and float(ait.data[512:].abs().sum()) == 0.0   # grown several times, zero tail


@pytest.mark.gpu
def test_getitem_small_first_capacity_on_the_gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    ait = _getitem_while_growing(16, "cuda:0", 2)
    assert ait.data.is_cuda and float(ait.data[512:].abs().sum()) == 0.0


def test_getitem_large_first_capacity():           # lrqk_attention_test.py:40-54
    ait = _getitem_while_growing(1024, None, 3)
    assert ait.capacity == 1024                    # never grown


def test_getitem_dim2_token_by_token():            # lrqk_attention_test.py:56-66
    g = torch.Generator().manual_seed(4)
    ait = AutoIncreaseTensor(capacity=16, dim=2)
    target = torch.randn(2, 8, 512, 128, generator=g)
    ait.append(target[:, :, 0:128])
    assert ait.capacity == 192                     # max(16, int(128 * 1.5)), lrqk_attention.py:880-889
    for i in range(128, 512):
        ait.append(target[:, :, i:i + 1])
        assert torch.equal(ait[:, :, 0:i + 1], target[:, :, 0:i + 1])
        assert ait.shape == (2, 8, i + 1, 128)
    assert float(ait.data[:, :, 512:].abs().sum()) == 0.0


def test_same_capacities_and_contents_as_the_oracle(oracle):
    g = torch.Generator().manual_seed(5)
    for dim, shape in ((0, (0, 8)), (2, (2, 3, 0, 4))):
        mine = AutoIncreaseTensor(capacity=6, dim=dim)
        ref = oracle.OracleAutoIncreaseTensor(capacity=6, dim=dim)
        for _ in range(40):
            n = int(torch.randint(1, 9, (1,), generator=g))
            piece = list(shape)
            piece[dim] = n
            x = torch.randn(piece, generator=g)
            mine.append(x)
            ref.append(x)
            assert mine.capacity == ref.capacity and len(mine) == len(ref)
            assert torch.equal(mine.data, ref.data)          # whole capacity, the zero tail included


def test_shared_kv_rows_and_extend():
    g = torch.Generator().manual_seed(6)
    kv = AutoIncreaseTensorSharedKV(capacity=8, dim=2, device="cpu", pin_memory=False)
    k, v = torch.randn(1, 2, 5, 4, generator=g), torch.randn(1, 2, 5, 4, generator=g)
    kv.append(k, v)
    assert kv.data.shape == (1, 2, 8, 8) and torch.equal(kv.tensor(), torch.cat([k, v], -1))
    first = kv.extend((1, 2, 0, 8), 7)                       # room for rows that a kernel writes
    assert first == 5 and len(kv) == 12 and kv.capacity == 18   # 8 -> 12 -> 18
    assert torch.equal(kv.tensor()[:, :, :5], torch.cat([k, v], -1))


def test_gather_rows_refuses_a_source_of_another_width():
    """ops.gather_rows takes the row width from the source: the 2d-wide [K|V] store as a source would be written
    past the end of the d-wide destination.  The check comes before anything touches a GPU."""
    from lrqk_amd import ops

    class _FakeCuda(torch.Tensor):
        """A CPU tensor that says it lives on the GPU, so that the argument checks can run without one."""
        @property
        def is_cuda(self):
            return True

    def fake(t):
        return t.as_subclass(_FakeCuda)

    dst = fake(torch.zeros(1, 4, 6, 8))
    idx = fake(torch.zeros(1, 4, 3, dtype=torch.int32))
    with pytest.raises(ValueError, match="do not match the destination"):
        ops.gather_rows(fake(torch.zeros(1, 2, 10, 16)), idx, dst, 3)          # [K|V] rows, 2d wide
    with pytest.raises(ValueError, match="do not match the destination"):
        ops.gather_rows(fake(torch.zeros(1, 2, 10, 8, dtype=torch.bfloat16)), idx, dst, 3)
    with pytest.raises(ValueError, match="count slots inside dst"):
        ops.gather_rows(fake(torch.zeros(1, 2, 10, 8)), idx, dst, 4)           # more slots than idx lists
