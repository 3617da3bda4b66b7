"""Host logic of the cache front door and its bounded buffers, without a GPU: the per-layer state
table of DynamicLRQKCache (contract of lrqk_attention.py:1861-1970) driven with a stand-in engine, and
PreAllocatedTensor / _CacheQKV (lrqk_attention.py:966-1028)."""
import pytest
import torch

from lrqk_amd.buffers import PreAllocatedTensor, _CacheQKV
from lrqk_amd.cache import DynamicLRQKCache


class _Recorder:
    """Stands in for an engine: remembers what the cache handed to it."""

    made = []

    def __init__(self, **kwargs):
        self.kwargs, self.prefilled, self.decoded, self.length = kwargs, None, 0, 0
        _Recorder.made.append(self)

    def prefill(self, query_states, key_states, value_states):
        self.prefilled = (query_states.clone(), key_states.clone(), value_states.clone())
        self.length = key_states.shape[2]

    def decode(self, q, k, v):
        self.decoded += 1
        self.length += 1
        return "K-active", "V-active"

    def __len__(self):
        return self.length


def _pieces(n, b=2, hq=4, hkv=2, d=8, seed=0):
    g = torch.Generator().manual_seed(seed + n)
    return (torch.randn((b, hq, n, d), generator=g), torch.randn((b, hkv, n, d), generator=g),
            torch.randn((b, hkv, n, d), generator=g))


def test_bounded_buffer():
    buf = PreAllocatedTensor(6, 1)
    assert not buf.has_data() and len(buf) == 0 and buf.dtype is None and buf.device is None
    a, b = torch.arange(12.).view(2, 2, 3), torch.arange(24.).view(2, 4, 3) + 100
    buf.append(a)
    assert buf.has_data() and buf.data.shape == (2, 6, 3) and buf.dtype == a.dtype and buf.device == a.device
    buf.append(b)
    assert len(buf) == 6 and torch.equal(buf.tensor(), torch.cat([a, b], 1)) and torch.equal(buf[1], torch.cat([a, b], 1)[1])
    with pytest.raises(ValueError, match="Not enough capacity"):
        buf.append(a[:, :1])
    assert len(buf) == 6                                   # a refused piece leaves the buffer as it was
    same = PreAllocatedTensor.from_tensor(5, 0, torch.ones(3, 2, dtype=torch.float64))
    assert len(same) == 3 and same.capacity == 5 and same.dtype == torch.float64 and same.data.shape == (5, 2)


def test_prompt_pieces_buffer():
    held = _CacheQKV(5, 2)
    q, k, v = _pieces(3)
    Q, K, V = held.append(q, k, v)
    assert len(held) == 3 and torch.equal(Q, q) and torch.equal(K, k) and torch.equal(V, v)
    q2, k2, v2 = _pieces(2)
    Q, K, V = held.append(q2, k2, v2)
    assert len(held) == 5 and torch.equal(K, torch.cat([k, k2], 2)) and torch.equal(V, torch.cat([v, v2], 2))
    assert held.Q.capacity == held.K.capacity == held.V.capacity == 5
    with pytest.raises(ValueError):
        held.append(*_pieces(1))


def test_state_table():
    _Recorder.made.clear()
    cache = DynamicLRQKCache(r=4, num_active_tokens=8, lite_tokens=2, max_iter=(3, 1), tol=1e-3, max_sequence_length=64,
                             num_key_value_groups=2, lwattn_factory=_Recorder)
    S = cache.State
    with pytest.raises(ValueError):
        cache.update(*_pieces(1)[:2], None, 0)
    assert len(cache) == 0                                 # a refused call touches no layer
    # long prompt: factorised at once; the mask is multiplied into K and V in place
    q, k, v = _pieces(9)
    mask = torch.ones(2, 9)
    mask[0, :2] = 0
    k_before = k.clone()
    K, V = cache.update(q, k, v, 0, attention_mask=mask)
    eng = cache.lwattn[0]
    assert K is k and V is v and cache.sequence_state[0] == S.decoding and len(_Recorder.made) == 1
    assert torch.equal(k[0, :, :2], torch.zeros_like(k[0, :, :2])) and torch.equal(k[1], k_before[1])
    assert torch.equal(eng.prefilled[1], k) and cache.get_seq_length(0) == 9 == cache.seen_tokens
    from lrqk_amd.factor import InitAQAK
    assert eng.kwargs == dict(num_lite_tokens=2, attn_topk=8, num_key_value_groups=2, r=4, max_iter=(3, 1), tol=1e-3,
                              capacity=64, init_aq_ak_method=InitAQAK.randn)
    assert cache.update(*_pieces(1), 0) == ("K-active", "V-active") and eng.decoded == 1
    # short pieces: returned raw the first time, as everything held so far afterwards, no engine yet
    q1, k1, v1 = _pieces(3)
    K, V = cache.update(q1, k1, v1, 1, attention_mask=None)
    assert K is k1 and cache.sequence_state[1] == S.collecting and len(_Recorder.made) == 1
    q2, k2, v2 = _pieces(4)
    K, V = cache.update(q2, k2, v2, 1, attention_mask=torch.zeros(2, 4))     # a mask is only used on the first call
    assert K.shape[2] == 7 and torch.equal(K, torch.cat([k1, k2], 2)) and cache.sequence_state[1] == S.collecting
    # too long a piece overflows the k-row buffer: ValueError, state kept
    with pytest.raises(ValueError):
        cache.update(*_pieces(2), 1)
    assert cache.sequence_state[1] == S.collecting and 1 in cache.temp_buff_cache_qkv
    # ... the overflow came after Q was appended (three separate buffers, as in the reference), so layer 1 is
    # finished on a fresh layer instead
    q1, k1, v1 = _pieces(5)
    cache.update(q1, k1, v1, 2)
    q2, k2, v2 = _pieces(3)
    K, V = cache.update(q2, k2, v2, 2)
    assert cache.sequence_state[2] == S.decoding and 2 not in cache.temp_buff_cache_qkv and len(_Recorder.made) == 2
    assert torch.equal(K, torch.cat([k1, k2], 2)) and torch.equal(cache.lwattn[2].prefilled[0], torch.cat([q1, q2], 2))
    assert len(cache) == 3
    with pytest.raises(NotImplementedError):
        cache[0]
    with pytest.raises(NotImplementedError):
        iter(cache)


class _WideRecorder(_Recorder):
    """An engine stand-in that returns an 'active set' of the width it was given."""

    def decode(self, q, k, v):
        self.decoded += 1
        self.length += 1
        self.last = (q.clone(), k.clone(), v.clone())
        return torch.cat([k, k], 2).repeat_interleave(2, 1), torch.cat([v, v], 2).repeat_interleave(2, 1)


def test_other_head_widths_are_padded_for_the_engine():
    """Rows of 96 fp32 elements reach the engine as rows of 128 with zero columns; the caller gets its own
    tensors back from the prompt call and rows of 96 from a decode call.  Widths the kernels take as they are
    (powers of two of at least 16 bytes) pass through untouched."""
    assert [DynamicLRQKCache._padded_width(d, 2) for d in (96, 80, 128, 64, 8, 4, 192, 256)] == \
        [128, 128, 128, 64, 8, 8, 256, 256]
    assert [DynamicLRQKCache._padded_width(d, 4) for d in (96, 4, 3, 2)] == [128, 4, 4, 4]
    _Recorder.made.clear()
    cache = DynamicLRQKCache(r=4, num_active_tokens=8, lite_tokens=2, num_key_value_groups=2, lwattn_factory=_WideRecorder)
    q, k, v = _pieces(9, d=96)
    K, V = cache.update(q, k, v, 0)
    eng = cache.lwattn[0]
    assert K is k and V is v
    for given, seen in zip((q, k, v), eng.prefilled):
        assert seen.shape[-1] == 128 and torch.equal(seen[..., :96], given) and seen[..., 96:].abs().sum() == 0
    q1, k1, v1 = _pieces(1, d=96)
    K, V = cache.update(q1, k1, v1, 0)
    assert eng.last[0].shape[-1] == 128 and torch.equal(eng.last[1][..., :96], k1)
    assert K.shape == (2, 4, 2, 96) and torch.equal(K[:, ::2, :1], k1) and torch.equal(V[:, ::2, :1], v1)
    eng.attn_in_step = True
    with pytest.raises(NotImplementedError):
        cache.update(q1, k1, v1, 0)
    # a width the kernels take: the engine gets the caller's own tensors
    q, k, v = _pieces(9, d=64)
    cache.update(q, k, v, 1)
    assert cache.lwattn[1].prefilled[1].shape[-1] == 64
    q1, k1, v1 = _pieces(1, d=64)
    K, V = cache.update(q1, k1, v1, 1)
    assert K.shape[-1] == 64 and cache.lwattn[1].last[1].data_ptr() != k1.data_ptr()  # (the stand-in clones)
