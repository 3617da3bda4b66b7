"""Pins the oracle's per-layer engine (ring buffer, flush, candidate range, host store,
active-set bookkeeping) against a hand-derived trace and whole-run invariants."""
import pytest
import torch


def _mk(oracle, L, k, g=2, r=3, **kw):
    return oracle.OracleLayer(num_lite_tokens=L, attn_topk=k, num_key_value_groups=g, r=r, max_iter=2,
                              tol=1e-8, capacity=16, compute_dtype=torch.float64, **kw)


def _tokens(gen, b, hq, hkv, n, d):
    return (torch.randn((b, hq, n, d), generator=gen), torch.randn((b, hkv, n, d), generator=gen),
            torch.randn((b, hkv, n, d), generator=gen))


def test_ring_trace_l10_L3(oracle):
    """l=10 prompt tokens, L=3, k=4: lite_indices / lite_len / current_len / host rows /
    candidate count m per step, derived by hand from lrqk_attention.py:1174-1196,
    1493-1496, 1562-1569."""
    g = torch.Generator().manual_seed(0)
    b, hq, hkv, d = 1, 4, 2, 8
    Q, K, V = _tokens(g, b, hq, hkv, 10, d)
    eng = _mk(oracle, L=3, k=4)
    eng.prefill(Q, K, V, generator=g)
    assert eng.lite_indices == [7, 8, 9] and eng.lite_len == 0 and eng.current_len == 10
    assert len(eng.KVcpu) == 10
    expect = [  # (lite_indices, lite_len, current_len, host rows, m)
        ([10, 8, 9], 1, 11, 10, 7),
        ([10, 11, 9], 2, 12, 10, 8),
        ([10, 11, 12], 0, 13, 13, 9),
        ([13, 11, 12], 1, 14, 13, 10),
    ]
    for li, ll, cur, rows, m in expect:
        q, k, v = _tokens(g, b, hq, hkv, 1, d)
        eng.decode(q, k, v)
        assert (eng.lite_indices, eng.lite_len, eng.current_len, len(eng.KVcpu), eng.last_m) == (li, ll, cur, rows, m)
        assert int(eng.last_new_indices.max()) < m


def test_zero_row_for_new_token(oracle):
    """The A_K row gathered for the token being decoded is all zeros (read from the
    zero-initialised tail before k_hat is appended)."""
    g = torch.Generator().manual_seed(1)
    Q, K, V = _tokens(g, 1, 4, 2, 12, 8)
    eng = _mk(oracle, L=3, k=4)
    eng.prefill(Q, K, V, generator=g)
    q, k, v = _tokens(g, 1, 4, 2, 1, 8)
    eng._append(k, v)
    act = eng._A_K_hitted_with_lite()
    assert act.shape == (1, 4, 7, 3)
    assert act[:, :, 4 + 0].abs().sum() == 0          # ring slot 0 holds the new token
    assert act[:, :, 4 + 1].abs().sum() > 0


def test_whole_run_invariants(oracle):
    """After every step: topk slots hold exactly the rows named by hit_indices, ring slots
    hold the ring tokens, and the host store holds every flushed token in order."""
    gen = torch.Generator().manual_seed(2)
    b, hq, hkv, d, L, k, g = 2, 4, 2, 8, 4, 8, 2
    l = 40
    Q, K, V = _tokens(gen, b, hq, hkv, l, d)
    eng = _mk(oracle, L=L, k=k)
    eng.prefill(Q, K, V, generator=gen)
    allK, allV = K.clone(), V.clone()
    n_evicted = 0
    for step in range(30):
        q, kk, vv = _tokens(gen, b, hq, hkv, 1, d)
        allK, allV = torch.cat([allK, kk], 2), torch.cat([allV, vv], 2)
        Kg, Vg = eng.decode(q, kk, vv)
        assert Kg.shape == (b, hq, k + L, d)
        hit = eng.hit_indices[..., 0]
        for h in range(hq):
            for bb in range(b):
                assert torch.equal(Kg[bb, h, :k], allK[bb, h // g, hit[bb, h]])
                assert torch.equal(Vg[bb, h, :k], allV[bb, h // g, hit[bb, h]])
                assert len(set(hit[bb, h].tolist())) == k
                for s, tok in enumerate(eng.lite_indices):
                    assert torch.equal(Kg[bb, h, k + s], allK[bb, h // g, tok])
        flushed = len(eng.KVcpu)
        assert torch.equal(eng.KVcpu.tensor()[..., :d], allK[:, :, :flushed])
        assert torch.equal(eng.KVcpu.tensor()[..., d:], allV[:, :, :flushed])
        assert eng.current_len == l + step + 1 and eng.A_K.shape[2] == eng.current_len
        # Q1: the token that just left the ring is not a candidate and not in the ring
        gap = eng.last_m
        assert gap not in eng.lite_indices and int(hit.max()) < gap
        n_evicted += int(eng.last_evict.sum())
    assert n_evicted > 0


def test_edge_branch_and_dense_identity(oracle):
    """Prefill with k <= l <= k+L keeps every token on the 'GPU' side and decode returns a
    growing prefix (lrqk_attention.py:1444-1466, 1526-1545).  On the first main-branch step
    the active set is every token except the one-token gap, so attention over the returned
    K,V equals dense attention with that single token masked."""
    gen = torch.Generator().manual_seed(3)
    b, hq, hkv, d, L, k, g = 1, 4, 2, 8, 3, 7, 2
    Q, K, V = _tokens(gen, b, hq, hkv, 8, d)
    eng = _mk(oracle, L=L, k=k)
    eng.prefill(Q, K, V, generator=gen)
    assert eng.lite_len == 1 and eng.lite_indices == [7, -1, -1] and len(eng.KVcpu) == 7
    allK, allV = K.clone(), V.clone()
    for step in range(2):
        q, kk, vv = _tokens(gen, b, hq, hkv, 1, d)
        allK, allV = torch.cat([allK, kk], 2), torch.cat([allV, vv], 2)
        Kg, Vg = eng.decode(q, kk, vv)
        assert Kg.shape[2] == 9 + step
        assert torch.equal(Kg, oracle.repeat_kv(allK, g))
    assert len(eng.KVcpu) == 10 and eng.lite_len == 0
    # first main-branch step
    q, kk, vv = _tokens(gen, b, hq, hkv, 1, d)
    allK, allV = torch.cat([allK, kk], 2), torch.cat([allV, vv], 2)
    Kg, Vg = eng.decode(q, kk, vv)
    assert eng.last_m == 7 and eng.lite_indices == [10, 8, 9] and not eng.last_evict.any()
    out = oracle.attention(q, Kg, Vg)
    keep = [t for t in range(11) if t != 7]
    dense = oracle.attention(q, oracle.repeat_kv(allK, g)[:, :, keep], oracle.repeat_kv(allV, g)[:, :, keep])
    assert torch.allclose(out, dense, atol=1e-12)


def test_no_hit_miss_variant_selects_the_same_set(oracle):
    gen = torch.Generator().manual_seed(4)
    b, hq, hkv, d = 1, 4, 2, 8
    Q, K, V = _tokens(gen, b, hq, hkv, 30, d)
    A0 = torch.randn((b, hq, 30, 3), generator=gen)
    e1, e2 = _mk(oracle, L=4, k=8), _mk(oracle, L=4, k=8, no_hit_miss=True)
    e1.prefill(Q, K, V, A_Q0=A0, A_K0=A0.flip(2))
    e2.prefill(Q, K, V, A_Q0=A0, A_K0=A0.flip(2))
    for _ in range(10):
        q, kk, vv = _tokens(gen, b, hq, hkv, 1, d)
        K1, V1 = e1.decode(q, kk, vv)
        K2, V2 = e2.decode(q, kk, vv)
        # same set, different slot order => identical attention
        assert torch.equal(e1.hit_indices.sort(2).values, e2.hit_indices)
        assert torch.allclose(oracle.attention(q, K1, V1), oracle.attention(q, K2, V2), atol=1e-12)


def test_prefill_requires_enough_tokens(oracle):
    gen = torch.Generator().manual_seed(5)
    Q, K, V = _tokens(gen, 1, 2, 2, 5, 8)
    eng = _mk(oracle, L=2, k=6, g=1)
    with pytest.raises(AssertionError):
        eng.prefill(Q, K, V, generator=gen)
