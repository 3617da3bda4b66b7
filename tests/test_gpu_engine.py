"""Engine-level parity: the GPU engine and the CPU oracle run the same seeded prefill +
decode trace in lockstep.

Floating-point stages (factor updates, attention) are compared within tolerance.  So that
the integer stages can then be compared BIT FOR BIT at every step, the oracle continues
each step from the GPU's (checked) factor outputs: same q_hat => the same proxy scores,
top-k ids, evicted slots, refetched rows, ring contents and host store are required.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _say(*a):
    print(*a, flush=True)


@pytest.fixture(scope="module")
def lrqk():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import lrqk_amd
    return lrqk_amd


def _rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / (b.norm() + 1e-300))


def _lockstep(lrqk, oracle, *, b, hq, hkv, d, l, r, k, L, steps, dtype, max_iter, tol, rho, cls=None, capacity=64,
              seed=0, fp_tol=None, no_hit_miss=False, sigma=0.01, compare_factors=True):
    from lrqk_amd import synth, ops
    g = hq // hkv
    gen = torch.Generator().manual_seed(seed)
    Q, WQ = synth.low_rank_noise(gen, b, hq, l, d, rho, sigma, dtype)
    K, WK = synth.low_rank_noise(gen, b, hkv, l, d, rho, sigma, dtype)
    V, WV = synth.low_rank_noise(gen, b, hkv, l, d, rho, sigma, dtype)
    A_Q0 = torch.randn((b, hq, l, r), generator=gen)
    A_K0 = torch.randn((b, hq, l, r), generator=gen)
    cls = cls or lrqk.LightAttentionIndicesFactory
    eng = cls(num_lite_tokens=L, attn_topk=k, num_key_value_groups=g, r=r, max_iter=max_iter, tol=tol,
              capacity=capacity)
    eng.init_factors = (A_Q0, A_K0)
    eng.attn_in_step = True
    orc = oracle.OracleLayer(num_lite_tokens=L, attn_topk=k, num_key_value_groups=g, r=r, max_iter=max_iter, tol=tol,
                             capacity=capacity, compute_dtype=torch.float64, no_hit_miss=no_hit_miss)
    # default tolerance of the small traces: their data has rank rho == r, so the r x r Gram
    # systems are ill-conditioned (cond ~ 1e4-1e5) and fp32 carries 1e-3..1e-2; the
    # full-shape traces below pass explicit, tighter limits
    lim = fp_tol or (2e-2 if dtype == torch.bfloat16 else 1e-2)

    # ---- prefill
    eng.prefill(Q.to(DEV), K.to(DEV), V.to(DEV))
    ref = oracle.cast_lrqk_prefill(Q, oracle.repeat_kv(K, g), r, max_iter[0], tol[0], A_Q0=A_Q0, A_K0=A_K0,
                                   compute_dtype=torch.float64)
    # fp32 kernels vs the fp64 oracle, both rounded to the storage dtype afterwards: most
    # elements agree exactly, a few differ by one unit in the last place
    gA_K, gB_K, gB_Q = eng.A_K.cpu(), eng.B_K.cpu(), eng.B_Q.cpu()
    gA_Qrow = eng.last_A_Q_row.cpu()
    if compare_factors:
        for name, got, exp in (("A_K", gA_K, ref[2]), ("B_K", gB_K, ref[3]), ("B_Q", gB_Q, ref[1]),
                               ("A_Q[-1]", gA_Qrow, ref[0][:, :, -1:])):
            assert _rel(got, exp) < lim, ("prefill", name, _rel(got, exp))
    # what the factors are for: the fit K ~ A_K B_K and the last query row q ~ a_q B_Q.  These
    # are well determined even where the individual factors are not (badly scaled r x r
    # systems: fp32 LAPACK itself is several percent away from fp64 there)
    K4 = oracle.repeat_kv(K, g).double()
    fit_g = _rel(gA_K.double() @ gB_K.double(), K4)
    fit_o = _rel(ref[2].double() @ ref[3].double(), K4)
    assert abs(fit_g - fit_o) < 2e-3 + 0.05 * fit_o, ("prefill fit K", fit_g, fit_o)
    qfit_g = _rel(gA_Qrow.double() @ gB_Q.double(), Q[:, :, -1:].double())
    qfit_o = _rel(ref[0][:, :, -1:].double() @ ref[1].double(), Q[:, :, -1:].double())
    assert abs(qfit_g - qfit_o) < 2e-2 + 0.1 * qfit_o, ("prefill fit q", qfit_g, qfit_o)
    # continue the oracle from the GPU's factors
    A_Q_full = torch.zeros((b, hq, l, r), dtype=dtype)
    A_Q_full[:, :, -1:] = gA_Qrow
    orc.prefill(Q, K, V, als_result=(A_Q_full, gB_Q, gA_K, gB_K))
    _compare_state(eng, orc, k, "prefill")

    # ---- decode
    stream = synth.DecodeStream(synth.Workload("t", hq, hkv, d, b, dtype, l, r, k, L, max_iter, tol, steps, rho, sigma),
                                Q[:, :, -1:], (WQ, WK, WV), gen)
    n_miss_total = 0
    for step in range(steps):
        q, kk, vv = stream.next()
        Kg, Vg = eng.decode(q.to(DEV), kk.to(DEV), vv.to(DEV))
        oB_Q, oB_K, ohq, ohk = orc.begin_decode(q, kk, vv)
        for name, got, exp in (("q_hat", eng.last_q_hat, ohq), ("k_hat", eng.last_k_hat, ohk),
                               ("B_Q", eng.B_Q, oB_Q), ("B_K", eng.B_K, oB_K)):
            assert _rel(got, exp) < lim, (step, name, _rel(got, exp))
        oK, oV = orc.finish_decode(eng.B_Q.cpu(), eng.B_K.cpu(), eng.last_q_hat.cpu(), eng.last_k_hat.cpu())
        assert Kg.shape == oK.shape, (step, Kg.shape, oK.shape)
        assert torch.equal(Kg.cpu(), oK) and torch.equal(Vg.cpu(), oV), step
        _compare_state(eng, orc, k, f"step {step}")
        if orc.current_len > orc.n:
            assert torch.equal(eng.last_evict.cpu().bool(), orc.last_evict), step
            assert torch.equal(eng.last_miss_count.cpu().long(), orc.last_evict.sum(-1)), step
            n_miss_total += int(orc.last_evict.sum())
            if eng.last_attn is not None:
                exp = oracle.attention(q, oK, oV)
                assert _rel(eng.last_attn, exp) < (8e-3 if dtype == torch.bfloat16 else 1e-4), step
    return eng, orc, n_miss_total


def _compare_state(eng, orc, k, where):
    assert eng.current_len == orc.current_len and eng.lite_len == orc.lite_len, where
    assert eng.lite_indices == orc.lite_indices, where
    assert len(eng.KVcpu) == len(orc.KVcpu), where
    torch.cuda.synchronize()
    assert torch.equal(eng.KVcpu.tensor(), orc.KVcpu.tensor()), where
    assert torch.equal(eng.hit_indices.cpu(), orc.hit_indices), where
    assert torch.equal(eng.A_K.cpu(), orc.A_K), where
    # the zero tail the next step will read (Q2)
    assert eng._A_K.data[:, :, eng.current_len:].abs().sum() == 0, where
    n_res = orc.Kgpu.shape[2]
    assert torch.equal(eng.Kgpu.cpu(), orc.Kgpu) and torch.equal(eng.Vgpu.cpu(), orc.Vgpu), where
    li = [t for t in orc.lite_indices if t >= 0]
    got = eng._active_idx[:, :, k:k + len(orc.lite_indices)].cpu()
    for s, t in enumerate(orc.lite_indices):
        if t >= 0:
            assert (got[:, :, s] == t).all(), where


def test_tiny_fp32_trace(lrqk, oracle):
    _say("tiny fp32 trace")
    _, _, n = _lockstep(lrqk, oracle, b=2, hq=4, hkv=2, d=16, l=40, r=4, k=8, L=4, steps=40, dtype=torch.float32,
                        max_iter=(2, 2), tol=(1e-8, 1e-8), rho=4, capacity=16)
    assert n > 0  # the trace exercises evictions


def test_tiny_bf16_trace(lrqk, oracle):
    _say("tiny bf16 trace")
    _lockstep(lrqk, oracle, b=1, hq=4, hkv=1, d=16, l=50, r=8, k=16, L=4, steps=24, dtype=torch.bfloat16,
              max_iter=(2, 2), tol=(1e-8, 1e-8), rho=8, capacity=32, fp_tol=2e-2)


def test_buffer_growth_during_decode(lrqk, oracle):
    """capacity 16 with a 40-token prompt: both the factor buffer and the pinned store are
    reallocated during the run and must keep their contents and zero tails."""
    _say("growth trace")
    eng, orc, _ = _lockstep(lrqk, oracle, b=1, hq=2, hkv=2, d=8, l=20, r=3, k=6, L=3, steps=60, dtype=torch.float32,
                            max_iter=(1, 1), tol=(1e-2, 1e-2), rho=3, capacity=8)
    assert eng._A_K.capacity == orc._A_K.capacity and eng.KVcpu.capacity == orc.KVcpu.capacity
    assert eng._A_K.capacity > 30


def test_growth_with_score_index_and_victim_cache(lrqk, oracle):
    """r 16 with a small capacity: the factor buffer is reallocated twice while decoding, so the
    8-bit score index is rebuilt from the new buffer and the victim cache's position table is
    re-sized; the trace must stay in lock step with the oracle throughout."""
    _say("growth trace, score index on")
    eng, orc, n = _lockstep(lrqk, oracle, b=1, hq=4, hkv=2, d=32, l=300, r=16, k=64, L=8, steps=400,
                            dtype=torch.bfloat16, max_iter=(2, 2), tol=(1e-2, 1e-2), rho=24, capacity=64, fp_tol=3e-2,
                            compare_factors=False)
    assert n > 0 and eng._A_K.capacity == orc._A_K.capacity and eng._A_K.capacity >= 675   # 450 -> 675 (-> 1012)


def test_edge_branch_then_main(lrqk, oracle):
    """k <= l <= k+L at prefill: the growing-prefix branch, then the switch to selection."""
    _say("edge trace")
    _lockstep(lrqk, oracle, b=1, hq=4, hkv=2, d=8, l=8, r=3, k=7, L=3, steps=12, dtype=torch.float32,
              max_iter=(2, 2), tol=(1e-8, 1e-8), rho=3, capacity=8)


def test_staged_fetch_trace(lrqk, oracle):
    """The same lock-step trace with the misses moved by host gather + hipMemcpyAsync on the side
    stream (buffer growth included: the pinned store is reallocated during the run)."""
    _say("staged fetch trace")

    class Staged(lrqk.LightAttentionIndicesFactory):
        def __init__(self, *a, **kw):
            super().__init__(*a, **kw)
            self.fetch_mode = "staged"

    _, _, n = _lockstep(lrqk, oracle, b=2, hq=4, hkv=2, d=16, l=40, r=4, k=8, L=4, steps=40, dtype=torch.float32,
                        max_iter=(2, 2), tol=(1e-8, 1e-8), rho=4, capacity=16, cls=Staged)
    assert n > 0


def test_victim_cache_is_invisible(lrqk):
    """The device-side cache of evicted rows only changes where a missed row comes from: two engines on
    the same stream, one with the cache and one without, must hold bit-identical K/V slots, ids and
    attention outputs after every step -- while a good part of the misses is served from the cache."""
    _say("victim cache on/off")
    from lrqk_amd import synth
    wl = synth.Workload("v", 8, 2, 64, 1, torch.bfloat16, 3000, 16, 256, 16, (2, 2), (1e-2, 1e-2), 48, rho=16)
    dev = torch.device(DEV)
    Q, K, V, bases, gen = synth.prompt_qkv(wl, 5, 3000, device=dev)
    A0 = synth.init_factors(wl, 3000, 6, device=dev)
    engs = []
    for rows in (0, 96):
        e = lrqk.LightAttentionIndicesFactory(num_lite_tokens=16, attn_topk=256, num_key_value_groups=4, r=16,
                                              max_iter=(2, 2), tol=(1e-2, 1e-2), capacity=1024)
        e.victim_rows = rows
        e.init_factors = (A0[0].clone(), A0[1].clone())
        e.attn_in_step = True
        e.prefill(Q, K, V)
        engs.append(e)
    stream = synth.DecodeStream(wl, Q[:, :, -1:], bases, gen)
    missed = 0
    engs[1].ws.victim_stats(reset=True)
    for step in range(48):
        q, k, v = [t.contiguous() for t in stream.next()]
        for e in engs:
            e.decode(q, k, v)
        a, b = engs
        assert torch.equal(a._active_idx, b._active_idx), step
        assert torch.equal(a.Kgpu, b.Kgpu) and torch.equal(a.Vgpu, b.Vgpu), step
        assert torch.equal(a.last_attn, b.last_attn), step
        assert torch.equal(a.B_Q, b.B_Q) and torch.equal(a.last_evict, b.last_evict), step
        missed += int(b.last_miss_count.sum())
    host = engs[1].ws.victim_stats()
    _say("missed rows", missed, "over the host link", host)
    assert missed > 0 and 0 < host < 0.9 * missed


def test_score_index_is_invisible(lrqk):
    """The 8-bit score index only prefilters the scan: engines with and without it, on the same
    stream, must select the same tokens and produce the same bits after every step, also once
    rows appended during decoding (indexed by the finish stage) are among the selected ones."""
    _say("score index on/off")
    from lrqk_amd import synth
    wl = synth.Workload("s", 8, 2, 64, 1, torch.bfloat16, 3000, 32, 256, 8, (2, 2), (1e-2, 1e-2), 96, rho=16)
    dev = torch.device(DEV)
    Q, K, V, bases, gen = synth.prompt_qkv(wl, 7, 3000, device=dev)
    A0 = synth.init_factors(wl, 3000, 8, device=dev)
    engs = []
    for on in (False, True):
        e = lrqk.LightAttentionIndicesFactory(num_lite_tokens=8, attn_topk=256, num_key_value_groups=4, r=32,
                                              max_iter=(2, 2), tol=(1e-2, 1e-2), capacity=1024)
        e.use_score_index = on
        e.init_factors = (A0[0].clone(), A0[1].clone())
        e.attn_in_step = True
        e.prefill(Q, K, V)
        engs.append(e)
    stream = synth.DecodeStream(wl, Q[:, :, -1:], bases, gen)
    late = 0
    for step in range(96):
        q, k, v = [t.contiguous() for t in stream.next()]
        for e in engs:
            e.decode(q, k, v)
        a, b = engs
        assert torch.equal(a._active_idx, b._active_idx), step
        assert torch.equal(a.last_evict, b.last_evict) and torch.equal(a.last_miss_count, b.last_miss_count), step
        assert torch.equal(a.Kgpu, b.Kgpu) and torch.equal(a.Vgpu, b.Vgpu), step
        assert torch.equal(a.last_attn, b.last_attn) and torch.equal(a.A_K, b.A_K), step
        late += int((b._active_idx[:, :, :256] >= 3000).sum())
    assert late > 0      # tokens appended during decoding were selected


def test_no_hit_miss_variant(lrqk, oracle):
    _say("no hit/miss trace")
    _lockstep(lrqk, oracle, b=1, hq=4, hkv=2, d=16, l=40, r=4, k=8, L=4, steps=12, dtype=torch.float32,
              max_iter=(2, 2), tol=(1e-8, 1e-8), rho=4, cls=lrqk.LightAttentionIndicesNoHitMiss, no_hit_miss=True)


def test_offload_prefill_variant(lrqk, oracle):
    _say("offload trace")
    _lockstep(lrqk, oracle, b=1, hq=4, hkv=2, d=16, l=40, r=4, k=8, L=4, steps=8, dtype=torch.float32,
              max_iter=(2, 2), tol=(1e-8, 1e-8), rho=4, cls=_OffloadProbe(lrqk))


def _OffloadProbe(lrqk):
    class Probe(lrqk.LightAttentionIndicesOffloadPrefill):
        """_compare_state reads GPU buffers right after prefill; restore them first."""

        def prefill(self, q, k, v):
            super().prefill(q, k, v)
            assert self.Kgpu is None and self._A_K.data is None      # parked
            self._restore(q.device)
    return Probe


def test_overridden_stage_is_used(lrqk, oracle):
    """A subclass replacing only_indices_in_cpu (the hit-rate hook of the reference's
    wikitext_hitrate.py:36-51) sees every call and the results stay identical."""
    _say("override trace")
    calls = []

    class Counting(lrqk.LightAttentionIndicesFactory):
        def only_indices_in_cpu(self, now_indices, new_indices):
            upd, mask = super().only_indices_in_cpu(now_indices, new_indices)
            calls.append(float(mask.sum()) / mask.numel())
            return upd, mask

    _lockstep(lrqk, oracle, b=1, hq=4, hkv=2, d=16, l=40, r=4, k=8, L=4, steps=10, dtype=torch.float32,
              max_iter=(2, 2), tol=(1e-8, 1e-8), rho=4, cls=Counting)
    assert len(calls) == 10 and all(0.0 <= c <= 1.0 for c in calls)


def test_qwen_shape_fp32_short(lrqk, oracle):
    """The CPU-runnable configuration (28 q / 4 kv heads, d 128, r 16, k 512, L 32, fp32,
    max_iter (1,1)) at a reduced context so the oracle finishes in seconds."""
    _say("qwen shape trace")
    _, _, n = _lockstep(lrqk, oracle, b=1, hq=28, hkv=4, d=128, l=1536, r=16, k=512, L=32, steps=40,
                        dtype=torch.float32, max_iter=(1, 1), tol=(1e-2, 1e-2), rho=32, capacity=4096, fp_tol=2e-3)
    assert n > 0


def test_llama_shape_bf16_short(lrqk, oracle):
    """Llama-3-8B attention shape (32 q / 8 kv heads, d 128, r 32, k 2048, L 64, bf16) at an
    8K context."""
    _say("llama shape trace")
    _lockstep(lrqk, oracle, b=1, hq=32, hkv=8, d=128, l=8192, r=32, k=2048, L=64, steps=6, dtype=torch.bfloat16,
              max_iter=(2, 2), tol=(1e-2, 1e-2), rho=32, capacity=4096, fp_tol=3e-2, compare_factors=False)


def test_cache_front_door(lrqk, oracle):
    """DynamicLRQKCache: pending -> collecting -> decoding, error behaviour, sequence length."""
    _say("cache front door")
    from lrqk_amd import synth
    gen = torch.Generator().manual_seed(1)
    b, hq, hkv, d, k, L, r = 1, 4, 2, 16, 8, 4, 4
    cache = lrqk.DynamicLRQKCache(r=r, num_active_tokens=k, lite_tokens=L, max_iter=(2, 2), tol=1e-8,
                                  max_sequence_length=32, num_key_value_groups=hq // hkv)
    with pytest.raises(ValueError):
        cache.update(None, None, None, 0)
    with pytest.raises(NotImplementedError):
        cache[0]
    with pytest.raises(NotImplementedError):
        iter(cache)
    assert cache.get_max_cache_shape() is None and len(cache) == 0

    def toks(n):
        return (torch.randn((b, hq, n, d), generator=gen).to(DEV), torch.randn((b, hkv, n, d), generator=gen).to(DEV),
                torch.randn((b, hkv, n, d), generator=gen).to(DEV))

    # layer 0: a 5-token prompt (shorter than k) -> collecting; 2 more -> still collecting; the 8th
    # token fills the buffer (its capacity is k, lrqk_attention.py:1827-1828) -> factorise
    q, kk, vv = toks(5)
    K0, V0 = cache.update(q, kk, vv, 0)
    assert K0 is kk and cache.sequence_state[0] == cache.State.collecting
    q, kk, vv = toks(2)
    K1, V1 = cache.update(q, kk, vv, 0)
    assert K1.shape == (b, hkv, 7, d) and cache.sequence_state[0] == cache.State.collecting
    q, kk, vv = toks(1)
    K2, V2 = cache.update(q, kk, vv, 0)
    assert K2.shape == (b, hkv, 8, d) and cache.sequence_state[0] == cache.State.decoding
    assert cache.get_seq_length(0) == 8 and cache.seen_tokens == 8 and 0 not in cache.temp_buff_cache_qkv
    # 8 tokens with k=8, L=4 -> prefix branch: decode returns a growing prefix
    q, kk, vv = toks(1)
    K3, V3 = cache.update(q, kk, vv, 0)
    assert K3.shape == (b, hq, 9, d) and cache.get_seq_length(0) == 9
    # layer 1: long prompt with a padding mask (multiplied into K,V in place)
    q, kk, vv = toks(30)
    mask = torch.ones((b, 30), device=DEV)
    mask[:, :3] = 0
    K4, V4 = cache.update(q, kk, vv, 1, attention_mask=mask)
    assert K4 is kk and kk[:, :, :3].abs().sum() == 0 and cache.sequence_state[1] == cache.State.decoding
    q, kk, vv = toks(1)
    K5, V5 = cache.update(q, kk, vv, 1)
    assert K5.shape == (b, hq, k + L, d) and len(cache) == 2
    # an overlong piece in collecting state overflows the pre-allocated buffer
    q, kk, vv = toks(5)
    cache.update(q, kk, vv, 2)
    q, kk, vv = toks(9)
    with pytest.raises(ValueError):
        cache.update(q, kk, vv, 2)


def test_cast_functions(lrqk, oracle):
    _say("cast functions")
    g = torch.Generator().manual_seed(2)
    b, H, l, d, r = 1, 4, 64, 16, 4
    Q = torch.randn((b, H, l, d), generator=g)
    K = torch.randn((b, H, l, d), generator=g)
    A0 = torch.randn((b, H, l, r), generator=g)
    out = lrqk.cast_lrqk_prefill(Q.to(DEV), K.to(DEV), r, max_iter=3, tol=0.0, init_factors=(A0, A0.flip(2)))
    A_Q, B_Q, A_K, B_K = out          # a generator, unpacked like the reference's callers do
    ref = oracle.als_prefill_w1(Q.double(), K.double(), A0.double(), A0.flip(2).double(), 3, 0.0)
    assert _rel(A_K @ B_K, ref[2] @ ref[3]) < 1e-3 and _rel(A_Q @ B_Q, ref[0] @ ref[1]) < 1e-3
    for m in ("top", "topcol", lrqk.InitAQAK.randn):
        o = tuple(lrqk.cast_lrqk_prefill(Q.to(DEV), K.to(DEV), r, max_iter=1, tol=0.0, init_method=m))
        assert o[0].shape == (b, H, l, r) and torch.isfinite(o[3]).all()
    with pytest.raises(ValueError):
        tuple(lrqk.cast_lrqk_prefill(Q.to(DEV), K.to(DEV), r, init_method="nope"))
    # decode cast: inputs untouched, outputs match the oracle
    x = dict(B_Q=torch.randn((b, H, r, d), generator=g), A_K=torch.randn((b, H, 20, r), generator=g),
             B_K=torch.randn((b, H, r, d), generator=g), K__=torch.randn((b, H, 20, d), generator=g),
             q=torch.randn((b, H, 1, d), generator=g), k=torch.randn((b, H, 1, d), generator=g))
    dev = {n: t.to(DEV) for n, t in x.items()}
    nB_Q, nB_K, qh, kh = lrqk.cast_lrqk_decode(**dev, max_iter=2, tol=0.0)
    ref = oracle.als_decode_w1(**{n: t.double() for n, t in x.items()}, max_iter=2, tol=0.0)
    assert torch.equal(dev["B_Q"].cpu(), x["B_Q"])
    for got, exp in zip((nB_Q, nB_K, qh, kh), ref):
        assert _rel(got, exp) < 2e-4
