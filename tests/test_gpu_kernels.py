"""Kernel-level parity: every C-ABI entry point against the CPU oracle on the same seeded
inputs.  Integer / index / byte results are compared bit for bit; floating point within
the tolerance written next to each assert."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from lrqk_amd import ops as o
    return o


@pytest.fixture(scope="module")
def ws(ops):
    return ops.Workspace()


def _say(*a):
    print(*a, flush=True)


# ---------------------------------------------------------------- scores

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("r", [3, 8, 16, 32, 64])
def test_proxy_scores_bit_exact(ops, oracle, dtype, r):
    _say("scores", dtype, r)
    g = torch.Generator().manual_seed(100 + r)
    b, H, cap, m = 2, 3, 1100, 1037
    A = torch.randn((b, H, cap, r), generator=g).to(dtype)
    q = torch.randn((b, H, 1, r), generator=g).to(dtype)
    for rnd in (False, True):
        exp = oracle.proxy_scores(A[:, :, :m].contiguous(), q, round_to_storage=rnd)
        got = ops.proxy_scores(A.to(DEV), q.to(DEV), m, round_to_storage=rnd).cpu()
        assert torch.equal(got.view(torch.int32), exp.view(torch.int32))


# ---------------------------------------------------------------- select

def _check_select(ops, ws, oracle, scores, k):
    exp = oracle.topk_sorted(scores, k)[..., 0].to(torch.int32)
    got = ops.select_from_scores(ws, scores.to(DEV), k).cpu()
    assert torch.equal(got, exp)


@pytest.mark.parametrize("m,k", [(9, 8), (100, 8), (1000, 64), (5000, 512), (40000, 2048)])
def test_select_random(ops, ws, oracle, m, k):
    _say("select random", m, k)
    g = torch.Generator().manual_seed(m)
    _check_select(ops, ws, oracle, torch.randn((2, 3, m), generator=g), k)


def test_select_ties(ops, ws, oracle):
    _say("select ties")
    # all equal
    _check_select(ops, ws, oracle, torch.zeros((1, 2, 3000)), 512)
    # two levels
    s = torch.ones((1, 1, 5000))
    s[0, 0, torch.tensor([4999, 2500, 7, 100, 101, 102, 2000, 2001, 1500, 5])] = 2.0
    _check_select(ops, ws, oracle, s, 64)
    # the k-th boundary tie spans several wavefronts and workgroups' worth of indices
    g = torch.Generator().manual_seed(1)
    s = (torch.randn((2, 2, 20000), generator=g) * 2).round() / 2
    _check_select(ops, ws, oracle, s, 2048)
    # bf16-quantised scores (about 2k distinct values)
    s = torch.randn((1, 4, 32768), generator=g).bfloat16().float()
    _check_select(ops, ws, oracle, s, 2048)
    # negatives, zeros of both signs
    s = torch.randn((1, 2, 4096), generator=g)
    s[:, :, ::3] = 0.0
    s[:, :, 1::3] = -0.0
    _check_select(ops, ws, oracle, s, 2000)
    _check_select(ops, ws, oracle, -torch.rand((1, 2, 4096), generator=g), 100)


def test_select_short_range_is_arange(ops, ws):
    _say("select short")
    for m in (1, 5, 8):
        got = ops.select_from_scores(ws, torch.randn((2, 2, m), device=DEV), 8).cpu()
        assert torch.equal(got, torch.arange(m, dtype=torch.int32).expand(2, 2, m))


@pytest.mark.parametrize("dtype,r", [(torch.bfloat16, 32), (torch.float32, 16)])
def test_score_select_full_size(ops, ws, oracle, dtype, r):
    """128K cached tokens, k = 2048: the fused scan + select against the oracle's full sort."""
    _say("score_select full", dtype, r)
    g = torch.Generator().manual_seed(7)
    b, H, m, cap = 1, 4, 131072 - 65, 131072
    A = torch.randn((b, H, cap, r), generator=g).to(dtype)
    q = torch.randn((b, H, 1, r), generator=g).to(dtype)
    for rnd in (True, False):
        exp = oracle.compute_hit_indices(q, A[:, :, :m].contiguous(), 2048, rnd)[..., 0].to(torch.int32)
        got = ops.score_select(ws, A.to(DEV), q.to(DEV), m, 2048, rnd).cpu()
        assert torch.equal(got, exp)
        # size-independent properties
        assert torch.all(got[..., 1:] > got[..., :-1]) and int(got.max()) < m


@pytest.mark.parametrize("H,m", [(4, 131072 - 65), (32, 270000)])
def test_score_select_full_size_with_score_index(ops, oracle, H, m):
    """The default scan of the decode step (8-bit score index, bf16, r 32, k 2048) at the full 128K range,
    and beyond it at the width of the Llama shape (32 heads x 270K rows: each workgroup of the scan walks
    more than its usual two tiles).  First call: no threshold carried yet, every head rescans; later calls
    with a drifting query: the prefiltered list.  Bit-exact against the oracle's full sort each time."""
    _say("score_select full size with score index", H, m)
    from lrqk_amd import synth
    ws = ops.Workspace()
    ws.score_index(True)
    g = torch.Generator().manual_seed(70 + H)
    r, k, cap = 32, 2048, m + 64
    A = (torch.randn((1, H, cap, r), generator=g) * 0.7).bfloat16()
    q = torch.randn((1, H, 1, r), generator=g)
    Ad = A.to(DEV)
    oracle.set_threads(16)
    try:
        for step in range(3):
            qb = q.bfloat16()
            exp = oracle.compute_hit_indices(qb, A[:, :, :m + step], k, True)[..., 0].to(torch.int32)
            got = ops.score_select(ws, Ad, qb.to(DEV), m + step, k, True).cpu()
            assert torch.equal(got, exp), step
            q = synth.rotate_query(g, q, 0.05)
    finally:
        oracle.set_threads(1)
    fast, full = ws.select_stats()
    _say("heads from the prefiltered list / rescanned:", fast, full)
    assert full >= H and fast >= H, (fast, full)


def test_score_select_filtered_path(ops, oracle):
    """Repeated calls on one workspace with a slowly drifting query: after the first call the
    heads are served from the candidate list of the streaming filter; every result must
    still equal the oracle's full sort, bit for bit."""
    _say("score_select filtered path")
    from lrqk_amd import synth
    ws = ops.Workspace()
    g = torch.Generator().manual_seed(11)
    b, H, m, cap, r, k = 1, 6, 30000, 30016, 32, 2048
    A = (torch.randn((b, H, cap, r), generator=g) * 0.5).bfloat16()
    q = torch.randn((b, H, 1, r), generator=g)
    Ad = A.to(DEV)
    ws.select_stats()
    for step in range(6):
        qb = q.bfloat16()
        exp = oracle.compute_hit_indices(qb, A[:, :, :m + step].contiguous(), k, True)[..., 0].to(torch.int32)
        got = ops.score_select(ws, Ad, qb.to(DEV), m + step, k, True).cpu()
        assert torch.equal(got, exp), step
        q = synth.rotate_query(g, q, 0.05)
    fast, full = ws.select_stats()
    assert full >= H and fast >= 4 * H, (fast, full)       # first call rescans, later calls do not
    # a jump of the score distribution must fall back, not fail: scale the query by 100 and by 0.01
    for scale in (100.0, 0.01, -1.0):
        qb = (q * scale).bfloat16()
        exp = oracle.compute_hit_indices(qb, A[:, :, :m].contiguous(), k, True)[..., 0].to(torch.int32)
        got = ops.score_select(ws, Ad, qb.to(DEV), m, k, True).cpu()
        assert torch.equal(got, exp), scale


def test_score_select_filtered_path_ties(ops, oracle):
    """Scores crafted through a one-hot query: heavy ties at the threshold on the filtered path."""
    _say("score_select filtered ties")
    ws = ops.Workspace()
    g = torch.Generator().manual_seed(12)
    b, H, m, r, k = 1, 3, 20000, 8, 512
    A = torch.zeros((b, H, m, r))
    A[..., 0] = (torch.randn((b, H, m), generator=g) * 2).round() / 2    # about 20 distinct score values
    A[..., 1:] = torch.randn((b, H, m, r - 1), generator=g)              # ignored by the query
    q = torch.zeros((b, H, 1, r))
    q[..., 0] = 1.0
    exp = oracle.compute_hit_indices(q, A, k, False)[..., 0].to(torch.int32)
    for _ in range(3):
        got = ops.score_select(ws, A.to(DEV), q.to(DEV), m, k, False).cpu()
        assert torch.equal(got, exp)
    fast, full = ws.select_stats()
    assert fast >= H, (fast, full)
    # all scores equal: the candidate list overflows every time and the rescan path answers
    A[..., 0] = 1.0
    got = ops.score_select(ws, A.to(DEV), q.to(DEV), m, k, False).cpu()
    assert torch.equal(got, torch.arange(k, dtype=torch.int32).expand(b, H, k))


@pytest.mark.parametrize("dtype,r", [(torch.bfloat16, 32), (torch.float32, 32), (torch.bfloat16, 16),
                                     (torch.bfloat16, 64), (torch.float32, 64)])
def test_score_select_with_score_index(ops, oracle, dtype, r):
    """The 8-bit score index only prefilters: with it the selection must equal the oracle's
    full sort bit for bit, also on rows chosen to stress its bound -- heads whose rows are
    almost rank one with the query across the dominant direction, columns of very different
    size, zero rows, a head of all zeros, duplicated columns, a dynamic range of 2^40, scores
    tied at the threshold -- while the query drifts, jumps and the number of rows grows."""
    _say("score_select with score index", dtype, r)
    from lrqk_amd import synth
    ws = ops.Workspace()
    ws.score_index(True)
    g = torch.Generator().manual_seed(21 + r)
    b, H, m, cap, k = 1, 8, 24000, 24064, 1024
    A = torch.randn((b, H, cap, r), generator=g)
    u = torch.randn((r,), generator=g)
    u /= u.norm()
    A[0, 1] = torch.randn((cap, 1), generator=g) * 30.0 * u + 0.05 * torch.randn((cap, r), generator=g)  # rank one + noise
    A[0, 2] *= torch.logspace(-3, 3, r)                                   # columns of very different size
    A[0, 3, ::3] = 0.0                                                    # zero rows
    A[0, 4] = 0.0                                                         # nothing at all
    A[0, 5, :, 1] = A[0, 5, :, 0]                                         # duplicated column
    A[0, 6] *= torch.exp2(torch.randint(-20, 21, (cap, 1), generator=g).float())   # row sizes over 2^40
    A[0, 7] = (A[0, 7] * 2).round() / 2                                   # few distinct values: ties
    A = A.to(dtype)
    q = torch.randn((b, H, 1, r), generator=g)
    q[0, 1, 0] -= (q[0, 1, 0] @ u) * u * 0.999                            # across the dominant direction
    q[0, 7, 0] = 0.0
    q[0, 7, 0, :2] = 1.0
    Ad = A.to(DEV)
    rnd = dtype == torch.bfloat16
    for step in range(5):
        qd = q.to(dtype)
        exp = oracle.compute_hit_indices(qd, A[:, :, :m + 7 * step].contiguous(), k, rnd)[..., 0].to(torch.int32)
        got = ops.score_select(ws, Ad, qd.to(DEV), m + 7 * step, k, rnd).cpu()
        assert torch.equal(got, exp), step
        q = synth.rotate_query(g, q, 0.05)
    fast, full = ws.select_stats()
    assert fast >= 12, (fast, full)         # later calls are served from the prefiltered list (heads 4 and 7 tie too much)
    for scale in (50.0, 0.02, -1.0):
        qd = (q * scale).to(dtype)
        exp = oracle.compute_hit_indices(qd, A[:, :, :m].contiguous(), k, rnd)[..., 0].to(torch.int32)
        got = ops.score_select(ws, Ad, qd.to(DEV), m, k, rnd).cpu()
        assert torch.equal(got, exp), scale
    # switching the index off and on again drops and rebuilds it
    ws.score_index(False)
    qd = q.to(dtype)
    exp = oracle.compute_hit_indices(qd, A[:, :, :m].contiguous(), k, rnd)[..., 0].to(torch.int32)
    assert torch.equal(ops.score_select(ws, Ad, qd.to(DEV), m, k, rnd).cpu(), exp)
    ws.score_index(True)
    assert torch.equal(ops.score_select(ws, Ad, qd.to(DEV), m, k, rnd).cpu(), exp)


def test_score_select_index_many_tiles_per_workgroup(ops, oracle):
    """Many heads and a long range: the scan launches only as many workgroups as the GPU holds, so each one
    walks ten tiles, and with k = 4096 it collects more rows than its list holds and rescores them in
    between.  Bit-exact against the oracle on the first call (rescan) and on the filtered calls."""
    _say("score_select with score index, many tiles per workgroup")
    from lrqk_amd import synth
    ws = ops.Workspace()
    ws.score_index(True)
    g = torch.Generator().manual_seed(77)
    b, H, m, r, k = 1, 512, 40000, 16, 4096
    A = (torch.randn((b, H, m, r), generator=g) * 0.5).bfloat16()
    q = torch.randn((b, H, 1, r), generator=g)
    Ad = A.to(DEV)
    ws.select_stats()
    for step in range(3):
        qb = q.bfloat16()
        exp = oracle.compute_hit_indices(qb, A, k, True)[..., 0].to(torch.int32)
        got = ops.score_select(ws, Ad, qb.to(DEV), m, k, True).cpu()
        assert torch.equal(got, exp), step
        q = synth.rotate_query(g, q, 0.03)
    fast, full = ws.select_stats()
    assert fast >= H, (fast, full)      # the later calls went through the filtered list


# ---------------------------------------------------------------- diff

def _check_diff(ops, oracle, now, new):
    b, H, k = now.shape
    upd, mask = oracle.only_indices_in_cpu(now.view(b, H, k, 1).long(), new.view(b, H, k, 1).long())
    hit = now.to(torch.int32).to(DEV).contiguous()
    ev, slots, cnt = ops.diff(new.to(torch.int32).to(DEV).contiguous(), hit)
    assert torch.equal(hit.cpu().long(), upd[..., 0])
    assert torch.equal(ev.cpu().bool(), mask)
    assert torch.equal(cnt.cpu().long(), mask.sum(-1))
    for i in range(b):
        for h in range(H):
            c = int(cnt[i, h])
            assert torch.equal(slots[i, h, :c].cpu().long(), mask[i, h].nonzero()[:, 0])


@pytest.mark.parametrize("m,cap,k,H,dtype", [(5000, 5008, 512, 3, torch.float32), (40000, 40000, 2048, 2, torch.bfloat16),
                                             (300000, 300032, 2048, 2, torch.bfloat16),
                                             (270000, 270000, 4096, 1, torch.bfloat16),
                                             (20000, 20000, 4100, 1, torch.float32),
                                             (2048, 2056, 2048, 2, torch.bfloat16), (7, 16, 7, 3, torch.float32)])
def test_score_select_diff_fused(ops, oracle, m, cap, k, H, dtype):
    """Selection and hit/miss diff in one pass against the oracle's two stages: one bitmap chunk
    (m <= 262144), several chunks, the largest fused k, a k beyond it (separate diff launch), and m == k (the first
    step after the growing-prefix branch: every row is selected).
    Second round on the same workspace goes through the filtered path."""
    _say("score_select_diff", m, k, H, dtype)
    ws = ops.Workspace()
    g = torch.Generator().manual_seed(m + k)
    r = 16
    A = torch.randn((1, H, cap, r), generator=g).to(dtype)
    q = torch.randn((1, H, 1, r), generator=g).to(dtype)
    # resident set: random unique tokens below m, in random order
    hit = torch.stack([torch.randperm(m, generator=g)[:k] for _ in range(H)]).view(1, H, k).to(torch.int32)
    Ad = A.to(DEV)
    hit_d = hit.to(DEV).contiguous()
    now = hit.long().unsqueeze(-1)
    for rnd in range(2):
        exp_new = oracle.compute_hit_indices(q, A[:, :, :m].contiguous(), k, True)
        exp_upd, exp_ev = oracle.only_indices_in_cpu(now, exp_new)
        new, evict, slots, count = ops.score_select_diff(ws, Ad, q.to(DEV), m, k, hit_d)
        assert torch.equal(new.cpu().long(), exp_new[..., 0]), rnd
        assert torch.equal(hit_d.cpu().long(), exp_upd[..., 0]), rnd
        assert torch.equal(evict.cpu().bool(), exp_ev), rnd
        assert torch.equal(count.cpu().long(), exp_ev.sum(-1)), rnd
        for h in range(H):
            c = int(count[0, h])
            assert slots[0, h, :c].cpu().tolist() == exp_ev[0, h].nonzero().view(-1).tolist()
        now = exp_upd
        q = (q.float() + 0.05 * torch.randn(q.shape, generator=g)).to(dtype)


@pytest.mark.parametrize("m,k,H,dtype,r,index,ties", [(40000, 512, 3, torch.bfloat16, 16, False, False),
                                                       (131500, 2048, 4, torch.bfloat16, 32, True, False),
                                                       (131500, 2048, 2, torch.bfloat16, 32, True, True),
                                                       (262144, 2048, 2, torch.bfloat16, 16, True, False),
                                                       (131500, 2048, 2, torch.bfloat16, 32, False, False),
                                                       (30000, 4096, 2, torch.float32, 16, True, False),
                                                       (90000, 8192, 1, torch.bfloat16, 32, True, False),
                                                       (9000, 1024, 2, torch.float32, 8, False, True)])
def test_score_select_diff_unordered(ops, oracle, m, k, H, dtype, r, index, ties):
    """The decode step's form of the fused select + diff (no ascending list; lrqk_score_select_diff with
    new_idx = NULL) against the oracle's two stages, over several rounds on one workspace (the first has no
    carried bound and rescans; later ones take the candidate list, also a list of more than 8192 entries
    when the query shrinks).  `ties`: scores take a handful of values, so the threshold cuts through a large
    class of equal scores and the lowest token ids of that class must win."""
    _say("score_select_diff unordered", m, k, H, dtype, r, index, ties)
    ws = ops.Workspace()
    ws.score_index(index)
    g = torch.Generator().manual_seed(m + k + r)
    if ties:
        A = torch.zeros((1, H, m, r))
        A[..., 0] = torch.randint(0, 40 if m > 100000 else 5, (1, H, m), generator=g).float()
        q = torch.zeros((1, H, 1, r))
        q[..., 0] = 1.0
        A, q = A.to(dtype), q.to(dtype)
    else:
        A = torch.randn((1, H, m, r), generator=g).to(dtype)
        q = torch.randn((1, H, 1, r), generator=g).to(dtype)
    hit = torch.stack([torch.randperm(m, generator=g)[:k] for _ in range(H)]).view(1, H, k).to(torch.int32)
    Ad = A.to(DEV)
    hit_d = hit.to(DEV).contiguous()
    now = hit.long().unsqueeze(-1)
    turn = not index and m > 100000
    if turn:
        # rows three times as long along the first coordinate: a query of the same length that turns towards it
        # spreads the scores 1.5 times as wide, and the plain scan's bound (which follows |q| only) lets ~10 k
        # rows through -- a list beyond the 8192 entries of the usual register budget
        A[..., 0] *= 3.0
        q[..., 0] = 0.0
        q = q / q.float().norm(dim=-1, keepdim=True)
        Ad = A.to(DEV)
    scales = [1.0, 1.0, 1.0, 0.45, 1.0, 2.5, 1.0]
    for rnd, sc in enumerate(scales):
        if turn and rnd in (3, 5):
            qf = q.float()
            qf[..., 0] = 0.4 if rnd == 3 else 0.0
            q = (qf / qf.norm(dim=-1, keepdim=True)).to(dtype)
        elif not ties:
            q = ((q.float() + 0.05 * torch.randn(q.shape, generator=g)) * sc).to(dtype)
        exp_new = oracle.compute_hit_indices(q, A, k, True)
        exp_upd, exp_ev = oracle.only_indices_in_cpu(now, exp_new)
        new, evict, slots, count = ops.score_select_diff(ws, Ad, q.to(DEV), m, k, hit_d, want_new=False)
        assert new is None
        assert torch.equal(hit_d.cpu().long(), exp_upd[..., 0]), rnd
        assert torch.equal(evict.cpu().bool(), exp_ev), rnd
        assert torch.equal(count.cpu().long(), exp_ev.sum(-1)), rnd
        for h in range(H):
            c = int(count[0, h])
            assert slots[0, h, :c].cpu().tolist() == exp_ev[0, h].nonzero().view(-1).tolist()
        now = exp_upd
    fast, full = ws.select_stats()
    _say("   heads served from the list:", fast, "rescanned:", full)
    assert fast > 0


def test_score_select_many_chunks(ops, ws, oracle):
    """More candidates than one bitmap chunk covers (262144): the ordered output runs chunk by chunk."""
    _say("score_select many chunks")
    g = torch.Generator().manual_seed(5)
    m, cap, r, k = 600000, 600000, 8, 2048
    A = torch.randn((1, 2, cap, r), generator=g).bfloat16()
    q = torch.randn((1, 2, 1, r), generator=g).bfloat16()
    exp = oracle.compute_hit_indices(q, A, k, True)[..., 0].to(torch.int32)
    for _ in range(2):   # second call: filtered path
        got = ops.score_select(ws, A.to(DEV), q.to(DEV), m, k, True).cpu()
        assert torch.equal(got, exp)


def test_diff_docstring_vector(ops, oracle):
    _say("diff docstring")
    now = torch.tensor([0, 1, 2, 6, 7]).view(1, 1, 5)
    new = torch.tensor([0, 2, 4, 5, 6]).view(1, 1, 5)
    _check_diff(ops, oracle, now, new)
    hit = now.to(torch.int32).to(DEV)
    ev, _, _ = ops.diff(new.to(torch.int32).to(DEV), hit)
    assert hit.view(-1).tolist() == [0, 4, 2, 6, 5] and ev.view(-1).tolist() == [0, 1, 0, 0, 1]


@pytest.mark.parametrize("k,seq", [(8, 32), (512, 4096), (2048, 40000), (2500, 5000), (8192, 60000)])
def test_diff_random(ops, oracle, k, seq):
    _say("diff random", k, seq)
    g = torch.Generator().manual_seed(k)
    b, H = 2, 4
    now = torch.stack([torch.randperm(seq, generator=g)[:k] for _ in range(b * H)]).view(b, H, k)
    # overlap heavy: new shares most entries with now
    new = now.clone()
    for i in range(b * H):
        row = new.view(b * H, k)[i]
        pool = torch.tensor(sorted(set(range(seq)) - set(row.tolist())))
        nrep = min(k // 5 + 1, pool.numel())
        pos = torch.randperm(k, generator=g)[:nrep]
        row[pos] = pool[torch.randperm(pool.numel(), generator=g)[:nrep]]
    new = new.sort(-1).values
    _check_diff(ops, oracle, now, new)


def test_diff_identical_and_disjoint(ops, oracle):
    _say("diff identical/disjoint")
    a = torch.arange(64).view(1, 1, 64)
    _check_diff(ops, oracle, a, a.clone())
    _check_diff(ops, oracle, a, a + 64)
    _check_diff(ops, oracle, a.flip(-1).contiguous(), a + 10)


def test_replace_all(ops):
    new = torch.arange(16, dtype=torch.int32, device=DEV).view(1, 2, 8)
    hit = torch.zeros((1, 2, 8), dtype=torch.int32, device=DEV)
    ev, slots, cnt = ops.diff(new, hit, replace_all=True)
    assert torch.equal(hit, new) and ev.all() and cnt.tolist() == [[8, 8]]
    assert torch.equal(slots.cpu(), torch.arange(8, dtype=torch.int32).expand(1, 2, 8))


# ---------------------------------------------------------------- row movers

@pytest.mark.parametrize("dtype,d", [(torch.bfloat16, 128), (torch.float32, 128), (torch.float32, 8),
                                     (torch.bfloat16, 64), (torch.bfloat16, 256)])
@pytest.mark.parametrize("pinned", [True, False])
def test_fetch_rows(ops, oracle, dtype, d, pinned):
    _say("fetch", dtype, d, pinned)
    g = torch.Generator().manual_seed(d)
    b, hq, hkv, cap, k, L = 2, 4, 2, 300, 16, 4
    grp = hq // hkv
    store = torch.randn((b, hkv, cap, 2 * d), generator=g).to(dtype)
    store_dev = store.pin_memory() if pinned else store.to(DEV)
    Kg = torch.randn((b, hq, k + L, d), generator=g).to(dtype)
    Vg = torch.randn((b, hq, k + L, d), generator=g).to(dtype)
    now = torch.stack([torch.randperm(200, generator=g)[:k] for _ in range(b * hq)]).view(b, hq, k)
    new = torch.stack([torch.randperm(200, generator=g)[:k].sort().values for _ in range(b * hq)]).view(b, hq, k)
    upd, mask = oracle.only_indices_in_cpu(now.view(b, hq, k, 1), new.view(b, hq, k, 1))
    rows = oracle.take_along_dim_with_mask(store, upd.view(b, hkv, grp, k), mask.view(b, hkv, grp, k))
    expK, expV = Kg.clone(), Vg.clone()
    expK[:, :, :k][mask] = rows[:, :d]
    expV[:, :, :k][mask] = rows[:, d:]
    hit = torch.zeros((b, hq, k + L), dtype=torch.int32)
    hit[:, :, :k] = now
    hit = hit.to(DEV)
    Kd, Vd = Kg.to(DEV), Vg.to(DEV)
    ev, slots, cnt = ops.diff(new.to(torch.int32).to(DEV), hit, k=k)
    ops.fetch_rows(store_dev, Kd, Vd, hit, slots, cnt, k)
    torch.cuda.synchronize()
    assert torch.equal(Kd.cpu(), expK) and torch.equal(Vd.cpu(), expV)
    assert torch.equal(hit[:, :, :k].cpu().long(), upd[..., 0])
    if pinned:
        # the staged path (host gather + hipMemcpyAsync on the side stream + scatter): same bytes, twice
        # in a row on one workspace (the second call reuses the staging block)
        ws = ops.Workspace()
        for _ in range(2):
            Kd2, Vd2 = Kg.to(DEV), Vg.to(DEV)
            ops.fetch_rows_staged(ws, store_dev, Kd2, Vd2, hit, slots, cnt, k)
            torch.cuda.synchronize()
            assert torch.equal(Kd2.cpu(), expK) and torch.equal(Vd2.cpu(), expV)
    else:
        with pytest.raises(ValueError):
            ops.fetch_rows_staged(ops.Workspace(), store_dev, Kd, Vd, hit, slots, cnt, k)


def test_gather_append_flush(ops, oracle):
    _say("gather/append/flush")
    g = torch.Generator().manual_seed(3)
    b, hq, hkv, l, d, k, L = 2, 4, 2, 50, 16, 8, 4
    grp = hq // hkv
    for dtype in (torch.float32, torch.bfloat16):
        src = torch.randn((b, hkv, l, d), generator=g).to(dtype)
        idx = torch.stack([torch.randperm(l, generator=g)[:k].sort().values for _ in range(b * hq)]).view(b, hq, k)
        dst = torch.zeros((b, hq, k + L, d), dtype=dtype, device=DEV)
        ops.gather_rows(src.to(DEV), idx.to(torch.int32).to(DEV), dst, k)
        exp = torch.take_along_dim(oracle.repeat_kv(src, grp), idx.unsqueeze(-1), 2)
        assert torch.equal(dst[:, :, :k].cpu(), exp) and dst[:, :, k:].abs().sum() == 0
        # append into ring slot 2
        kn = torch.randn((b, hkv, 1, d), generator=g).to(dtype)
        vn = torch.randn((b, hkv, 1, d), generator=g).to(dtype)
        vdst = torch.zeros_like(dst)
        act = torch.full((b, hq, k + L), -1, dtype=torch.int32, device=DEV)
        ops.append_token(kn.to(DEV), vn.to(DEV), dst, vdst, k + 2, act, 77)
        assert torch.equal(dst[:, :, k + 2:k + 3].cpu(), oracle.repeat_kv(kn, grp))
        assert torch.equal(vdst[:, :, k + 2:k + 3].cpu(), oracle.repeat_kv(vn, grp))
        assert (act[:, :, k + 2] == 77).all() and (act[:, :, :k + 2] == -1).all()
        # flush the ring to a pinned store
        store = torch.zeros((b, hkv, 40, 2 * d), dtype=dtype).pin_memory()
        ring = torch.randn((b, hq, L, d), generator=g).to(dtype)
        dst[:, :, k:] = ring.to(DEV)
        vdst[:, :, k:] = (ring * 2).to(DEV)
        ops.flush_ring(dst, vdst, k, L, store, 10, hkv)
        torch.cuda.synchronize()
        assert torch.equal(store[:, :, 10:10 + L, :d], ring[:, ::grp])
        assert torch.equal(store[:, :, 10:10 + L, d:], (ring * 2)[:, ::grp])
        assert store[:, :, :10].abs().sum() == 0 and store[:, :, 10 + L:].abs().sum() == 0


# ---------------------------------------------------------------- attention

@pytest.mark.parametrize("dtype,d,n", [(torch.bfloat16, 128, 2112), (torch.float32, 128, 544), (torch.float32, 16, 12),
                                       (torch.bfloat16, 64, 1), (torch.float32, 8, 100),
                                       # other head widths: 64 (eight lanes per row) and 256 (a row fills half a wave)
                                       (torch.bfloat16, 64, 300), (torch.bfloat16, 256, 500), (torch.float32, 256, 130)])
def test_attention(ops, ws, oracle, dtype, d, n):
    _say("attention", dtype, d, n)
    g = torch.Generator().manual_seed(n)
    b, H = 2, 4
    q = torch.randn((b, H, 1, d), generator=g).to(dtype)
    K = torch.randn((b, H, n + 3, d), generator=g).to(dtype)
    V = torch.randn((b, H, n + 3, d), generator=g).to(dtype)
    exp = oracle.attention(q, K[:, :, :n], V[:, :, :n])
    got = ops.attention(ws, q.to(DEV), K.to(DEV), V.to(DEV), n).cpu().double()
    rel = (got - exp).norm() / exp.norm()
    # fp32 accumulation; bf16 output rounding bounds the bf16 case (2^-9 per element)
    assert rel < (3e-3 if dtype == torch.bfloat16 else 1e-5), rel
    # sharply peaked scores (large logits) must not overflow
    q2 = (q.float() * 30).to(dtype)
    exp = oracle.attention(q2, K[:, :, :n], V[:, :, :n])
    got = ops.attention(ws, q2.to(DEV), K.to(DEV), V.to(DEV), n).cpu().double()
    assert torch.isfinite(got).all() and (got - exp).norm() / exp.norm() < (4e-3 if dtype == torch.bfloat16 else 1e-4)


# ---------------------------------------------------------------- ALS decode

def _als_inputs(g, b, hq, hkv, n, d, r, cap, dtype):
    x = dict(B_Q=torch.randn((b, hq, r, d), generator=g) * 0.5, B_K=torch.randn((b, hq, r, d), generator=g) * 0.5,
             A=torch.randn((b, hq, cap, r), generator=g), Kp=torch.randn((b, hq, n, d), generator=g),
             q=torch.randn((b, hq, 1, d), generator=g), k=torch.randn((b, hkv, 1, d), generator=g))
    return {k_: v.to(dtype) for k_, v in x.items()}


@pytest.mark.parametrize("dtype,hq,hkv,n,d,r", [(torch.float32, 4, 2, 12, 16, 4), (torch.float32, 28, 4, 544, 128, 16),
                                                (torch.bfloat16, 32, 8, 2112, 128, 32), (torch.float32, 2, 2, 70, 8, 3),
                                                # head widths 64 and 256 (bf16 rows that the d = 128 kernel does not take)
                                                (torch.bfloat16, 8, 2, 300, 64, 16), (torch.bfloat16, 4, 1, 272, 256, 32),
                                                (torch.float32, 4, 2, 150, 64, 8),
                                                # ranks beyond 32: 64 and 40 (bf16 rows of 128 elements: 2 x 2 matrix-core
                                                # tiles), 48 in fp32 (the general kernels)
                                                (torch.bfloat16, 8, 2, 600, 128, 64), (torch.float32, 2, 1, 200, 64, 48),
                                                (torch.bfloat16, 4, 4, 333, 128, 40),
                                                # ... an odd one (A_K rows one element at a time), 56, 64 in fp32
                                                (torch.float32, 2, 1, 100, 64, 33), (torch.bfloat16, 2, 2, 150, 128, 56),
                                                (torch.float32, 4, 2, 272, 128, 64)])
@pytest.mark.parametrize("max_iter,tol", [(1, 0.0), (2, 0.0), (3, 1e30), (4, 1e-6)])
def test_als_decode(ops, ws, oracle, dtype, hq, hkv, n, d, r, max_iter, tol):
    _check_als_decode(ops, ws, oracle, dtype, hq, hkv, n, d, r, max_iter, tol)


@pytest.mark.parametrize("n", [1100, 2000, 2700, 3500, 4160, 6000, 8256])
def test_als_decode_split_counts(ops, ws, oracle, n):
    """The Gram sums arrive in ceil(n / 128) partials (at most 32) and the solve kernel is compiled per
    group of four of that count: one case per group not met by the shapes above."""
    _check_als_decode(ops, ws, oracle, torch.float32, 2, 1, n, 64, 16, 2, 0.0)


def _check_als_decode(ops, ws, oracle, dtype, hq, hkv, n, d, r, max_iter, tol):
    _say("als_decode", dtype, hq, n, d, r, max_iter, tol)
    g = torch.Generator().manual_seed(n + r)
    b, cap = 1, 3 * n
    x = _als_inputs(g, b, hq, hkv, n, d, r, cap, dtype)
    idx = torch.stack([torch.randperm(cap - 1, generator=g)[:n] for _ in range(b * hq)]).view(b, hq, n)
    A = x["A"].clone()
    A[:, :, cap - 1] = 0  # the append row starts as zeros
    A_act = torch.take_along_dim(A, idx.unsqueeze(-1), 2)
    repk = oracle.repeat_kv(x["k"], hq // hkv)
    ref = oracle.als_decode_w1(x["B_Q"].double(), A_act.double(), x["B_K"].double(), x["Kp"].double(),
                               x["q"].double(), repk.double(), max_iter, tol)
    bq, bk, ad = x["B_Q"].to(DEV), x["B_K"].to(DEV), A.to(DEV)
    qh, kh = ops.als_decode(ws, bq, bk, ad, idx.to(torch.int32).to(DEV), x["Kp"].to(DEV), n, x["q"].to(DEV),
                            x["k"].to(DEV), max_iter, tol, append_row=cap - 1)
    # fp32 arithmetic against an fp64 reference: 2e-4 relative; bf16 storage adds the output
    # rounding of 2^-9 per element
    lim = 6e-3 if dtype == torch.bfloat16 else 2e-4
    for name, got, exp in (("q_hat", qh, ref[2]), ("k_hat", kh, ref[3]), ("B_Q", bq, ref[0]), ("B_K", bk, ref[1])):
        rel = (got.cpu().double() - exp).norm() / exp.norm()
        assert rel < lim, (name, float(rel))
    assert torch.equal(ad[:, :, cap - 1].cpu(), kh[:, :, 0].cpu())          # appended row
    assert torch.equal(ad[:, :, :cap - 1].cpu(), A[:, :, :cap - 1])         # nothing else touched


def test_als_decode_ill_conditioned(ops, ws, oracle):
    """Factors whose Gram matrices have condition numbers around 1e5 and entries far from 1 (what a real
    stream produces: the r x r inverses run in fp32 without pivoting, on the matrix scaled to unit
    diagonal).  The same bound against fp64 as for well-conditioned factors must hold."""
    _say("als_decode ill-conditioned")
    g = torch.Generator().manual_seed(77)
    b, hq, hkv, n, d, r, cap = 1, 4, 2, 300, 64, 32, 640
    x = _als_inputs(g, b, hq, hkv, n, d, r, cap, torch.float32)
    spec = torch.logspace(0, -2.5, r)                      # singular values over 2.5 decades: cond(G) ~ 1e5
    x["A"] = x["A"] * spec * 40.0                          # and a diagonal far above 1
    x["B_Q"] = x["B_Q"] * spec.unsqueeze(-1) * 25.0
    x["B_K"] = x["B_K"] * spec.unsqueeze(-1) * 25.0
    idx = torch.stack([torch.randperm(cap - 1, generator=g)[:n] for _ in range(b * hq)]).view(b, hq, n)
    A = x["A"].clone()
    A[:, :, cap - 1] = 0
    A_act = torch.take_along_dim(A, idx.unsqueeze(-1), 2)
    G_Q = x["B_Q"].double() @ x["B_Q"].double().transpose(-1, -2) + A_act.double().transpose(-1, -2) @ A_act.double()
    cond = torch.linalg.cond(G_Q).max().item()
    assert 1e3 < cond < 1e7, cond
    repk = oracle.repeat_kv(x["k"], hq // hkv)
    ref = oracle.als_decode_w1(x["B_Q"].double(), A_act.double(), x["B_K"].double(), x["Kp"].double(),
                               x["q"].double(), repk.double(), 2, 0.0)
    bq, bk, ad = x["B_Q"].to(DEV), x["B_K"].to(DEV), A.to(DEV)
    qh, kh = ops.als_decode(ws, bq, bk, ad, idx.to(torch.int32).to(DEV), x["Kp"].to(DEV), n, x["q"].to(DEV),
                            x["k"].to(DEV), 2, 0.0, append_row=cap - 1)
    lim = 2e-4  # as for well-conditioned factors (measured 1e-6 at cond 1.3e5)
    for name, got, exp in (("q_hat", qh, ref[2]), ("k_hat", kh, ref[3])):
        assert torch.isfinite(got).all(), name
        rel = (got.cpu().double() - exp).norm() / exp.norm()
        print(name, "cond %.2e rel %.2e lim %.2e" % (cond, float(rel), lim), flush=True)
        assert rel < lim, (name, float(rel), cond)


def test_als_decode_prefix_branch(ops, ws, oracle):
    """active_idx = NULL: rows 0..n-1 of A_K (the growing-prefix branch)."""
    _say("als_decode prefix")
    g = torch.Generator().manual_seed(5)
    b, hq, hkv, n, d, r, cap = 2, 4, 2, 20, 16, 4, 64
    x = _als_inputs(g, b, hq, hkv, 30, d, r, cap, torch.float32)
    ref = oracle.als_decode_w1(x["B_Q"].double(), x["A"][:, :, :n].double(), x["B_K"].double(),
                               x["Kp"][:, :, :n].double(), x["q"].double(),
                               oracle.repeat_kv(x["k"], 2).double(), 2, 0.0)
    bq, bk, ad = x["B_Q"].to(DEV), x["B_K"].to(DEV), x["A"].to(DEV)
    qh, kh = ops.als_decode(ws, bq, bk, ad, None, x["Kp"].to(DEV), n, x["q"].to(DEV), x["k"].to(DEV), 2, 0.0, n)
    assert (qh.cpu().double() - ref[2]).norm() / ref[2].norm() < 2e-4
    assert (bk.cpu().double() - ref[1]).norm() / ref[1].norm() < 2e-4
    assert torch.equal(ad[:, :, n].cpu(), kh[:, :, 0].cpu())


# ---------------------------------------------------------------- ALS prefill

def test_als_prefill_long_sums(ops, ws, oracle):
    """The Gram sums of a 128K prompt, bf16 input: the first B factors (no iteration: two Gram passes and the
    r x r solves, on well-conditioned random factors) against fp64.  The matrix cores do not round to nearest
    when they accumulate, which biases long sums of squares (2.2e-6 here when a whole split of the long axis
    is summed inside one accumulator); summed tile by tile the result stays below the fp32 pipe's 8.4e-7."""
    _say("als_prefill long sums")
    g = torch.Generator().manual_seed(5)
    b, hq, hkv, l, d, r = 1, 2, 1, 131072, 128, 32
    Q = torch.randn((b, hq, l, d), generator=g).to(torch.bfloat16)
    K = torch.randn((b, hkv, l, d), generator=g).to(torch.bfloat16)
    A_Q0 = torch.randn((b, hq, l, r), generator=g)
    A_K0 = torch.randn((b, hq, l, r), generator=g)
    ref = oracle.als_prefill_w1(Q.double(), oracle.repeat_kv(K, hq // hkv).double(), A_Q0.double(), A_K0.double(), 0, 0.0)
    got = ops.als_prefill(ws, Q.to(DEV), K.to(DEV), A_Q0.to(DEV), A_K0.to(DEV), 0, 0.0)
    for name, x, y in (("B_Q", got[1], ref[1]), ("B_K", got[3], ref[3])):
        rel = float((x.cpu().double() - y).norm() / y.norm())
        print(name, "rel err %.3e" % rel, flush=True)
        assert rel < 7e-7, (name, rel)


@pytest.mark.parametrize("dtype,hq,hkv,l,d,r,iters,tol",
                         [(torch.float32, 4, 2, 40, 16, 4, 2, 0.0), (torch.float32, 4, 2, 700, 16, 4, 0, 0.0),
                          (torch.float32, 28, 4, 1024, 128, 16, 1, 1e-2), (torch.bfloat16, 8, 2, 3000, 128, 32, 3, 0.0),
                          (torch.float32, 2, 1, 333, 8, 3, 6, 1e30), (torch.float32, 2, 1, 333, 8, 3, 6, 5e-2),
                          (torch.bfloat16, 4, 2, 1500, 64, 8, 2, 0.0), (torch.bfloat16, 2, 2, 777, 256, 32, 2, 0.0),
                          (torch.bfloat16, 2, 1, 500, 12, 4, 2, 0.0), (torch.float32, 2, 1, 4500, 96, 24, 2, 0.0),
                          # bf16 input on the bf16 matrix cores: d = 96 (rows not a whole number of 32-column
                          # blocks), one block, a prompt shorter than one tile, a ragged last tile per split
                          (torch.bfloat16, 2, 1, 1000, 96, 24, 2, 0.0), (torch.bfloat16, 2, 2, 333, 32, 16, 2, 0.0),
                          (torch.bfloat16, 2, 1, 37, 64, 8, 1, 0.0), (torch.bfloat16, 4, 1, 20011, 128, 32, 2, 0.0),
                          # the iteration on Gram matrices (bf16 rows of 128): ranks below 32 (identity padding of the
                          # r x r systems), one iteration, and the batch-wide stopping test after the first / a later one
                          (torch.bfloat16, 4, 2, 2000, 128, 16, 3, 0.0), (torch.bfloat16, 2, 1, 1500, 128, 24, 1, 0.0),
                          (torch.bfloat16, 2, 1, 1200, 128, 32, 6, 1e30), (torch.bfloat16, 4, 2, 1500, 128, 20, 6, 5e-2),
                          # head groupings: one query head per kv head and eight (the last pass then goes head by head)
                          (torch.bfloat16, 2, 2, 900, 128, 32, 2, 0.0), (torch.bfloat16, 8, 1, 1100, 128, 16, 2, 0.0),
                          # a rank that is no multiple of the four pivots of an elimination step
                          (torch.bfloat16, 4, 1, 600, 128, 6, 2, 0.0),
                          # ranks beyond 32 (the general kernels): 64 with rows of 128 elements, 48, 40
                          (torch.bfloat16, 4, 2, 1500, 128, 64, 2, 0.0), (torch.float32, 2, 1, 700, 64, 48, 2, 0.0),
                          (torch.bfloat16, 2, 1, 900, 128, 40, 3, 0.0), (torch.float32, 2, 1, 500, 64, 33, 2, 0.0),
                          (torch.float32, 2, 2, 600, 128, 64, 2, 0.0)])
def test_als_prefill(ops, ws, oracle, dtype, hq, hkv, l, d, r, iters, tol):
    _say("als_prefill", dtype, hq, l, d, r, iters, tol)
    from lrqk_amd import synth
    g = torch.Generator().manual_seed(l)
    b = 1
    Q, _ = synth.low_rank_noise(g, b, hq, l, d, max(r, 4), 0.05, dtype)
    K, _ = synth.low_rank_noise(g, b, hkv, l, d, max(r, 4), 0.05, dtype)
    A_Q0 = torch.randn((b, hq, l, r), generator=g)
    A_K0 = torch.randn((b, hq, l, r), generator=g)
    ref = oracle.als_prefill_w1(Q.double(), oracle.repeat_kv(K, hq // hkv).double(), A_Q0.double(), A_K0.double(),
                                iters, tol)
    got = ops.als_prefill(ws, Q.to(DEV), K.to(DEV), A_Q0.to(DEV), A_K0.to(DEV), iters, tol)
    # A_Q, A_K are only defined up to the conditioning of the r x r systems; compare the
    # products the path actually uses (fits and proxy scores), fp32 vs fp64: 1e-3
    AQ, BQ, AK, BK = [t.cpu().double() for t in got]
    for name, x, y in (("A_Q B_Q", AQ @ BQ, ref[0] @ ref[1]), ("A_K B_K", AK @ BK, ref[2] @ ref[3]),
                       ("A_Q A_K^T last row", AQ[:, :, -1:] @ AK.transpose(-1, -2), ref[0][:, :, -1:] @ ref[2].transpose(-1, -2)),
                       ("A_K", AK, ref[2]), ("B_K", BK, ref[3]), ("A_Q", AQ, ref[0]), ("B_Q", BQ, ref[1])):
        rel = (x - y).norm() / y.norm()
        # the individual factors depend on the conditioning of the r x r systems: 5e-3
        assert rel < (5e-3 if name in ("A_K", "B_K", "A_Q", "B_Q") else 1e-3), (name, float(rel))


def test_als_prefill_large_sums_every_head(ops, ws, oracle):
    """128K rows of rank-r data factorised at rank r from random factors: after the first iteration the K side's
    r x r systems have diagonals around 1e12 and condition numbers around 1e5.  The elimination used to leave
    D^-1 X in its pivot rows as X - (I - D^-1) X, which cancels in the leading digits at that size: B_K of one head
    in ten came out 5e-3 off its own system and A_K B_K up to 0.26 off the fp64 oracle, on heads that a check of
    two heads did not happen to look at.  Every head of a block that held four such heads is compared here; the
    oracle's own fp32 run is up to 3e-2 off on this prompt, the limit is 1e-3 (measured: 3.4e-4 at most)."""
    _say("als_prefill 128K, a block of heads")
    from lrqk_amd import synth
    oracle.set_threads(16)
    try:
        b, hq, hkv, l, d, r, iters = 1, 32, 8, 131072, 128, 32, 2
        gen = torch.Generator(device=DEV).manual_seed(0)
        Q, _ = synth.low_rank_noise(gen, b, hq, l, d, 32, 0.01, torch.bfloat16)
        K, _ = synth.low_rank_noise(gen, b, hkv, l, d, 32, 0.01, torch.bfloat16)
        A_Q0 = torch.randn((b, hq, l, r), generator=gen, device=DEV)
        A_K0 = torch.randn((b, hq, l, r), generator=gen, device=DEV)
        got = ops.als_prefill(ws, Q, K, A_Q0.clone(), A_K0.clone(), iters, 0.0)
        hs = list(range(15, 23))
        AQ, BQ, AK, BK = [t[:, hs].cpu().double() for t in got]
        del got
        ref = oracle.als_prefill_w1(Q[:, hs].cpu().double(), oracle.repeat_kv(K.cpu(), hq // hkv)[:, hs].double(),
                                    A_Q0[:, hs].cpu().double(), A_K0[:, hs].cpu().double(), iters, 0.0)
        for j, h in enumerate(hs):
            for name, x, y in (("A_K B_K", AK[0, j] @ BK[0, j], ref[2][0, j] @ ref[3][0, j]),
                               ("A_Q B_Q", AQ[0, j] @ BQ[0, j], ref[0][0, j] @ ref[1][0, j])):
                rel = float((x - y).norm() / y.norm())
                _say(f"   head {h} {name}: {rel:.2e}")
                assert rel < 1e-3, (h, name, rel)
    finally:
        oracle.set_threads(1)


def test_als_prefill_benchmark_configuration(ops, ws, oracle):
    """The prefill-factorisation benchmark exactly as it is specified: 32 query / 8 kv heads, 32768 tokens,
    d 128, bf16 rows of rank 48 plus N(0, 0.05) noise, r 32, max_iter 4, tol 1e-8 -- against the fp64 oracle
    on four query heads (of different kv groups), together with both fit residuals."""
    _say("als_prefill benchmark configuration")
    from lrqk_amd import synth
    w = synth.WORKLOADS["llama8b_32k_prefill_als"]
    l, r, d = w.context, w.r, w.head_dim
    assert (w.num_heads, w.num_kv_heads, l, r, w.max_iter[0], w.tol[0], w.rho, w.sigma) == (32, 8, 32768, 32, 4, 1e-8, 48, 0.05)
    Qd, Kd, _, _, _ = synth.prompt_qkv(w, 0, l, device=DEV)
    A0 = synth.init_factors(w, l, 1, device=DEV)
    got = ops.als_prefill(ws, Qd, Kd, A0[0].clone(), A0[1].clone(), w.max_iter[0], w.tol[0])
    heads = [0, 9, 22, 31]
    g = w.groups
    Q = Qd[:, heads].cpu().double()
    K = Kd[:, [h // g for h in heads]].cpu().double()
    ref = oracle.als_prefill_w1(Q, K, A0[0][:, heads].cpu().double(), A0[1][:, heads].cpu().double(), w.max_iter[0], w.tol[0])
    AQ, BQ, AK, BK = [t[:, heads].cpu().double() for t in got]

    def rel(x, y):
        return float((x - y).norm() / y.norm())

    # fp32 arithmetic (bf16 matrix cores on three-way split operands) against fp64: 1e-3 on what the path uses,
    # 5e-3 on the individual factors (conditioning of the r x r systems)
    for name, x, y, lim in (("A_K B_K", AK @ BK, ref[2] @ ref[3], 1e-3), ("A_Q B_Q", AQ @ BQ, ref[0] @ ref[1], 1e-3),
                            ("A_Q[-1] A_K^T", AQ[:, :, -1:] @ AK.transpose(-1, -2), ref[0][:, :, -1:] @ ref[2].transpose(-1, -2), 1e-3),
                            ("A_K", AK, ref[2], 5e-3), ("B_K", BK, ref[3], 5e-3), ("A_Q", AQ, ref[0], 5e-3), ("B_Q", BQ, ref[1], 5e-3)):
        dev = rel(x, y)
        print("  %-14s deviation from fp64 %.2e (limit %.0e)" % (name, dev, lim), flush=True)
        assert dev < lim, (name, dev)
    res_g, res_o = rel(AK @ BK, K), rel(ref[2] @ ref[3], K)
    resq_g, resq_o = rel(AQ @ BQ, Q), rel(ref[0] @ ref[1], Q)
    print("  residual K: kernel %.6f oracle %.6f; residual Q: kernel %.6f oracle %.6f" % (res_g, res_o, resq_g, resq_o),
          flush=True)
    assert abs(res_g - res_o) < 1e-4 and abs(resq_g - resq_o) < 1e-4


def test_random_kernel_shapes(ops, ws, oracle):
    """160 seeded random shapes through the checks above (factor update incl. the general-rank kernels, attention,
    hit/miss diff, selection with tied and quantised scores): sizes next to the powers of two and split boundaries
    that the fixed cases are built around, not on them."""
    import random
    for i in range(160):
        rng = random.Random(4200 + i)
        kind = rng.choice(["als", "als", "attention", "diff", "select"])
        dtype = rng.choice([torch.float32, torch.bfloat16])
        if kind == "als":
            d = rng.choice([8, 16, 32, 64, 128, 256] if dtype == torch.float32 else [16, 32, 64, 128, 256])
            hkv = rng.choice([1, 2, 3])
            r = min(rng.choice([2, 3, 4, 8, 16, 24, 32, 33, 40, 48, 64]), d // 2)
            if dtype == torch.bfloat16:
                r = max(8, r // 8 * 8)                       # 16-byte rows of A_K
            if r > 32 and d == 256:
                r = 32                                       # (refused: ranks above 32 take rows of at most 128 elements)
            n = max(rng.choice([r + 1, 2 * r + 3, 70, 129, 300, 544, 1000, 2112, 3000, 4160]), r + 1)
            max_iter, tol = rng.choice([(1, 0.0), (2, 0.0), (3, 1e30), (4, 1e-6), (8, 1e-8)])
            _check_als_decode(ops, ws, oracle, dtype, hkv * rng.choice([1, 2, 4]), hkv, n, d, r, max_iter, tol)
        elif kind == "attention":
            d = rng.choice([8, 16, 32, 64, 128, 256] if dtype == torch.float32 else [16, 32, 64, 128, 256])
            test_attention(ops, ws, oracle, dtype, d,
                           rng.choice([1, 2, 12, 63, 64, 65, 100, 255, 256, 257, 544, 1000, 2112, 4224, 9000]))
        elif kind == "diff":
            k = rng.choice([1, 2, 8, 100, 512, 1000, 2048, 2500, 4096, 5000, 8192])
            test_diff_random(ops, oracle, k, k + rng.choice([1, 5, k, 10 * k]))
        else:
            m = rng.choice([9, 100, 1000, 5000, 40000, 70000])
            k = rng.choice([1, 8, 64, 512, 2048, 4096, 8192])
            g = torch.Generator().manual_seed(i)
            s = torch.randn((2, 3, m), generator=g)
            mode = rng.choice(["plain", "few values", "bf16 values"])
            s = (s * 2).round() / 2 if mode == "few values" else (s.bfloat16().float() if mode == "bf16 values" else s)
            _say("select", m, k, mode)
            if m <= k:
                got = ops.select_from_scores(ws, s.to(DEV), k).cpu()
                assert torch.equal(got, torch.arange(m, dtype=torch.int32).expand(2, 3, m))
            else:
                _check_select(ops, ws, oracle, s, k)


def test_measurement_probes(ops):
    """The plain read / copy kernels and the event-pair calibration that the bench line carries: the copy
    really copies, the rates and the bracket are finite and of a plausible order of magnitude."""
    print("probes: bandwidth + event pair", flush=True)
    read_gbs, copy_gbs = ops.probe_bandwidth(64 << 20, 3, DEV)
    assert 50.0 < read_gbs < 20000.0 and 50.0 < copy_gbs < 20000.0, (read_gbs, copy_gbs)
    pair = ops.probe_event_pair(16, DEV)
    assert 0.0 < pair < 500.0, pair
    pair2 = ops.probe_event_pair(16, DEV, kernels=2)
    assert pair < pair2 + 5.0 < 505.0, (pair, pair2)
    with pytest.raises(ValueError):
        ops.probe_event_pair(0, DEV)
    with pytest.raises(ValueError):
        ops.probe_event_pair(4, DEV, kernels=0)
    # every variant of the read sweep runs and reads a plausible rate (ragged size: the last vectors are clamped)
    table, best = ops.probe_read_sweep((64 << 20) + 4096 + 16, 2, DEV)
    assert len(table) == 24 and all(50.0 < v < 20000.0 for v in table.values()), table
    assert best == max(table.values())
    # launches that take slices of the buffer in turn
    table, best = ops.probe_read_sweep(64 << 20, 1, DEV, slice_bytes=8 << 20)
    assert len(table) == 24 and all(20.0 < v < 20000.0 for v in table.values()), table
    with pytest.raises(ValueError):
        ops.probe_read_sweep(64 << 20, 1, DEV, slice_bytes=24)
