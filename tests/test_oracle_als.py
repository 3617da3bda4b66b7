"""Pins the floating-point half of the oracle (ALS prefill, ALS decode, attention) against
numpy's least-squares routine, closed forms and invariants.  fp64 throughout so that a
dropped term, a wrong sign or a transposed operand is far outside the tolerance."""
import numpy as np
import pytest
import torch

F64 = torch.float64


def _rand(gen, *shape):
    return torch.randn(shape, generator=gen, dtype=F64)


def _lstsq(A, B):
    return torch.from_numpy(np.linalg.lstsq(A.numpy(), B.numpy(), rcond=None)[0])


# ---------------------------------------------------------------- prefill

def test_prefill_zero_iterations_is_lstsq(oracle):
    g = torch.Generator().manual_seed(0)
    Q, K = _rand(g, 1, 2, 30, 8), _rand(g, 1, 2, 30, 8)
    A_Q0, A_K0 = _rand(g, 1, 2, 30, 3), _rand(g, 1, 2, 30, 3)
    A_Q, B_Q, A_K, B_K = oracle.als_prefill_w1(Q, K, A_Q0, A_K0, max_iter=0)
    assert torch.equal(A_Q, A_Q0) and torch.equal(A_K, A_K0)
    for h in range(2):
        assert torch.allclose(B_Q[0, h], _lstsq(A_Q0[0, h], Q[0, h]), atol=1e-10)
        assert torch.allclose(B_K[0, h], _lstsq(A_K0[0, h], K[0, h]), atol=1e-10)


def test_prefill_one_iteration_vs_stacked_least_squares(oracle):
    """Each block update minimises f over that block; written as an independent stacked
    least-squares problem solved by numpy.  Catches Jacobi-vs-Gauss-Seidel, transposes, signs."""
    g = torch.Generator().manual_seed(1)
    l, d, r = 24, 6, 3
    Q, K = _rand(g, 1, 1, l, d), _rand(g, 1, 1, l, d)
    A_Q0, A_K0 = _rand(g, 1, 1, l, r), _rand(g, 1, 1, l, r)
    A_Q, B_Q, A_K, B_K = oracle.als_prefill_w1(Q, K, A_Q0, A_K0, max_iter=1, tol=0.0)
    q, k, aq0, ak0 = Q[0, 0], K[0, 0], A_Q0[0, 0], A_K0[0, 0]
    bq0, bk0 = _lstsq(aq0, q), _lstsq(ak0, k)
    I = torch.eye(d, dtype=F64)
    # A_Q: min |Q K^T - A_Q A_K0^T|^2 + |Q - A_Q B_Q0|^2  ==  min |[K;I] Q^T - [A_K0; B_Q0^T] A_Q^T|^2
    aq1 = _lstsq(torch.cat([ak0, bq0.T]), torch.cat([k, I]) @ q.T).T
    # A_K with the NEW A_Q: min |K Q^T - A_K A_Q1^T|^2 + |K - A_K B_K0|^2
    ak1 = _lstsq(torch.cat([aq1, bk0.T]), torch.cat([q, I]) @ k.T).T
    assert torch.allclose(A_Q[0, 0], aq1, atol=1e-9)
    assert torch.allclose(A_K[0, 0], ak1, atol=1e-9)
    assert torch.allclose(B_Q[0, 0], _lstsq(aq1, q), atol=1e-9)
    assert torch.allclose(B_K[0, 0], _lstsq(ak1, k), atol=1e-9)


def test_prefill_objective_monotone_and_orthogonality(oracle):
    g = torch.Generator().manual_seed(2)
    Q, K = _rand(g, 2, 3, 64, 16), _rand(g, 2, 3, 64, 16)
    A_Q0, A_K0 = _rand(g, 2, 3, 64, 4), _rand(g, 2, 3, 64, 4)
    trace = []
    A_Q, B_Q, A_K, B_K = oracle.als_prefill_w1(Q, K, A_Q0, A_K0, max_iter=6, tol=0.0, trace=trace)
    f = torch.stack([t[1] for t in trace])  # [steps,b,H]
    assert len(trace) == 6 * 3 + 1
    assert torch.all(f[1:] <= f[:-1] * (1 + 1e-12) + 1e-9)
    assert torch.all(f[-1] < 0.9 * f[0])
    # normal equations of the final B solve
    assert torch.matmul(A_Q.transpose(-1, -2), Q - torch.matmul(A_Q, B_Q)).abs().max() < 1e-8
    assert torch.matmul(A_K.transpose(-1, -2), K - torch.matmul(A_K, B_K)).abs().max() < 1e-8


def test_prefill_recovers_exact_low_rank(oracle):
    g = torch.Generator().manual_seed(3)
    r = 4
    Q = _rand(g, 1, 2, 80, r) @ _rand(g, 1, 2, r, 16)
    K = _rand(g, 1, 2, 80, r) @ _rand(g, 1, 2, r, 16)
    A_Q, B_Q, A_K, B_K = oracle.als_prefill_w1(Q, K, _rand(g, 1, 2, 80, r), _rand(g, 1, 2, 80, r), 30, 0.0)
    assert (Q - A_Q @ B_Q).norm() / Q.norm() < 1e-6
    assert (K - A_K @ B_K).norm() / K.norm() < 1e-6
    QK = Q @ K.transpose(-1, -2)
    assert (QK - A_Q @ A_K.transpose(-1, -2)).norm() / QK.norm() < 1e-5


def test_prefill_early_exit_is_batch_wide(oracle):
    g = torch.Generator().manual_seed(4)
    Q, K = _rand(g, 1, 2, 40, 8), _rand(g, 1, 2, 40, 8)
    A_Q0, A_K0 = _rand(g, 1, 2, 40, 3), _rand(g, 1, 2, 40, 3)
    big = oracle.als_prefill_w1(Q, K, A_Q0, A_K0, max_iter=5, tol=1e30)   # breaks after iteration 1
    one = oracle.als_prefill_w1(Q, K, A_Q0, A_K0, max_iter=1, tol=0.0)
    for a, b in zip(big, one):
        assert torch.equal(a, b)


def test_prefill_scale_equivariance(oracle):
    # (Q,K,A0) -> (cQ, K/c, cA_Q0, A_K0/c) leaves QK^T fixed but rescales the other two terms,
    # so only a joint scaling of everything is an equivariance: f(cQ,cK) with cA0 gives cA, B fixed.
    g = torch.Generator().manual_seed(5)
    Q, K = _rand(g, 1, 1, 30, 8), _rand(g, 1, 1, 30, 8)
    a, b = _rand(g, 1, 1, 30, 3), _rand(g, 1, 1, 30, 3)
    P = torch.randperm(30, generator=g)
    x = oracle.als_prefill_w1(Q, K, a, b, 3, 0.0)
    # row permutation of Q (with its A_Q0) permutes A_Q and changes nothing else
    y = oracle.als_prefill_w1(Q[:, :, P], K, a[:, :, P], b, 3, 0.0)
    assert torch.allclose(y[0], x[0][:, :, P], atol=1e-9) and torch.allclose(y[1], x[1], atol=1e-9)
    assert torch.allclose(y[2], x[2], atol=1e-9) and torch.allclose(y[3], x[3], atol=1e-9)


def test_cast_prefill_dtype_and_injection(oracle):
    g = torch.Generator().manual_seed(6)
    Q = torch.randn((1, 2, 32, 8), generator=g).bfloat16()
    K = torch.randn((1, 2, 32, 8), generator=g).bfloat16()
    A0 = torch.randn((1, 2, 32, 4), generator=g)
    out = oracle.cast_lrqk_prefill(Q, K, 4, 2, 1e-8, A_Q0=A0, A_K0=A0.flip(2))
    assert all(o.dtype == torch.bfloat16 for o in out)
    assert out[0].shape == (1, 2, 32, 4) and out[1].shape == (1, 2, 4, 8)
    for m in ("top", "topcol"):
        o = oracle.cast_lrqk_prefill(Q, K, 4, 1, 1e-8, init_method=m)
        assert o[2].shape == (1, 2, 32, 4)
    with pytest.raises(ValueError):
        oracle.cast_lrqk_prefill(Q, K, 4, 1, 1e-8, init_method="nope")


def test_init_top_and_topcol_pick_heaviest_columns(oracle):
    Q = torch.zeros((1, 1, 5, 6))
    K = torch.zeros((1, 1, 5, 6))
    Q[..., 1] = 3.0; Q[..., 4] = 2.0; Q[..., 0] = 0.5
    K[..., 2] = 5.0; K[..., 4] = 1.0; K[..., 5] = 0.1
    AQ, AK = oracle.init_aq_ak(Q, K, 2, "top")
    assert torch.equal(AQ[0, 0, 0], torch.tensor([3.0, 2.0])) and torch.equal(AK[0, 0, 0], torch.tensor([5.0, 1.0]))
    AQ, AK = oracle.init_aq_ak(Q, K, 2, "topcol")  # column sums |Q|+|K|: col2=25, col1=15, col4=15 -> 2 then 1 or 4
    assert AK[0, 0, 0, 0] == 5.0 and AQ[0, 0, 0, 0] == 0.0


# ---------------------------------------------------------------- decode

def _decode_inputs(g, b=1, H=2, n=20, d=8, r=3):
    return dict(B_Q=_rand(g, b, H, r, d), A_K=_rand(g, b, H, n, r), B_K=_rand(g, b, H, r, d),
                K__=_rand(g, b, H, n, d), q=_rand(g, b, H, 1, d), k=_rand(g, b, H, 1, d))


def test_decode_half_steps_vs_stacked_least_squares(oracle):
    g = torch.Generator().manual_seed(10)
    x = _decode_inputs(g)
    trace = []
    oracle.als_decode_w1(**x, max_iter=3, tol=0.0, trace=trace)
    assert trace[0][0] == "k0" and len(trace) == 4
    for h in range(2):
        BQ, AK, BK, Kk, q, k = (x[n][0, h] for n in ("B_Q", "A_K", "B_K", "K__", "q", "k"))
        s = (q @ k.T)
        # k_hat_0 = argmin |k_hat B_K - k|
        k0 = _lstsq(BK.T, k.T).T
        assert torch.allclose(trace[0][1][0, h], k0, atol=1e-10)
        for it in trace[1:]:
            k_in, q_hat, k_out = it[1][0, h], it[2][0, h], it[3][0, h]
            # q_hat = argmin |q_hat B_Q - q|^2 + |q_hat A_K^T - q K__^T|^2 + (q_hat k_in^T - q k^T)^2
            qh = _lstsq(torch.cat([BQ.T, AK, k_in]), torch.cat([q.T, Kk @ q.T, s])).T
            assert torch.allclose(q_hat, qh, atol=1e-9)
            # k_hat' = argmin |k_hat B_K - k|^2 + (q_hat k_hat^T - q k^T)^2
            kh = _lstsq(torch.cat([BK.T, q_hat]), torch.cat([k.T, s])).T
            assert torch.allclose(k_out, kh, atol=1e-9)
        # consecutive iterations chain
        assert torch.equal(trace[2][1], trace[1][3])


def test_decode_B_step_is_exact_line_search(oracle):
    g = torch.Generator().manual_seed(11)
    x = _decode_inputs(g)
    B_Q, B_K, hq, hk = oracle.als_decode_w1(**x, max_iter=2, tol=0.0)
    # with the exact minimising step the fit q_hat B_Q' = q is exact (up to the 1e-6 epsilon)
    assert torch.allclose(hq @ B_Q, x["q"], atol=5e-4)
    assert torch.allclose(hk @ B_K, x["k"], atol=5e-4)
    # and B moves along -dB only: B' - B is rank one with row space spanned by (q_hat B - q)
    dB = (B_Q - x["B_Q"])[0, 0]
    assert np.linalg.matrix_rank(dB.numpy(), tol=1e-9) == 1
    e = (hq @ x["B_Q"] - x["q"])[0, 0]
    lr = 1.0 / float((hq[0, 0] ** 2).sum())
    assert torch.allclose(dB, -lr * hq[0, 0].T @ e, atol=5e-4)


def test_decode_iteration_clamp_and_batchwide_exit(oracle):
    g = torch.Generator().manual_seed(12)
    x = _decode_inputs(g, b=2, H=3)
    a = oracle.als_decode_w1(**x, max_iter=0, tol=0.0)
    b = oracle.als_decode_w1(**x, max_iter=1, tol=0.0)
    c = oracle.als_decode_w1(**x, max_iter=7, tol=1e30)
    for u, v, w in zip(a, b, c):
        assert torch.equal(u, v) and torch.equal(u, w)
    d = oracle.als_decode_w1(**x, max_iter=2, tol=0.0)
    assert not torch.equal(d[2], b[2])


def test_cast_decode_rounds_to_storage(oracle):
    g = torch.Generator().manual_seed(13)
    x = {k: v.bfloat16() for k, v in _decode_inputs(g).items()}
    out = oracle.cast_lrqk_decode(**x, max_iter=2, tol=1e-8)
    assert all(o.dtype == torch.bfloat16 for o in out)
    ref = oracle.als_decode_w1(**{k: v.double() for k, v in x.items()}, max_iter=2, tol=1e-8)
    for o, t in zip(out, ref):
        assert (o.double() - t).norm() / t.norm() < 2e-2


# ---------------------------------------------------------------- attention

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_vs_sdpa(oracle, dtype):
    g = torch.Generator().manual_seed(20)
    q = torch.randn((2, 4, 1, 16), generator=g).to(dtype)
    K = torch.randn((2, 4, 33, 16), generator=g).to(dtype)
    V = torch.randn((2, 4, 33, 16), generator=g).to(dtype)
    out = oracle.attention(q, K, V)
    ref = torch.nn.functional.scaled_dot_product_attention(q.double(), K.double(), V.double())
    assert torch.allclose(out, ref, atol=1e-12)
    # one key: the output is that value row
    assert torch.allclose(oracle.attention(q, K[:, :, :1], V[:, :, :1]), V[:, :, :1].double())


def test_fp32_run_against_fp64_run_on_rank_r_data(oracle):
    """How far an fp32 run of the prefill factorisation is from an fp64 run of the same algorithm on the
    decode benchmark's data (rows of rank 32 plus N(0, 0.01) noise, bf16, r 32, max_iter 2, Llama head
    size): the r x r systems reach condition numbers of 1e5..1e6, so the individual factors of the two runs
    differ by percents, while everything the path uses them for (the fits A_K B_K, A_Q B_Q and the proxy
    scores A_Q[-1] A_K^T) agrees to better than 2e-3.  This is why the GPU traces at that shape compare
    products, with a limit of three times this deviation, and not the factors element by element.  On the
    prefill benchmark's data (rank 48 + 0.05 noise) the systems are benign and the factors agree as well."""
    from lrqk_amd import synth
    orc = oracle

    def run(rho, sigma, iters):
        g = torch.Generator().manual_seed(0)
        b, hq, hkv, l, d, r = 1, 4, 1, 8192, 128, 32
        Q, _ = synth.low_rank_noise(g, b, hq, l, d, rho, sigma, torch.bfloat16)
        K, _ = synth.low_rank_noise(g, b, hkv, l, d, rho, sigma, torch.bfloat16)
        A_Q0 = torch.randn((b, hq, l, r), generator=g)
        A_K0 = torch.randn((b, hq, l, r), generator=g)
        Kr = orc.repeat_kv(K, hq // hkv)
        r64 = orc.als_prefill_w1(Q.double(), Kr.double(), A_Q0.double(), A_K0.double(), iters, 0.0)
        r32 = orc.als_prefill_w1(Q.float(), Kr.float(), A_Q0.float(), A_K0.float(), iters, 0.0)
        rel = lambda x, y: float((x.double() - y).norm() / y.norm())
        factors = {n: rel(x, y) for n, x, y in zip(("A_Q", "B_Q", "A_K", "B_K"), r32, r64)}
        prods = {"A_K B_K": rel(r32[2] @ r32[3], r64[2] @ r64[3]), "A_Q B_Q": rel(r32[0] @ r32[1], r64[0] @ r64[1]),
                 "scores": rel(r32[0][:, :, -1:] @ r32[2].transpose(-1, -2), r64[0][:, :, -1:] @ r64[2].transpose(-1, -2))}
        cond = float(torch.linalg.cond(r64[0].transpose(-1, -2) @ r64[0]).max())
        return factors, prods, cond

    factors, prods, cond = run(32, 0.01, 2)
    print("rank-32 data: cond %.1e factors %s products %s" % (cond, factors, prods))
    assert cond > 1e4
    assert max(factors.values()) > 5e-3          # the factors themselves are not comparable at 1e-3 ...
    assert max(prods.values()) < 2e-3            # ... their products are
    factors, prods, cond = run(48, 0.05, 4)
    print("rank-48 data: cond %.1e factors %s products %s" % (cond, factors, prods))
    assert cond < 1e4 and max(factors.values()) < 1e-4 and max(prods.values()) < 1e-4
