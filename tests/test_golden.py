"""Committed fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py).

CPU: the oracle reproduces every fixture (a change of the oracle that alters results fails
here).  GPU: the HIP stages reproduce them through the C ABI -- integer outputs bit for bit,
floating point within the stated tolerances.
"""
import os

import numpy as np
import pytest
import torch

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DEV = "cuda:0"
TIE_CASES = ["all_equal", "two_level", "boundary_tie", "signed_zero", "short_row"]


def _load(name):
    return {k: v for k, v in np.load(os.path.join(GOLD, name), allow_pickle=False).items()}


def _t(a):
    return torch.from_numpy(np.ascontiguousarray(a))


# ------------------------------------------------------------------------------- CPU: oracle
def test_oracle_diff_docstring(oracle):
    g = _load("diff_docstring.npz")
    now, new = _t(g["now"]).view(1, 1, -1, 1), _t(g["new"]).view(1, 1, -1, 1)
    upd, ev = oracle.only_indices_in_cpu(now, new)
    assert upd.view(-1).tolist() == g["updated"].tolist()
    assert ev.view(-1).to(torch.uint8).tolist() == g["evict"].tolist()


@pytest.mark.parametrize("case", TIE_CASES)
def test_oracle_topk_ties(oracle, case):
    g = _load("topk_ties.npz")
    sc, k = _t(g[case + "_scores"]), int(g[case + "_k"])
    got = oracle.topk_sorted(sc.view(1, 1, -1), k).view(-1)
    assert got.tolist() == g[case + "_idx"].tolist()
    # independent of the oracle's sort: numpy lexsort on (index, -score)
    order = np.lexsort((np.arange(sc.numel()), -(sc.numpy() + 0.0)))[:k]
    assert sorted(order.tolist()) == got.tolist()


def test_oracle_trace_small(oracle):
    g = _load("trace_small.npz")
    b, hq, hkv, d, r, k, L, l, steps = g["shape"].tolist()
    eng = oracle.OracleLayer(num_lite_tokens=L, attn_topk=k, num_key_value_groups=hq // hkv, r=r, max_iter=(2, 2),
                             tol=(1e-8, 1e-8), capacity=16, compute_dtype=torch.float64)
    eng.prefill(_t(g["Q"]), _t(g["K"]), _t(g["V"]), A_Q0=_t(g["A_Q0"]), A_K0=_t(g["A_K0"]))
    assert torch.equal(eng.hit_indices, _t(g["prefill_hit"]))
    torch.testing.assert_close(eng.B_Q, _t(g["prefill_B_Q"]), rtol=1e-5, atol=1e-6)
    for s in range(steps):
        Ko, Vo = eng.decode(_t(g["step_q"][s]), _t(g["step_k"][s]), _t(g["step_v"][s]))
        assert eng.last_m == int(g["step_m"][s])
        assert torch.equal(eng.last_new_indices, _t(g["step_new_idx"][s])), s
        assert torch.equal(eng.hit_indices, _t(g["step_hit_after"][s])), s
        assert torch.equal(eng.last_evict.to(torch.uint8), _t(g["step_evict"][s])), s
        torch.testing.assert_close(Ko, _t(g["step_Kact"][s]), rtol=0, atol=0)
        torch.testing.assert_close(eng.last_q_hat, _t(g["step_q_hat"][s]), rtol=1e-5, atol=1e-6)
    assert eng.lite_indices == g["final_lite_indices"].tolist()
    torch.testing.assert_close(eng.KVcpu.tensor(), _t(g["final_store"]), rtol=0, atol=0)


# ------------------------------------------------------------------------------- GPU: HIP stages
@pytest.fixture(scope="module")
def hip():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from lrqk_amd import ops
    return ops, ops.Workspace()


@pytest.mark.gpu
def test_hip_diff_docstring(hip):
    ops, ws = hip
    g = _load("diff_docstring.npz")
    hit = _t(g["now"]).to(torch.int32).view(1, 1, -1).to(DEV)
    new = _t(g["new"]).to(torch.int32).view(1, 1, -1).to(DEV)
    evict, slots, count = ops.diff(new, hit)
    assert hit.view(-1).tolist() == g["updated"].tolist()
    assert evict.view(-1).tolist() == g["evict"].tolist()
    assert int(count) == 2 and slots.view(-1)[:2].tolist() == [1, 4]


@pytest.mark.gpu
@pytest.mark.parametrize("case", TIE_CASES)
def test_hip_topk_ties(hip, case):
    ops, ws = hip
    g = _load("topk_ties.npz")
    sc, k = _t(g[case + "_scores"]), int(g[case + "_k"])
    got = ops.select_from_scores(ws, sc.view(1, 1, -1).to(DEV), k)
    assert got.view(-1).tolist() == g[case + "_idx"].tolist()


@pytest.mark.gpu
def test_hip_trace_small_stages(hip):
    """Every step of the 40-step trace, stage by stage from the recorded state: selection and diff
    exact; factor update 2e-3 relative to the fp64 record (fp32 arithmetic, r x r systems of a
    rank-3 stream); attention 1e-5 relative (fp32 storage)."""
    ops, ws = hip
    g = _load("trace_small.npz")
    b, hq, hkv, d, r, k, L, l, steps = g["shape"].tolist()
    a_k = _t(g["final_A_K"]).to(DEV).contiguous()   # rows are append-only: a prefix is the state of any step
    worst = 0.0
    for s in range(steps):
        print("trace step", s, flush=True)
        m = int(g["step_m"][s])
        q_hat = _t(g["step_q_hat"][s]).to(DEV)
        new = ops.score_select(ws, a_k, q_hat, m, k)
        assert torch.equal(new.cpu().long(), _t(g["step_new_idx"][s]).squeeze(-1)), s
        hit = _t(g["step_hit_before"][s]).squeeze(-1).to(torch.int32).to(DEV).contiguous()
        evict, slots, count = ops.diff(new.contiguous(), hit)
        assert torch.equal(hit.cpu().long(), _t(g["step_hit_after"][s]).squeeze(-1)), s
        assert torch.equal(evict.cpu(), _t(g["step_evict"][s])), s
        assert torch.equal(count.cpu().long(), _t(g["step_evict"][s]).long().sum(-1)), s
        # attention over the recorded active set
        out = ops.attention(ws, _t(g["step_q"][s]).to(DEV), _t(g["step_Kact"][s]).to(DEV).contiguous(),
                            _t(g["step_Vact"][s]).to(DEV).contiguous())
        exp = _t(g["step_attn"][s])
        assert float((out.cpu() - exp).norm() / exp.norm()) < 1e-5, s
        # factor update from the recorded inputs
        b_q, b_k = _t(g["step_B_Q_in"][s]).to(DEV).contiguous(), _t(g["step_B_K_in"][s]).to(DEV).contiguous()
        act = _t(g["step_A_act_in"][s]).to(DEV).contiguous()
        qh, kh = ops.als_decode(ws, b_q, b_k, act, None, _t(g["step_K_prev"][s]).to(DEV).contiguous(), k + L,
                                _t(g["step_q"][s]).to(DEV), _t(g["step_k"][s]).to(DEV), 2, 1e-8)
        for got, name in ((qh, "q_hat"), (kh, "k_hat"), (b_q, "B_Q"), (b_k, "B_K")):
            e = _t(g["step_" + name][s])
            rel = float((got.cpu() - e).norm() / e.norm())
            worst = max(worst, rel)
            assert rel < 2e-3, (s, name, rel)
    print("worst factor deviation", worst, flush=True)
