"""Pins the bit-exact half of the oracle: proxy score, top-k order, hit/miss diff, gathers,
buffers.  None of these tests restates the oracle's formula: each compares against a held
known answer, a library routine, brute force, or the reference's own compiled C++."""
import importlib.util
import os
import sys

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REF_SO = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "take_along_dim_grouped.so")


def _ref_module():
    if not os.path.exists(REF_SO):
        pytest.skip("oracle/_ref not built")
    spec = importlib.util.spec_from_file_location("take_along_dim_grouped", REF_SO)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


# ---------------------------------------------------------------- proxy score

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("r", [8, 16, 32])
def test_scores_match_fp64_dot(oracle, dtype, r):
    g = torch.Generator().manual_seed(r)
    A = torch.randn((2, 3, 257, r), generator=g).to(dtype)
    q = torch.randn((2, 3, 1, r), generator=g).to(dtype)
    s = oracle.proxy_scores(A, q, round_to_storage=False)
    ref = torch.matmul(A.double(), q.double().transpose(-1, -2)).squeeze(-1)
    # an fp32 fma chain of r terms: error <= r * eps * sum|a_j q_j|
    bound = r * 2.0 ** -24 * torch.matmul(A.double().abs(), q.double().abs().transpose(-1, -2)).squeeze(-1)
    assert torch.all((s.double() - ref).abs() <= bound + 1e-30)


def test_scores_bf16_rounding_is_nearest_even(oracle):
    g = torch.Generator().manual_seed(5)
    A = torch.randn((1, 2, 1000, 32), generator=g).bfloat16()
    q = torch.randn((1, 2, 1, 32), generator=g).bfloat16()
    s32 = oracle.proxy_scores(A, q, round_to_storage=False)
    sbf = oracle.proxy_scores(A, q, round_to_storage=True)
    assert torch.equal(sbf, s32.bfloat16().float())  # torch's cast is RNE


def test_scores_exact_on_small_integers(oracle):
    # integer-valued inputs make every partial sum exact: any order gives the same bits
    g = torch.Generator().manual_seed(3)
    A = torch.randint(-8, 9, (1, 1, 64, 16), generator=g).float()
    q = torch.randint(-8, 9, (1, 1, 1, 16), generator=g).float()
    s = oracle.proxy_scores(A, q)
    assert torch.equal(s, torch.matmul(A, q.transpose(-1, -2)).squeeze(-1))
    # a transposed / shifted operand would fail this
    assert torch.equal(oracle.proxy_scores(A.bfloat16(), q.bfloat16(), False), s)


def test_negative_zero_is_canonical(oracle):
    A = torch.tensor([[[[-1.0, 0.0], [0.0, 0.0], [1.0, 0.0]]]])
    q = torch.tensor([[[[0.0, 1.0]]]])
    s = oracle.proxy_scores(A, q)
    assert not torch.signbit(s).any()


# ---------------------------------------------------------------- top-k

def _brute_topk(scores: np.ndarray, k: int) -> np.ndarray:
    idx = np.arange(scores.shape[0])
    order = np.lexsort((idx, -scores.astype(np.float64)))  # primary: score desc; secondary: idx asc
    return np.sort(order[:k])


@pytest.mark.parametrize("m,k", [(9, 8), (100, 8), (1000, 64), (5000, 512)])
def test_topk_vs_lexsort(oracle, m, k):
    g = torch.Generator().manual_seed(m)
    s = torch.randn((2, 2, m), generator=g)
    out = oracle.topk_sorted(s, k)
    for b in range(2):
        for h in range(2):
            assert np.array_equal(out[b, h, :, 0].numpy(), _brute_topk(s[b, h].numpy(), k))


def test_topk_ties_lowest_index(oracle):
    # all equal -> first k
    s = torch.zeros((1, 1, 300))
    assert torch.equal(oracle.topk_sorted(s, 64)[0, 0, :, 0], torch.arange(64))
    # two levels: 10 high values anywhere, the rest tied -> highs + lowest-index of the rest
    s = torch.ones((1, 1, 300))
    hi = torch.tensor([299, 250, 7, 100, 101, 102, 200, 201, 150, 5])
    s[0, 0, hi] = 2.0
    exp = sorted(set(hi.tolist()) | set([i for i in range(300) if i not in set(hi.tolist())][:54]))
    assert oracle.topk_sorted(s, 64)[0, 0, :, 0].tolist() == exp
    # heavy quantisation (bf16-like): compare with brute force
    g = torch.Generator().manual_seed(0)
    s = (torch.randn((1, 1, 4096), generator=g) * 4).round() / 4
    assert np.array_equal(oracle.topk_sorted(s, 512)[0, 0, :, 0].numpy(), _brute_topk(s[0, 0].numpy(), 512))


def test_topk_properties(oracle):
    g = torch.Generator().manual_seed(11)
    s = torch.randn((1, 3, 2000), generator=g).bfloat16().float()
    out = oracle.topk_sorted(s, 256)[..., 0]
    for h in range(3):
        sel = out[0, h]
        assert torch.all(sel[1:] > sel[:-1])  # strictly ascending, unique
        mask = torch.zeros(2000, dtype=torch.bool)
        mask[sel] = True
        assert s[0, h][mask].min() >= s[0, h][~mask].max()


def test_short_candidate_range_is_arange(oracle):
    A = torch.randn((2, 2, 5, 4))
    q = torch.randn((2, 2, 1, 4))
    out = oracle.compute_hit_indices(q, A, 8)
    assert out.shape == (2, 2, 5, 1) and torch.equal(out[1, 1, :, 0], torch.arange(5))
    out = oracle.compute_hit_indices(q, A, 5)
    assert torch.equal(out[0, 0, :, 0], torch.arange(5))


def test_negative_scores_order(oracle):
    s = torch.tensor([[[-3.0, -1.0, -2.0, -0.5, -4.0]]])
    assert oracle.topk_sorted(s, 2)[0, 0, :, 0].tolist() == [1, 3]
    s = torch.tensor([[[-3.0, 1.0, -2.0, 0.0, 4.0, -0.0]]])
    assert oracle.topk_sorted(s, 3)[0, 0, :, 0].tolist() == [1, 3, 4]
    # -0 and +0 are one value (as for torch.topk): the tie goes to the lower index
    s = torch.tensor([[[-0.0, 0.0, 0.0, -1.0]]])
    assert oracle.topk_sorted(s, 2)[0, 0, :, 0].tolist() == [0, 1]
    assert torch.topk(s[0, 0], 3).values.tolist() == [0.0, 0.0, 0.0]


# ---------------------------------------------------------------- diff

def test_diff_reference_docstring_vector(oracle):
    # lrqk_attention.py:1279-1290
    now = torch.tensor([0, 1, 2, 6, 7]).view(1, 1, 5, 1)
    new = torch.tensor([0, 2, 4, 5, 6]).view(1, 1, 5, 1)
    upd, mask = oracle.only_indices_in_cpu(now, new)
    assert upd.view(-1).tolist() == [0, 4, 2, 6, 5]
    assert mask.view(-1).int().tolist() == [0, 1, 0, 0, 1]


def test_diff_matches_torch_boolean_assignment(oracle):
    # the reference's five torch lines (:1305-1313) evaluated by stock torch on random sets
    g = torch.Generator().manual_seed(2)
    b, H, seq, k = 2, 8, 64, 16
    now = torch.stack([torch.randperm(seq, generator=g)[:k] for _ in range(b * H)]).view(b, H, k, 1)
    new = torch.stack([torch.randperm(seq, generator=g)[:k].sort().values for _ in range(b * H)]).view(b, H, k, 1)
    M = now.view(b, H, k, 1) == new.view(b, H, 1, k)
    now_in_new = ~M.any(dim=3)
    new_in_now = ~M.any(dim=2)
    exp = now.clone()
    exp[now_in_new] = new[new_in_now]
    upd, mask = oracle.only_indices_in_cpu(now, new)
    assert torch.equal(upd, exp) and torch.equal(mask, now_in_new)
    # set identities
    for i in range(b):
        for h in range(H):
            assert set(upd[i, h, :, 0].tolist()) == set(new[i, h, :, 0].tolist())
            keep = ~mask[i, h]
            assert torch.equal(upd[i, h, keep, 0], now[i, h, keep, 0])
            assert int(mask[i, h].sum()) == len(set(new[i, h, :, 0].tolist()) - set(now[i, h, :, 0].tolist()))


def test_diff_identical_and_disjoint(oracle):
    a = torch.arange(8).view(1, 1, 8, 1)
    upd, mask = oracle.only_indices_in_cpu(a, a.clone())
    assert torch.equal(upd, a) and not mask.any()
    upd, mask = oracle.only_indices_in_cpu(a, a + 8)
    assert torch.equal(upd, a + 8) and mask.all()


# ---------------------------------------------------------------- gathers

def test_d0_index_select_vs_torch_and_reference(oracle):
    # cpp_kernel/main_test.py:11-23, seeded
    g = torch.Generator().manual_seed(7)
    ref = _ref_module() if os.path.exists(REF_SO) else None
    for dtype in (torch.float32, torch.bfloat16):
        for _ in range(4):
            ndim = int(torch.randint(128, 513, (1,), generator=g))
            topk = int(torch.randint(10, 513, (1,), generator=g))
            src = torch.randn((6400, ndim), generator=g).to(dtype)
            idx = torch.randint(0, 6400, (topk,), generator=g)
            out = oracle.d0_index_select(src, idx)
            assert torch.equal(out, torch.index_select(src, 0, idx))
            if ref is not None:
                dst = torch.empty((topk, ndim), dtype=dtype)
                ref.d0_indices_select(dst, src, idx)
                assert torch.equal(out, dst)


def test_take_along_dim_with_mask_vs_reference_cpp(oracle):
    ref = _ref_module()
    g = torch.Generator().manual_seed(9)
    b, hkv, grp, seq, hd, k = 2, 8, 4, 32, 64, 8  # the shape of cpp_kernel/main_demo.py:150-152
    src = torch.randn((b, hkv, seq, hd), generator=g).to(torch.bfloat16)
    ind = torch.randint(0, seq, (b, hkv, grp, k), generator=g)
    mask = torch.rand((b, hkv, grp, k), generator=g) < 0.4
    exp = ref.take_along_dim_with_mask(src, ind, mask)
    out = oracle.take_along_dim_with_mask(src, ind, mask)
    assert torch.equal(out, exp)
    # and the two-stage route of lrqk_attention.py:101-117
    lin = oracle.linear_indices(hkv, seq, ind, mask)
    assert torch.equal(oracle.d0_index_select(src.view(-1, hd), lin), exp)


def test_take_along_dim_with_mask_bruteforce(oracle):
    # cpp_kernel/main_demo.py:186-194
    g = torch.Generator().manual_seed(10)
    b, hkv, grp, seq, hd, k = 2, 3, 2, 16, 8, 5
    src = torch.randn((b, hkv, seq, hd), generator=g)
    ind = torch.randint(0, seq, (b, hkv, grp, k), generator=g)
    mask = torch.rand((b, hkv, grp, k), generator=g) < 0.5
    out = oracle.take_along_dim_with_mask(src, ind, mask)
    full = torch.zeros((b, hkv, grp, k, hd))
    full[mask] = out
    for i in range(b):
        for j in range(hkv):
            for c in range(grp):
                for m in range(k):
                    if mask[i, j, c, m]:
                        assert torch.equal(full[i, j, c, m], src[i, j, ind[i, j, c, m]])
                    else:
                        assert full[i, j, c, m].abs().sum() == 0


# ---------------------------------------------------------------- buffers (lrqk_attention_test.py:10-66)

def test_auto_increase_len_and_getitem(oracle):
    g = torch.Generator().manual_seed(4)
    t = oracle.OracleAutoIncreaseTensor(capacity=16, dim=0)
    ref = torch.empty((0, 8))
    for _ in range(30):
        n = int(torch.randint(1, 20, (1,), generator=g))
        x = torch.randn((n, 8), generator=g)
        t.append(x)
        ref = torch.cat([ref, x])
        assert len(t) == ref.shape[0]
        assert torch.equal(t[:], ref)
        assert t.capacity > len(t)
        assert t.data[len(t):].abs().sum() == 0  # zero-initialised tail


def test_auto_increase_dim2_growth(oracle):
    t = oracle.OracleAutoIncreaseTensor(capacity=4, dim=2)
    x = torch.randn(2, 8, 10, 128)
    t.append(x)
    assert t.capacity == 15 and t.shape == (2, 8, 10, 128)
    y = torch.randn(2, 8, 7, 128)
    t.append(y)
    assert t.capacity == 22 and torch.equal(t.tensor(), torch.cat([x, y], 2))
    assert t.data[:, :, 17:].abs().sum() == 0
