#!/usr/bin/env python3
"""Writes the fixtures in this folder (run from the repository root: python tests/golden/make_golden.py).

Everything is produced by the CPU oracle from fixed CPU seeds; nothing is read from the
reference tree at run time.  The one vector the reference itself holds -- the hit/miss diff
example in the docstring of only_indices_in_cpu (lrqk_attention.py:1279-1290) -- is typed in
below as data.

  diff_docstring.npz  now/new -> updated/evict of the reference's own example
  topk_ties.npz       tie-heavy score rows and the ids the order (score desc, index asc) selects
  trace_small.npz     b=2, Hq=4, Hkv=2, d=16, r=4, k=8, L=4: prompt of 24 tokens + 40 decode
                      steps; per step the factor outputs, candidate count, selected ids,
                      resident ids after the diff, evict mask, active K/V and attention output
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import lrqk_oracle as orc  # noqa: E402


def diff_docstring():
    now = np.array([0, 1, 2, 6, 7], dtype=np.int64)
    new = np.array([0, 2, 4, 5, 6], dtype=np.int64)
    updated = np.array([0, 4, 2, 6, 5], dtype=np.int64)
    evict = np.array([0, 1, 0, 0, 1], dtype=np.uint8)
    np.savez(os.path.join(HERE, "diff_docstring.npz"), now=now, new=new, updated=updated, evict=evict)


def topk_ties():
    g = torch.Generator().manual_seed(11)
    cases = {}
    # all scores equal: the k lowest ids
    cases["all_equal"] = (torch.full((1000,), 0.5), 100)
    # two levels, the upper one smaller than k: all of it + the lowest ids of the lower one
    s = torch.zeros(1000)
    s[torch.randperm(1000, generator=g)[:37]] = 1.0
    cases["two_level"] = (s, 100)
    # distinct top part, then a tie at the k-th place that spans several 64-lane groups
    s = -torch.rand(2000, generator=g)
    top = torch.randperm(2000, generator=g)
    s[top[:60]] = 1.0 + torch.rand(60, generator=g)
    s[top[60:360]] = 0.75
    cases["boundary_tie"] = (s, 128)
    # signed zeros compare equal; a NaN-free mix of negative values
    s = torch.zeros(300)
    s[::2] = -0.0
    s[5] = -1.0
    cases["signed_zero"] = (s, 64)
    # m <= k
    cases["short_row"] = (torch.rand(20, generator=g), 64)
    out = {}
    for name, (sc, k) in cases.items():
        idx = orc.topk_sorted(sc.view(1, 1, -1), k).view(-1).numpy()
        out[name + "_scores"] = sc.numpy().astype(np.float32)
        out[name + "_k"] = np.int64(k)
        out[name + "_idx"] = idx.astype(np.int64)
    np.savez(os.path.join(HERE, "topk_ties.npz"), **out)


def trace_small():
    b, hq, hkv, d, r, k, L, l, steps = 2, 4, 2, 16, 4, 8, 4, 24, 40
    g = torch.Generator().manual_seed(2024)
    rho = 3

    def lowrank(n, heads):
        U = torch.randn((b, heads, n, rho), generator=g) / rho ** 0.25
        W = torch.randn((b, heads, rho, d), generator=g) / rho ** 0.25
        return U @ W + 0.05 * torch.randn((b, heads, n, d), generator=g)

    Q, K, V = lowrank(l, hq), lowrank(l, hkv), torch.randn((b, hkv, l, d), generator=g)
    A_Q0 = torch.randn((b, hq, l, r), generator=g)
    A_K0 = torch.randn((b, hq, l, r), generator=g)
    eng = orc.OracleLayer(num_lite_tokens=L, attn_topk=k, num_key_value_groups=hq // hkv, r=r, max_iter=(2, 2),
                          tol=(1e-8, 1e-8), capacity=16, compute_dtype=torch.float64)
    eng.prefill(Q, K, V, A_Q0=A_Q0, A_K0=A_K0)
    rec = {n: [] for n in ("q", "k", "v", "B_Q_in", "B_K_in", "A_act_in", "K_prev", "B_Q", "B_K", "q_hat", "k_hat",
                           "m", "new_idx", "hit_before", "hit_after", "evict", "Kact", "Vact", "attn")}
    out = dict(Q=Q, K=K, V=V, A_Q0=A_Q0, A_K0=A_K0, prefill_B_Q=eng.B_Q.clone(), prefill_B_K=eng.B_K.clone(),
               prefill_A_K=eng.A_K.clone(), prefill_hit=eng.hit_indices.clone())
    for _ in range(steps):
        q, kn, vn = lowrank(1, hq), lowrank(1, hkv), torch.randn((b, hkv, 1, d), generator=g)
        rec["q"].append(q); rec["k"].append(kn); rec["v"].append(vn)
        rec["B_Q_in"].append(eng.B_Q.clone()); rec["B_K_in"].append(eng.B_K.clone())
        rec["hit_before"].append(eng.hit_indices.clone())
        B_Q, B_K, hq_, hk_ = eng.begin_decode(q, kn, vn)
        rec["A_act_in"].append(eng._A_K_hitted_with_lite().clone())
        rec["K_prev"].append(eng.Kgpu.clone())
        Ko, Vo = eng.finish_decode(B_Q, B_K, hq_, hk_)
        rec["B_Q"].append(B_Q.clone()); rec["B_K"].append(B_K.clone())
        rec["q_hat"].append(hq_.clone()); rec["k_hat"].append(hk_.clone())
        rec["m"].append(torch.tensor(eng.last_m))
        rec["new_idx"].append(eng.last_new_indices.clone())
        rec["hit_after"].append(eng.hit_indices.clone())
        rec["evict"].append(eng.last_evict.to(torch.uint8))
        rec["Kact"].append(Ko.clone()); rec["Vact"].append(Vo.clone())
        rec["attn"].append(orc.attention(q, Ko, Vo, torch.float64).to(torch.float32))
    for n, v in rec.items():
        out["step_" + n] = torch.stack(v)
    out["final_A_K"] = eng.A_K.clone()
    out["final_store"] = eng.KVcpu.tensor().clone()
    out["final_lite_indices"] = torch.tensor(eng.lite_indices)
    np.savez_compressed(os.path.join(HERE, "trace_small.npz"), **{n: v.numpy() for n, v in out.items()},
                        shape=np.array([b, hq, hkv, d, r, k, L, l, steps], dtype=np.int64))


if __name__ == "__main__":
    diff_docstring()
    topk_ties()
    trace_small()
    for f in sorted(os.listdir(HERE)):
        print(f, os.path.getsize(os.path.join(HERE, f)))
