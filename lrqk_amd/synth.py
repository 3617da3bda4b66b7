"""Seeded synthetic inputs of the benchmark configurations.

Everything is drawn on the CPU from ``torch.Generator().manual_seed(seed)`` so the same
numbers reach the CPU checker and the GPU.  The low-rank + noise generator is
``X = U W + sigma E`` per (batch, head) with ``U [l,rho]``, ``W [rho,d]`` entries of standard
deviation ``rho ** -0.25`` each (so that an entry of ``U W`` has unit variance) and
``E ~ N(0,1)``.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Tuple

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    num_heads: int
    num_kv_heads: int
    head_dim: int
    batch: int
    dtype: torch.dtype
    context: int
    r: int
    num_active_tokens: int
    lite_tokens: int
    max_iter: Tuple[int, int]
    tol: Tuple[float, float]
    decode_steps: int
    rho: int = 32
    sigma: float = 0.01

    @property
    def groups(self) -> int:
        return self.num_heads // self.num_kv_heads


WORKLOADS = {
    # Qwen2.5-7B attention shape, fp32, the CPU-runnable case.
    "qwen7b_4k_fp32": Workload("qwen7b_4k_fp32", 28, 4, 128, 1, torch.float32, 4096, 16, 512, 32,
                               (1, 1), (1e-2, 1e-2), 64),
    # Llama-3-8B attention shape, bf16.
    "llama8b_32k_bf16": Workload("llama8b_32k_bf16", 32, 8, 128, 1, torch.bfloat16, 32768, 32, 2048, 64,
                                 (2, 2), (1e-2, 1e-2), 256),
    "llama8b_128k_bf16": Workload("llama8b_128k_bf16", 32, 8, 128, 1, torch.bfloat16, 131072, 32, 2048, 64,
                                  (2, 2), (1e-2, 1e-2), 512),
    # prefill factorisation only
    "llama8b_32k_prefill_als": Workload("llama8b_32k_prefill_als", 32, 8, 128, 1, torch.bfloat16, 32768, 32,
                                        2048, 64, (4, 4), (1e-8, 1e-8), 0, rho=48, sigma=0.05),
    # small shape for unit tests
    "tiny": Workload("tiny", 4, 2, 16, 2, torch.float32, 40, 4, 8, 4, (2, 2), (1e-8, 1e-8), 40, rho=4),
}


def low_rank_noise(gen: torch.Generator, b: int, h: int, l: int, d: int, rho: int, sigma: float,
                   dtype: torch.dtype = torch.float32, W: torch.Tensor = None):
    """Returns (X [b,h,l,d] in ``dtype``, W [b,h,rho,d] fp32).  Pass ``W`` to draw more rows
    from the same subspace (new decode tokens)."""
    std = rho ** -0.25
    dev = gen.device
    if W is None:
        W = torch.randn((b, h, rho, d), generator=gen, device=dev) * std
    out = torch.empty((b, h, l, d), dtype=dtype, device=dev)
    step = 16384
    for s in range(0, l, step):
        e = min(l, s + step)
        U = torch.randn((b, h, e - s, rho), generator=gen, device=dev) * std
        X = torch.matmul(U, W)
        if sigma:
            X = X + sigma * torch.randn((b, h, e - s, d), generator=gen, device=dev)
        out[:, :, s:e] = X.to(dtype)
    return out, W


def prompt_qkv(w: Workload, seed: int = 0, context: int = None, device="cpu"):
    """Q [b,Hq,l,d], K,V [b,Hkv,l,d] in the workload dtype, and the subspace bases so decode
    tokens can follow the same statistics.  ``device`` selects where the numbers are drawn
    (the CPU stream is the portable one; a GPU draw is only reproducible on that GPU type)."""
    gen = torch.Generator(device=device).manual_seed(seed)
    l = context or w.context
    Q, WQ = low_rank_noise(gen, w.batch, w.num_heads, l, w.head_dim, w.rho, w.sigma, w.dtype)
    K, WK = low_rank_noise(gen, w.batch, w.num_kv_heads, l, w.head_dim, w.rho, w.sigma, w.dtype)
    V, WV = low_rank_noise(gen, w.batch, w.num_kv_heads, l, w.head_dim, w.rho, w.sigma, w.dtype)
    return Q, K, V, (WQ, WK, WV), gen


def rotate_query(gen: torch.Generator, q: torch.Tensor, angle_std: float = 0.05, n_rot: int = None):
    """q_{t+1} = R_t q_t, R_t a product of Givens rotations on disjoint random coordinate
    pairs with angles ~ N(0, angle_std).  q fp32 [b,H,1,d]."""
    b, H, _, d = q.shape
    n_rot = n_rot or d // 2
    dev = gen.device
    perm = torch.randperm(d, generator=gen, device=dev)
    i, j = perm[0:2 * n_rot:2], perm[1:2 * n_rot:2]
    th = torch.randn((b, H, 1, n_rot), generator=gen, device=dev) * angle_std
    c, s = torch.cos(th), torch.sin(th)
    out = q.clone()
    qi, qj = q[..., i], q[..., j]
    out[..., i] = c * qi - s * qj
    out[..., j] = s * qi + c * qj
    return out


class DecodeStream:
    """Per-step (q,k,v) of a decode run: queries drift by small rotations from the last
    prompt query, new keys/values come from the prompt's subspaces."""

    def __init__(self, w: Workload, Q_last: torch.Tensor, bases, gen: torch.Generator):
        self.w = w
        self.q = Q_last.float().clone()  # [b,Hq,1,d]
        self.WQ, self.WK, self.WV = bases
        self.gen = gen

    def next(self):
        w = self.w
        self.q = rotate_query(self.gen, self.q)
        k, _ = low_rank_noise(self.gen, w.batch, w.num_kv_heads, 1, w.head_dim, w.rho, w.sigma, w.dtype, self.WK)
        v, _ = low_rank_noise(self.gen, w.batch, w.num_kv_heads, 1, w.head_dim, w.rho, w.sigma, w.dtype, self.WV)
        return self.q.to(w.dtype), k, v


def init_factors(w: Workload, l: int, seed: int = 1, device="cpu"):
    """Injected A_Q0, A_K0 (the ``randn`` initialiser with a fixed seed): fp32 [b,Hq,l,r]."""
    gen = torch.Generator(device=device).manual_seed(seed)
    A_Q0 = torch.randn((w.batch, w.num_heads, l, w.r), generator=gen, device=device)
    A_K0 = torch.randn((w.batch, w.num_heads, l, w.r), generator=gen, device=device)
    return A_Q0, A_K0
