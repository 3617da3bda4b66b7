"""CPU oracle for the LRQK per-layer prefill / decode path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this module; it is
the checker the HIP path is compared against (tests, the smoke check) and the code the
CPU baseline times.  It restates the reference's algorithm op for op with torch CPU
tensors; the bit-exact stages (proxy score, top-k order, hit/miss diff, row gather) are
delegated to the plain-C restatement in ``lrqk_oracle.c`` so that the floating-point
summation order is fixed (an ``fmaf`` chain).

Every function cites the reference lines it follows (paths relative to the reference
tree, all in ``lrqk_attention.py`` unless another file is named).

What pins each function (see tests/test_oracle_*.py):
  als_prefill_w1   normal-equation orthogonality, monotone objective, exact-rank
                   recovery, max_iter=0 == numpy lstsq
  als_decode_w1    k_hat_0 == lstsq, every half-step solves its stated r x r system,
                   the B step is the exact line-search minimiser
  proxy scores     fp64 dot products (tolerance) ; top-k: brute-force numpy lexsort
  only_indices_in_cpu  the reference's docstring vector (:1279-1290) + set identities
  gathers          the reference's own compiled C++ (oracle/_ref) and numpy indexing
  attention        torch.nn.functional.scaled_dot_product_attention on CPU
  OracleAutoIncreaseTensor  the four behaviours of lrqk_attention_test.py:10-66
  OracleLayer      the hand-derived ring trace (l=10, L=3) and the dense-attention
                   identity when k+L covers the context
"""
from __future__ import annotations

import ctypes
import enum
import os
from typing import Optional, Tuple

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liblrqk_oracle.so")
_lib = None


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                f"{_LIB_PATH} is not built; run `make -C {_HERE}` (or __graft_entry__.build())")
        lib = ctypes.CDLL(_LIB_PATH)
        i64, i32, vp = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p
        lib.oracle_proxy_scores.argtypes = [vp, vp, i64, i32, i32, i32, vp]
        lib.oracle_proxy_scores.restype = i32
        lib.oracle_topk_sorted.argtypes = [vp, i64, i64, vp]
        lib.oracle_topk_sorted.restype = i64
        lib.oracle_only_indices.argtypes = [vp, vp, i64, vp, vp]
        lib.oracle_only_indices.restype = i64
        lib.oracle_linear_indices.argtypes = [vp, vp, i64, i64, i64, i64, i64, vp]
        lib.oracle_linear_indices.restype = i64
        lib.oracle_d0_indices_select.argtypes = [vp, vp, vp, i64, i64]
        lib.oracle_d0_indices_select.restype = None
        lib.oracle_take_along_dim_with_mask.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, vp]
        lib.oracle_take_along_dim_with_mask.restype = i64
        _lib = lib
    return _lib


def _dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return 0
    if dt == torch.bfloat16:
        return 1
    raise ValueError(f"unsupported storage dtype {dt}")


# --------------------------------------------------------------------------- helpers

def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """:36-39 -> transformers repeat_kv: [b,Hkv,s,d] -> [b,Hkv*n_rep,s,d], head h reads h//n_rep."""
    b, hkv, s, d = x.shape
    if n_rep == 1:
        return x
    return x[:, :, None, :, :].expand(b, hkv, n_rep, s, d).reshape(b, hkv * n_rep, s, d)


def ensure_tuple2(x):
    """:42-47"""
    if isinstance(x, (tuple, list)):
        assert len(x) == 2, "must be a tuple or list of length 2"
        return tuple(x)
    return (x, x)


class InitAQAK(enum.Enum):
    """:140-143"""
    randn = enum.auto()
    top = enum.auto()
    topcol = enum.auto()


def init_aq_ak(Q, K, r, method=InitAQAK.randn, generator: Optional[torch.Generator] = None):
    """:145-209.  ``randn`` draws from a CPU generator (the reference uses the device RNG,
    which no other device can reproduce; callers that need parity inject A_Q0/A_K0)."""
    if isinstance(method, str):
        if method not in InitAQAK.__members__:
            raise ValueError(f"Unknown init_method: {method}")
        method = InitAQAK[method]
    b, h, l, d = Q.shape
    if method == InitAQAK.randn:
        AQ = torch.randn((b, h, l, r), dtype=Q.dtype, generator=generator)
        AK = torch.randn((b, h, l, r), dtype=K.dtype, generator=generator)
        return AQ, AK
    qs = Q.abs().sum(dim=2, keepdim=True)
    ks = K.abs().sum(dim=2, keepdim=True)
    if method == InitAQAK.topcol:
        idx = torch.topk(qs + ks, k=r, dim=-1).indices
        iq = ik = idx
    elif method == InitAQAK.top:
        iq = torch.topk(qs, k=r, dim=-1).indices
        ik = torch.topk(ks, k=r, dim=-1).indices
    else:
        raise ValueError(f"Unknown init_method: {method}")
    AQ = torch.gather(Q, -1, iq.expand(-1, -1, l, -1))
    AK = torch.gather(K, -1, ik.expand(-1, -1, l, -1))
    return AQ, AK


def _solve(A, B, left=True):
    return torch.linalg.solve(A, B, left=left)


def _T(x):
    return x.transpose(-1, -2)


# --------------------------------------------------------------------------- ALS prefill

def als_prefill_w1(Q, K, A_Q, A_K, max_iter=8, tol=1e-5, trace=None):
    """:319-423 (_lrqk_prefill_inv_w1).  All tensors [b,H,*,*] in one compute dtype.
    Gauss-Seidel: the A_K update already uses the new A_Q (:385,:387).  ``delta`` is the
    max of two batch-wide MSEs and the loop breaks for the whole batch at once (:398-413).
    ``trace`` (a list) receives the objective after each block update when given."""
    mm = torch.matmul

    def objective(AQ, BQ, AK, BK):
        # f = 1/2|QK^T - AQ AK^T|^2 + 1/2|Q - AQ BQ|^2 + 1/2|K - AK BK|^2 without forming QK^T:
        # |QK^T - AQ AK^T|^2 = tr(Q^TQ K^TK) - 2 tr(Q^TAQ AK^TK) + tr(AQ^TAQ AK^TAK)
        t1 = (mm(_T(Q), Q) * mm(_T(K), K)).sum(dim=(-1, -2))
        t2 = (mm(_T(Q), AQ) * mm(_T(K), AK)).sum(dim=(-1, -2))
        t3 = (mm(_T(AQ), AQ) * mm(_T(AK), AK)).sum(dim=(-1, -2))
        f = 0.5 * (t1 - 2 * t2 + t3)
        f = f + 0.5 * (Q - mm(AQ, BQ)).square().sum(dim=(-1, -2))
        f = f + 0.5 * (K - mm(AK, BK)).square().sum(dim=(-1, -2))
        return f

    for _ in range(max_iter):
        AQTAQ = mm(_T(A_Q), A_Q)
        AKTAK = mm(_T(A_K), A_K)
        B_Q = _solve(AQTAQ, mm(_T(A_Q), Q))
        B_K = _solve(AKTAK, mm(_T(A_K), K))
        if trace is not None:
            trace.append(("B", objective(A_Q, B_Q, A_K, B_K)))

        BQBQT = mm(B_Q, _T(B_Q))
        RHS_Q = mm(_T(K), A_K) + _T(B_Q)
        new_A_Q = mm(Q, _solve(AKTAK + BQBQT, RHS_Q, left=False))
        if trace is not None:
            trace.append(("AQ", objective(new_A_Q, B_Q, A_K, B_K)))

        AQTAQ = mm(_T(new_A_Q), new_A_Q)
        BKBKT = mm(B_K, _T(B_K))
        RHS_K = mm(_T(Q), new_A_Q) + _T(B_K)
        new_A_K = mm(K, _solve(AQTAQ + BKBKT, RHS_K, left=False))
        if trace is not None:
            trace.append(("AK", objective(new_A_Q, B_Q, new_A_K, B_K)))

        delta = max(torch.mean((A_Q - new_A_Q) ** 2), torch.mean((A_K - new_A_K) ** 2))
        A_Q, A_K = new_A_Q, new_A_K
        if delta < tol:
            break

    AQTAQ = mm(_T(A_Q), A_Q)
    AKTAK = mm(_T(A_K), A_K)
    B_Q = _solve(AQTAQ, mm(_T(A_Q), Q))
    B_K = _solve(AKTAK, mm(_T(A_K), K))
    if trace is not None:
        trace.append(("Bfinal", objective(A_Q, B_Q, A_K, B_K)))
    return A_Q, B_Q, A_K, B_K


def cast_lrqk_prefill(Q, K, r, max_iter=8, tol=1e-5, init_method=InitAQAK.randn,
                      A_Q0=None, A_K0=None, generator=None, compute_dtype=torch.float32):
    """:772-800.  Upcast to the compute dtype (fp32 in the reference), run the w1 variant
    (the only reachable one, :790 with weights fixed at 1), cast back to K.dtype."""
    out_dtype = K.dtype
    Qc, Kc = Q.to(compute_dtype), K.to(compute_dtype)
    if A_Q0 is None or A_K0 is None:
        A_Q0, A_K0 = init_aq_ak(Qc, Kc, r, init_method, generator)
    out = als_prefill_w1(Qc, Kc, A_Q0.to(compute_dtype), A_K0.to(compute_dtype), max_iter, tol)
    return tuple(o.to(out_dtype) for o in out)


# --------------------------------------------------------------------------- ALS decode

def gd_B_lr(dB, hat, epsilon=1e-6):
    """:651-665"""
    dB_norm = dB.square().sum(dim=(2, 3), keepdim=True)
    hat_dB = torch.matmul(hat, dB)
    return dB_norm / (hat_dB.square().sum(dim=(2, 3), keepdim=True) + epsilon)


def als_decode_w1(B_Q, A_K, B_K, K__, q, k, max_iter=2, tol=1e-3, trace=None):
    """:529-628 (_lrqk_decode_inv_w1).  Shapes: B_* [b,H,r,d], A_K [b,H,n,r], K__ [b,H,n,d],
    q,k [b,H,1,d].  The convergence test is one MSE over the whole batch (:603-609)."""
    mm = torch.matmul
    max_iter = max(max_iter, 1)
    ktBKT = mm(k, _T(B_K))
    BKBKT = mm(B_K, _T(B_K))
    rhs_q = mm(q, _T(B_Q)) + mm(mm(q, _T(K__)), A_K)
    G_Q = mm(B_Q, _T(B_Q)) + mm(_T(A_K), A_K)
    s = mm(q, _T(k))
    hat_k = _solve(BKBKT, ktBKT, left=False)
    if trace is not None:
        trace.append(("k0", hat_k.clone()))
    hat_q = None
    for _ in range(max_iter):
        hat_q = _solve(G_Q + mm(_T(hat_k), hat_k), rhs_q + mm(s, hat_k), left=False)
        new_hat_k = _solve(BKBKT + mm(_T(hat_q), hat_q), ktBKT + mm(s, hat_q), left=False)
        if trace is not None:
            trace.append(("iter", hat_k.clone(), hat_q.clone(), new_hat_k.clone()))
        delta = torch.mean((hat_k - new_hat_k) ** 2)
        hat_k = new_hat_k
        if delta < tol:
            break
    dBQ = mm(_T(hat_q), mm(hat_q, B_Q) - q)
    dBK = mm(_T(hat_k), mm(hat_k, B_K) - k)
    B_Q = B_Q - gd_B_lr(dBQ, hat_q) * dBQ
    B_K = B_K - gd_B_lr(dBK, hat_k) * dBK
    return B_Q, B_K, hat_q, hat_k


def cast_lrqk_decode(B_Q, A_K, B_K, K__, q, k, max_iter=8, tol=1e-5, compute_dtype=torch.float32):
    """:803-839"""
    out_dtype = k.dtype
    c = compute_dtype
    out = als_decode_w1(B_Q.to(c), A_K.to(c), B_K.to(c), K__.to(c), q.to(c), k.to(c), max_iter, tol)
    return tuple(o.to(out_dtype) for o in out)


# --------------------------------------------------------------------------- selection

_THREADS = 1


def set_threads(n: int):
    """Heads are independent: run the per-head C calls on ``n`` threads (ctypes drops the GIL)."""
    global _THREADS
    _THREADS = max(1, int(n))


def _per_head(fn, count):
    if _THREADS == 1 or count == 1:
        for i in range(count):
            fn(i)
        return
    from concurrent.futures import ThreadPoolExecutor
    with ThreadPoolExecutor(max_workers=min(_THREADS, count)) as ex:
        list(ex.map(fn, range(count)))


def proxy_scores(A_K_m: torch.Tensor, q_hat: torch.Tensor, round_to_storage: bool = True) -> torch.Tensor:
    """:1260-1263.  A_K_m [b,H,m,r], q_hat [b,H,1,r] in the storage dtype -> fp32 [b,H,m].
    fp32 fmaf chain over j; with bf16 storage and round_to_storage the result is rounded to
    bf16 (what the reference's bf16 matmul returns)."""
    lib = _load()
    b, H, m, r = A_K_m.shape
    code = _dtype_code(A_K_m.dtype)
    A = A_K_m
    if A.stride(3) != 1 or A.stride(2) != r:   # rows must be contiguous; heads may be strided views
        A = A.contiguous()
    qh = q_hat.contiguous()
    out = torch.empty((b, H, m), dtype=torch.float32)
    esz = A.element_size()
    rb = 1 if (round_to_storage and code == 1) else 0
    sb, sh = A.stride(0), A.stride(1)

    def one(i):
        off = (i // H) * sb + (i % H) * sh
        rc = lib.oracle_proxy_scores(A.data_ptr() + off * esz, qh.data_ptr() + i * r * esz,
                                     m, r, code, rb, out.data_ptr() + i * m * 4)
        if rc != 0:
            raise RuntimeError(f"oracle_proxy_scores failed: {rc}")

    _per_head(one, b * H)
    return out


def topk_sorted(scores: torch.Tensor, k: int) -> torch.Tensor:
    """:1266-1273 under the stated order (score desc, index asc).  scores fp32 [b,H,m] ->
    int64 [b,H,min(k,m),1] ascending."""
    lib = _load()
    b, H, m = scores.shape
    kk = min(k, m)
    sc = scores.contiguous()
    out = torch.empty((b, H, kk), dtype=torch.int32)
    def one(i):
        n = lib.oracle_topk_sorted(sc.data_ptr() + i * m * 4, m, k, out.data_ptr() + i * kk * 4)
        if n != kk:
            raise RuntimeError("oracle_topk_sorted failed")

    _per_head(one, b * H)
    return out.to(torch.int64).unsqueeze(-1)


def compute_hit_indices(q_hat, A_K_m, attn_topk, round_to_storage=True) -> torch.Tensor:
    """:1235-1273"""
    b, H, m, _ = A_K_m.shape
    if m <= attn_topk:
        return torch.arange(m, dtype=torch.int64).reshape(1, 1, -1, 1).expand(b, H, -1, 1).contiguous()
    return topk_sorted(proxy_scores(A_K_m, q_hat, round_to_storage), attn_topk)


def only_indices_in_cpu(now: torch.Tensor, new: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """:1275-1315.  now,new int64 [b,H,k,1] -> (updated [b,H,k,1] int64, evict mask [b,H,k] bool)."""
    lib = _load()
    b, H, k, _ = now.shape
    a = now.reshape(b * H, k).to(torch.int32).contiguous()
    c = new.reshape(b * H, k).to(torch.int32).contiguous()
    upd = torch.empty_like(a)
    ev = torch.empty((b * H, k), dtype=torch.uint8)
    def one(i):
        n = lib.oracle_only_indices(a.data_ptr() + i * k * 4, c.data_ptr() + i * k * 4, k,
                                    upd.data_ptr() + i * k * 4, ev.data_ptr() + i * k)
        if n < 0:
            raise RuntimeError("shape mismatch: evicted and missing counts differ")

    _per_head(one, b * H)
    return upd.to(torch.int64).reshape(b, H, k, 1), ev.bool().reshape(b, H, k)


def linear_indices(kv_heads: int, seq_len: int, indices: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
    """:78-98.  indices,mask [b,Hkv,g,k] -> int64 [n_true]."""
    lib = _load()
    b, hkv, g, k = indices.shape
    assert hkv == kv_heads
    ind = indices.to(torch.int32).contiguous()
    mk = mask.to(torch.uint8).contiguous()
    out = torch.empty(int(mk.sum()), dtype=torch.int64)
    n = lib.oracle_linear_indices(ind.data_ptr(), mk.data_ptr(), b, hkv, g, k, seq_len, out.data_ptr())
    assert n == out.numel()
    return out


def d0_index_select(src: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    """cpp_kernel/__init__.py:7-16 + take_along_dim_grouped.cpp:133-183.  src [N,w], idx int64 [n]."""
    lib = _load()
    src = src.contiguous()
    idx = idx.to(torch.int64).contiguous()
    out = torch.empty((idx.numel(), src.shape[1]), dtype=src.dtype)
    lib.oracle_d0_indices_select(out.data_ptr(), src.data_ptr(), idx.data_ptr(), idx.numel(),
                                 src.shape[1] * src.element_size())
    return out


def take_along_dim_with_mask(src: torch.Tensor, indices: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
    """:101-117 and take_along_dim_grouped.cpp:13-124.  src [b,Hkv,seq,w]; indices,mask [b,Hkv,g,k]."""
    lib = _load()
    b, hkv, seq, w = src.shape
    _, _, g, k = indices.shape
    src = src.contiguous()
    ind = indices.to(torch.int32).contiguous()
    mk = mask.to(torch.uint8).contiguous()
    out = torch.empty((int(mk.sum()), w), dtype=src.dtype)
    n = lib.oracle_take_along_dim_with_mask(src.data_ptr(), ind.data_ptr(), mk.data_ptr(), b, hkv, g, k,
                                            seq, w * src.element_size(), out.data_ptr())
    assert n == out.shape[0]
    return out


# --------------------------------------------------------------------------- attention

def attention(q: torch.Tensor, K: torch.Tensor, V: torch.Tensor, compute_dtype=torch.float64) -> torch.Tensor:
    """Call sites :2326-2327 (flash_attn_with_kvcache(q,k,v,causal=True) with ONE query: the
    causal mask removes nothing), scale 1/sqrt(d).  q [b,H,1,d], K,V [b,H,n,d] -> [b,H,1,d]
    in the compute dtype (textbook softmax)."""
    d = q.shape[-1]
    qc, Kc, Vc = q.to(compute_dtype), K.to(compute_dtype), V.to(compute_dtype)
    s = torch.matmul(qc, _T(Kc)) / (d ** 0.5)
    p = torch.softmax(s, dim=-1)
    return torch.matmul(p, Vc)


# --------------------------------------------------------------------------- buffers

class OracleAutoIncreaseTensor:
    """:844-957.  Zero-initialised buffer growing by ``scaling_ratio`` along ``dim``."""

    def __init__(self, capacity=4096, dim=0, scaling_ratio=1.5, dtype=None):
        self.capacity = capacity
        self.dim = dim
        self.scaling_ratio = scaling_ratio
        self.dtype = dtype
        self.data: Optional[torch.Tensor] = None
        self.current_len = 0

    def append(self, x: torch.Tensor):
        if self.dtype is None:
            self.dtype = x.dtype
        length = x.size(self.dim)
        target = self.current_len + length
        if self.data is None:
            init_cap = max(self.capacity, int(length * self.scaling_ratio))
            shape = list(x.shape)
            shape[self.dim] = init_cap
            self.data = torch.zeros(shape, dtype=self.dtype)
            self.capacity = init_cap
        elif target >= self.capacity:
            new_cap = self.capacity
            while new_cap <= target:
                new_cap = int(new_cap * self.scaling_ratio)
            shape = list(self.data.shape)
            shape[self.dim] = new_cap
            new = torch.zeros(shape, dtype=self.dtype)
            new.narrow(self.dim, 0, self.current_len).copy_(self.data.narrow(self.dim, 0, self.current_len))
            self.data = new
            self.capacity = new_cap
        self.data.narrow(self.dim, self.current_len, length).copy_(x.to(self.dtype))
        self.current_len += length

    def tensor(self):
        return self.data.narrow(self.dim, 0, self.current_len)

    def __len__(self):
        return self.current_len

    def __getitem__(self, idx):
        if self.data is None:
            raise IndexError("Cache is empty")
        return self.tensor()[idx]

    @property
    def shape(self):
        s = list(self.data.shape)
        s[self.dim] = self.current_len
        return torch.Size(s)


# --------------------------------------------------------------------------- the layer engine

class OracleLayer:
    """:1031-1613 (LightAttentionIndicesFactory) on CPU tensors.

    ``compute_dtype`` is the dtype of the ALS arithmetic (fp32 in the reference, fp64 to
    act as ground truth); state is kept in the storage dtype of the inputs (Q4)."""

    def __init__(self, num_lite_tokens=1, attn_topk=128, num_key_value_groups=1, r=16, max_iter=2,
                 tol=1e-4, capacity=4096, init_aq_ak_method=InitAQAK.randn, scaling_ratio=1.5,
                 compute_dtype=torch.float32, round_scores_to_storage=True, no_hit_miss=False):
        self.L = num_lite_tokens
        self.k = attn_topk
        self.g = num_key_value_groups
        self.r = r
        self.max_iter = ensure_tuple2(max_iter)
        self.tol = ensure_tuple2(tol)
        self.init = init_aq_ak_method
        self.n = attn_topk + num_lite_tokens
        self.compute_dtype = compute_dtype
        self.round_scores = round_scores_to_storage
        self.no_hit_miss = no_hit_miss
        self.prefill_length = 0
        self.current_len = 0
        self.B_Q = None
        self.B_K = None
        self._A_K = OracleAutoIncreaseTensor(capacity, 2, scaling_ratio)
        self.KVcpu = OracleAutoIncreaseTensor(capacity, 2, scaling_ratio)
        self.Kgpu = None
        self.Vgpu = None
        self.lite_len = 0
        self.lite_indices = [-1] * self.L
        self.hit_indices = None
        # per-step diagnostics
        self.last_q_hat = None
        self.last_k_hat = None
        self.last_new_indices = None
        self.last_evict = None
        self.last_m = None

    def __len__(self):
        return self.current_len

    @property
    def A_K(self):
        return self._A_K.tensor()

    def _lite(self, src):
        """:1124-1131"""
        return src[:, 0:src.shape[1]:self.g, self.k:self.k + self.L, :]

    def _kv_append(self, k, v):
        """:959-963"""
        self.KVcpu.append(torch.cat([k, v], dim=-1))

    def _append(self, k, v):
        """:1174-1196"""
        s = self.k + self.lite_len
        self.Kgpu[:, :, s:s + 1, :] = repeat_kv(k, self.g)
        self.Vgpu[:, :, s:s + 1, :] = repeat_kv(v, self.g)
        self.lite_indices[self.lite_len] = self.current_len
        self.lite_len += 1
        self.current_len += 1
        if self.lite_len >= self.L:
            self._kv_append(self._lite(self.Kgpu), self._lite(self.Vgpu))
            self.lite_len = 0

    def _A_K_hitted_with_lite(self):
        """:1156-1171 (gather on the full-capacity, zero-initialised buffer: Q2)"""
        b, H, _, _ = self.hit_indices.shape
        lite = torch.tensor(self.lite_indices, dtype=torch.int64).reshape(1, 1, -1, 1).expand(b, H, -1, 1)
        idx = torch.cat([self.hit_indices, lite], dim=2)
        return torch.take_along_dim(self._A_K.data, idx, 2)

    def prefill(self, q, k, v, A_Q0=None, A_K0=None, generator=None, als_result=None):
        """:1385-1504.  ``als_result`` = (A_Q, B_Q, A_K, B_K) in the storage dtype replaces the
        oracle's own factorisation (to continue from the factors of the implementation under
        test once those were checked within tolerance)."""
        b, H, l, d = q.shape
        assert l >= self.k, "seq_len must be larger than attn_topk"
        repk = repeat_kv(k, self.g)
        self.Kgpu = torch.zeros((b, H, self.n, d), dtype=q.dtype)
        self.Vgpu = torch.zeros((b, H, self.n, d), dtype=q.dtype)
        self.prefill_length = l
        self.current_len = l
        if als_result is not None:
            A_Q, B_Q, A_K, B_K = als_result
        else:
            A_Q, B_Q, A_K, B_K = cast_lrqk_prefill(q, repk, self.r, self.max_iter[0], self.tol[0], self.init,
                                                   A_Q0, A_K0, generator, self.compute_dtype)
        self.B_Q, self.B_K = B_Q, B_K
        self._A_K.append(A_K)
        self.last_A_Q = A_Q
        if l <= self.n:
            self._kv_append(k.narrow(2, 0, self.k), v.narrow(2, 0, self.k))
            rem = l - self.k
            self.lite_len = rem
            self.lite_indices = list(range(self.k, self.k + rem)) + [-1] * (self.L - rem)
            self.Kgpu.narrow(2, 0, l).copy_(repk)
            self.Vgpu.narrow(2, 0, l).copy_(repeat_kv(v, self.g))
            self.hit_indices = torch.arange(self.k, dtype=torch.int64).view(1, 1, self.k, 1).expand(
                b, H, self.k, 1).contiguous()
        else:
            self._kv_append(k, v)
            hit = compute_hit_indices(A_Q[:, :, -1:, :].contiguous(), A_K[:, :, 0:l - self.L, :].contiguous(),
                                      self.k, self.round_scores)
            self.hit_indices = hit
            repv = repeat_kv(v, self.g)
            self.Kgpu[:, :, :self.k, :] = torch.take_along_dim(repk, hit, 2)
            self.Vgpu[:, :, :self.k, :] = torch.take_along_dim(repv, hit, 2)
            lb = l - self.L
            self.lite_indices = list(range(lb, l))
            self.lite_len = 0
            self.Kgpu[:, :, self.k:, :] = repk.narrow(2, lb, self.L)
            self.Vgpu[:, :, self.k:, :] = repv.narrow(2, lb, self.L)

    def decode(self, q, k, v):
        """:1506-1613 (and :1688-1775 when no_hit_miss)"""
        return self.finish_decode(*self.begin_decode(q, k, v))

    def begin_decode(self, q, k, v):
        """Ring append + the factor update (:1519-1559), returned but not yet applied."""
        self._append(k, v)
        repk = repeat_kv(k, self.g)
        if self.current_len <= self.n:
            return cast_lrqk_decode(self.B_Q, self.A_K, self.B_K, self.Kgpu.narrow(2, 0, self.current_len - 1), q,
                                    repk, self.max_iter[1], self.tol[1], self.compute_dtype)
        return cast_lrqk_decode(self.B_Q, self._A_K_hitted_with_lite(), self.B_K, self.Kgpu, q, repk,
                                self.max_iter[1], self.tol[1], self.compute_dtype)

    def finish_decode(self, B_Q, B_K, hq, hk):
        """The rest of the step (:1540-1545 / :1560-1613) from given ALS outputs; split out so a
        test can inject the ALS result of the implementation under test (after checking it
        within tolerance) and compare the integer stages bit for bit."""
        self.B_Q, self.B_K = B_Q, B_K
        self._A_K.append(hk)
        self.last_q_hat, self.last_k_hat = hq, hk
        if self.current_len <= self.n:
            return self.Kgpu.narrow(2, 0, self.current_len), self.Vgpu.narrow(2, 0, self.current_len)
        m = self.lite_indices[self.lite_len] - 1
        self.last_m = m
        new = compute_hit_indices(hq, self.A_K.narrow(2, 0, m), self.k, self.round_scores)
        self.last_new_indices = new
        b, H = new.shape[:2]
        d = self.Kgpu.shape[-1]
        hkv = H // self.g
        if self.no_hit_miss:
            self.hit_indices = new
            mask = torch.ones((b, H, self.k), dtype=torch.bool)
        else:
            self.hit_indices, mask = only_indices_in_cpu(self.hit_indices, new)
        self.last_evict = mask
        rows = take_along_dim_with_mask(self.KVcpu.data, self.hit_indices.view(b, hkv, self.g, -1),
                                        mask.view(b, hkv, self.g, -1))
        if rows.numel() > 0:
            self.Kgpu[:, :, :self.k][mask] = rows[:, :d]
            self.Vgpu[:, :, :self.k][mask] = rows[:, d:]
        return self.Kgpu, self.Vgpu
