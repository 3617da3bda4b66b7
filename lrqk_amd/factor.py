"""Free functions of the factorisation interface (lrqk_attention.py:36-47, 140-209, 772-839):
repeat_kv, the A_Q/A_K initialisers, cast_lrqk_prefill and cast_lrqk_decode.  The
arithmetic of both casts runs in liblrqk_hip.so."""
from __future__ import annotations

import enum
from typing import Optional, Tuple, Union

import torch

from . import ops


def repeat_kv(hidden_states: torch.Tensor, n_rep: int) -> torch.Tensor:
    """[b,Hkv,s,d] -> [b,Hkv*n_rep,s,d]; output head h reads input head h // n_rep."""
    b, hkv, s, d = hidden_states.shape
    if n_rep == 1:
        return hidden_states
    return hidden_states[:, :, None, :, :].expand(b, hkv, n_rep, s, d).reshape(b, hkv * n_rep, s, d)


def _ensure_tuple2(x):
    if isinstance(x, (tuple, list)):
        assert len(x) == 2, "must be a tuple or list of length 2"
        return tuple(x)
    return (x, x)


class InitAQAK(enum.Enum):
    randn = enum.auto()
    top = enum.auto()
    topcol = enum.auto()


def _init_AQ_AK(Q: torch.Tensor, K: torch.Tensor, r: int, init_method: Union[InitAQAK, str] = InitAQAK.randn,
                generator: Optional[torch.Generator] = None):
    """lrqk_attention.py:145-209.  Q,K fp32 [b,H,l,d] -> A_Q0, A_K0 fp32 [b,H,l,r]."""
    if isinstance(init_method, str):
        if init_method not in InitAQAK.__members__:
            raise ValueError(f"Unknown init_method: {init_method}. Current support {list(InitAQAK.__members__.keys())}")
        init_method = InitAQAK[init_method]
    b, H, l, d = Q.shape
    if init_method == InitAQAK.randn:
        AQ = torch.randn((b, H, l, r), dtype=Q.dtype, device=Q.device, generator=generator)
        AK = torch.randn((b, H, l, r), dtype=K.dtype, device=K.device, generator=generator)
        return AQ, AK
    q_mass = Q.abs().sum(dim=2, keepdim=True)
    k_mass = K.abs().sum(dim=2, keepdim=True)
    if init_method == InitAQAK.topcol:
        cols_q = cols_k = torch.topk(q_mass + k_mass, k=r, dim=-1).indices
    elif init_method == InitAQAK.top:
        cols_q = torch.topk(q_mass, k=r, dim=-1).indices
        cols_k = torch.topk(k_mass, k=r, dim=-1).indices
    else:
        raise ValueError(f"Unknown init_method: {init_method}")
    AQ = torch.gather(Q, -1, cols_q.expand(-1, -1, l, -1)).contiguous()
    AK = torch.gather(K, -1, cols_k.expand(-1, -1, K.shape[2], -1)).contiguous()
    return AQ, AK


def cast_lrqk_prefill(Q: torch.Tensor, K: torch.Tensor, r: int, lambda_Q: float = 1.0, lambda_K: float = 1.0,
                      max_iter: int = 8, tol: float = 1e-5, init_method: Union[InitAQAK, str] = InitAQAK.randn,
                      init_factors: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                      workspace: Optional[ops.Workspace] = None):
    """lrqk_attention.py:772-800.  Q [b,Hq,l,d]; K [b,Hq,l,d] or un-repeated [b,Hkv,l,d].
    Returns a generator of (A_Q, B_Q, A_K, B_K) in K.dtype, like the reference.
    ``init_factors`` = (A_Q0, A_K0) fp32 [b,Hq,l,r] replaces the random draw."""
    if lambda_Q != 1.0 or lambda_K != 1.0:
        raise NotImplementedError("only lambda_Q = lambda_K = 1 is implemented")
    ws = workspace or ops.default_workspace()
    out_dtype = K.dtype
    Qc, Kc = Q.contiguous(), K.contiguous()
    if init_factors is not None:
        A_Q0 = init_factors[0].to(device=Q.device, dtype=torch.float32).clone().contiguous()
        A_K0 = init_factors[1].to(device=Q.device, dtype=torch.float32).clone().contiguous()
    else:
        g = Q.shape[1] // K.shape[1]
        A_Q0, A_K0 = _init_AQ_AK(Qc.float(), repeat_kv(Kc, g).float(), r, init_method)
    A_Q, B_Q, A_K, B_K = ops.als_prefill(ws, Qc, Kc, A_Q0, A_K0, max_iter, tol)
    return (o.to(dtype=out_dtype) for o in (A_Q, B_Q, A_K, B_K))


def cast_lrqk_decode(B_Q: torch.Tensor, A_K: torch.Tensor, B_K: torch.Tensor, K__: torch.Tensor, q: torch.Tensor,
                     k: torch.Tensor, lambda_dec_q: float = 1.0, lambda_dec_k: float = 1.0, max_iter: int = 8,
                     tol: float = 1e-5, workspace: Optional[ops.Workspace] = None):
    """lrqk_attention.py:803-839.  B_Q,B_K [b,H,r,d]; A_K [b,H,n,r]; K__ [b,H,n,d]; q,k [b,H,1,d].
    Returns a generator of (B_Q', B_K', q_hat, k_hat) in k.dtype; inputs are not modified."""
    if lambda_dec_q != 1.0 or lambda_dec_k != 1.0:
        raise NotImplementedError("only lambda_dec_q = lambda_dec_k = 1 is implemented")
    ws = workspace or ops.default_workspace()
    dt = k.dtype
    bq, bk = B_Q.to(dt).clone().contiguous(), B_K.to(dt).clone().contiguous()
    n = A_K.shape[2]
    q_hat, k_hat = ops.als_decode(ws, bq, bk, A_K.to(dt).contiguous(), None, K__.to(dt).contiguous(), n,
                                  q.to(dt), k.to(dt).contiguous(), max_iter, tol, append_row=-1)
    return (o for o in (bq, bk, q_hat, k_hat))
