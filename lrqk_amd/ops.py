"""Tensor-level wrappers over the C ABI.  torch is used only for device memory and the
current stream; every computation below happens in liblrqk_hip.so."""
from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import check


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return _lib.F32
    if t.dtype == torch.bfloat16:
        return _lib.BF16
    raise ValueError(f"unsupported dtype {t.dtype}: the kernels store float32 or bfloat16")


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _need_cuda(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise ValueError("tensor must live on the GPU")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


class Workspace:
    """Owns one lrqk_ctx (device scratch).  Not thread safe; one per engine."""

    def __init__(self):
        self._h = ctypes.c_void_p()
        check(_lib.load().lrqk_ctx_create(ctypes.byref(self._h)))

    @property
    def handle(self):
        return self._h

    def reserve(self, bh, max_tokens, topk, n_active, r, d):
        check(_lib.load().lrqk_ctx_reserve(self._h, bh, max_tokens, topk, n_active, r, d))

    def set_fetch_mode(self, mode: str, host_threads: int = 0):
        """'direct': the fetch kernel reads the pinned store itself (default); 'staged': host gather +
        hipMemcpyAsync on a side stream, as the reference stages its misses."""
        check(_lib.load().lrqk_ctx_set_fetch_mode(self.handle, {"direct": 0, "staged": 1}[mode], int(host_threads)))

    def score_index(self, enable: bool):
        """Switch the 8-bit score index of the scan on or off; either way what was indexed is dropped."""
        check(_lib.load().lrqk_ctx_score_index(self.handle, 1 if enable else 0))

    def victim_cache(self, rows_per_head: int):
        """Size (and empty) the victim cache of the fused decode step; 0 switches it off."""
        check(_lib.load().lrqk_ctx_victim_cache(self.handle, int(rows_per_head)))

    def factor_state(self, enable: bool = True):
        """Switch the kept state of the decode step's factor update on or off; either way what is kept is
        dropped (call it after changing B_Q, B_K, the active ids or rows behind the library's back)."""
        check(_lib.load().lrqk_ctx_factor_state(self.handle, 1 if enable else 0))

    def last_iterates(self, token: Optional[int] = None) -> Optional[torch.Tensor]:
        """fp64 [bh, max_iter, 2, r]: (q_hat, k_hat) of every iteration of the last decode step that ran from
        kept state, before any rounding; None if no such step ran (with ``token``: if that token's step did not)."""
        bh, it, r, tok = ctypes.c_int(), ctypes.c_int(), ctypes.c_int(), ctypes.c_int64()
        lib = _lib.load()
        check(lib.lrqk_last_iterates(self.handle, None, 0, ctypes.byref(bh), ctypes.byref(it), ctypes.byref(r),
                                     ctypes.byref(tok)))
        if bh.value * it.value * r.value == 0 or (token is not None and tok.value != token):
            return None
        out = torch.empty((bh.value, it.value, 2, r.value), dtype=torch.float64)
        check(lib.lrqk_last_iterates(self.handle, out.data_ptr(), out.numel(), ctypes.byref(bh), ctypes.byref(it),
                                     ctypes.byref(r), ctypes.byref(tok)))
        return out

    def victim_stats(self, reset: bool = True) -> int:
        """Rows the fused decode step fetched over the host link since the last reset."""
        n = ctypes.c_int64()
        check(_lib.load().lrqk_victim_stats(self.handle, ctypes.byref(n), 1 if reset else 0))
        return n.value

    def timing_enable(self, max_launches: int, every: int = 1):
        """Bracket (every `every`-th of) the next proxy-score launches with HIP events, at most max_launches."""
        check(_lib.load().lrqk_timing_enable(self._h, max_launches))
        check(_lib.load().lrqk_timing_stride(self._h, every))

    def timing_read(self):
        """(summed proxy-score kernel time in ms, launches) since the last read."""
        ms, n = ctypes.c_double(), ctypes.c_int()
        check(_lib.load().lrqk_timing_read(self._h, ctypes.byref(ms), ctypes.byref(n)))
        return ms.value, n.value

    def select_stats(self, reset: bool = True):
        """(heads served from the candidate list, heads that rescanned) since the last reset."""
        a, b = ctypes.c_int(), ctypes.c_int()
        check(_lib.load().lrqk_select_stats(self._h, ctypes.byref(a), ctypes.byref(b), 1 if reset else 0))
        return a.value, b.value

    def scan_stats(self):
        """(rows covered, rows rescored exactly) by the last scan through the score index; (0, 0) otherwise."""
        a, b = ctypes.c_int64(), ctypes.c_int64()
        check(_lib.load().lrqk_scan_stats(self._h, ctypes.byref(a), ctypes.byref(b)))
        return a.value, b.value

    def select_stats_detail(self):
        """(lists too short, lists overflowed) among the rescans of the last select_stats()."""
        a, b = ctypes.c_int(), ctypes.c_int()
        check(_lib.load().lrqk_select_stats_detail(self._h, ctypes.byref(a), ctypes.byref(b)))
        return a.value, b.value

    def close(self):
        if self._h:
            _lib.load().lrqk_ctx_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


_default_ws: Optional[Workspace] = None


def default_workspace() -> Workspace:
    global _default_ws
    if _default_ws is None:
        _default_ws = Workspace()
    return _default_ws


# --------------------------------------------------------------------------- selection

def proxy_scores(a_k: torch.Tensor, q_hat: torch.Tensor, m: Optional[int] = None,
                 round_to_storage: bool = True) -> torch.Tensor:
    """a_k [b,H,cap,r] (contiguous), q_hat [b,H,1,r] -> fp32 [b,H,m]."""
    _need_cuda(a_k, q_hat)
    b, H, cap, r = a_k.shape
    m = cap if m is None else m
    assert a_k.is_contiguous() and 0 <= m <= cap
    qh = q_hat.reshape(b * H, r).contiguous()
    out = torch.empty((b, H, m), dtype=torch.float32, device=a_k.device)
    check(_lib.load().lrqk_proxy_scores(a_k.data_ptr(), cap * r, qh.data_ptr(), b * H, m, r, _dt(a_k),
                                        1 if (round_to_storage and a_k.dtype == torch.bfloat16) else 0,
                                        out.data_ptr(), _stream(a_k)))
    return out


def score_select(ws: Workspace, a_k: torch.Tensor, q_hat: torch.Tensor, m: int, topk: int,
                 round_to_storage: bool = True, out: Optional[torch.Tensor] = None,
                 head_rows: Optional[int] = None) -> torch.Tensor:
    """Top-k token ids (ascending) of q_hat . a_k[:m]^T per head: int32 [b,H,min(topk,m)].
    a_k is [b,H,cap,r] contiguous, or (with head_rows) a view whose heads start head_rows rows
    apart and whose rows are contiguous."""
    _need_cuda(a_k, q_hat)
    b, H, cap, r = a_k.shape
    if head_rows is None:
        assert a_k.is_contiguous()
    else:
        cap = head_rows
    assert 0 <= m <= cap
    qh = q_hat.reshape(b * H, r).contiguous()
    kk = min(topk, m)
    if out is None:
        out = torch.empty((b, H, kk), dtype=torch.int32, device=a_k.device)
    assert out.dtype == torch.int32 and out.is_contiguous() and out.shape[-1] >= kk
    check(_lib.load().lrqk_score_select(ws.handle, a_k.data_ptr(), cap * r, qh.data_ptr(), b * H, m, r, topk,
                                        _dt(a_k), 1 if (round_to_storage and a_k.dtype == torch.bfloat16) else 0,
                                        out.data_ptr(), out.shape[-1], _stream(a_k)))
    return out


def score_select_diff(ws: Workspace, a_k: torch.Tensor, q_hat: torch.Tensor, m: int, topk: int, hit: torch.Tensor,
                      round_to_storage: bool = True, want_new: bool = True):
    """score_select + diff in one pass (m >= topk).  hit int32 [b,H,>=topk] is updated in place.
    Returns (new_idx int32 [b,H,topk], evict u8 [b,H,topk], miss_slots int32 [b,H,topk], miss_count int32 [b,H]).
    want_new=False: only what changes is produced (new_idx is None), as inside the decode step."""
    _need_cuda(a_k, q_hat, hit)
    b, H, cap, r = a_k.shape
    assert a_k.is_contiguous() and hit.is_contiguous() and hit.dtype == torch.int32 and topk <= m <= cap
    qh = q_hat.reshape(b * H, r).contiguous()
    dev = a_k.device
    new = torch.empty((b, H, topk), dtype=torch.int32, device=dev) if want_new else None
    evict = torch.empty((b, H, topk), dtype=torch.uint8, device=dev)
    miss_slots = torch.empty((b, H, topk), dtype=torch.int32, device=dev)
    miss_count = torch.empty((b, H), dtype=torch.int32, device=dev)
    check(_lib.load().lrqk_score_select_diff(ws.handle, a_k.data_ptr(), cap * r, qh.data_ptr(), b * H, m, r, topk,
                                             _dt(a_k), 1 if (round_to_storage and a_k.dtype == torch.bfloat16) else 0,
                                             _ptr(new), hit.data_ptr(), hit.shape[-1], evict.data_ptr(),
                                             miss_slots.data_ptr(), miss_count.data_ptr(), _stream(a_k)))
    return new, evict, miss_slots, miss_count


def select_from_scores(ws: Workspace, scores: torch.Tensor, topk: int) -> torch.Tensor:
    """scores fp32 [b,H,m] -> int32 [b,H,min(topk,m)] ascending."""
    _need_cuda(scores)
    b, H, m = scores.shape
    sc = scores.contiguous().float()
    kk = min(topk, m)
    out = torch.empty((b, H, kk), dtype=torch.int32, device=scores.device)
    check(_lib.load().lrqk_select_from_scores(ws.handle, sc.data_ptr(), b * H, m, topk, out.data_ptr(), kk,
                                              _stream(scores)))
    return out


def diff(new_idx: torch.Tensor, hit: torch.Tensor, k: Optional[int] = None, replace_all: bool = False):
    """In-place hit/miss diff.  new_idx int32 [b,H,>=k] ascending; hit int32 [b,H,stride] (first k
    entries are the resident set; may be a wider buffer).  Returns (evict u8 [b,H,k], miss_slots
    int32 [b,H,k], miss_count int32 [b,H])."""
    _need_cuda(new_idx, hit)
    b, H = hit.shape[:2]
    k = hit.shape[2] if k is None else k
    assert new_idx.dtype == torch.int32 and hit.dtype == torch.int32
    assert new_idx.is_contiguous() and hit.is_contiguous()
    dev = hit.device
    evict = torch.empty((b, H, k), dtype=torch.uint8, device=dev)
    miss_slots = torch.empty((b, H, k), dtype=torch.int32, device=dev)
    miss_count = torch.empty((b, H), dtype=torch.int32, device=dev)
    fn = _lib.load().lrqk_replace_all if replace_all else _lib.load().lrqk_diff
    check(fn(new_idx.data_ptr(), new_idx.shape[2], hit.data_ptr(), hit.shape[2], b * H, k, evict.data_ptr(),
             miss_slots.data_ptr(), miss_count.data_ptr(), _stream(hit)))
    return evict, miss_slots, miss_count


def fetch_rows(kv_store: torch.Tensor, k_act: torch.Tensor, v_act: torch.Tensor, hit: torch.Tensor,
               miss_slots: torch.Tensor, miss_count: torch.Tensor, k: int):
    """kv_store [b,Hkv,cap,2d] (pinned host or device), k_act/v_act [b,Hq,n,d]."""
    _need_cuda(k_act, v_act, hit, miss_slots, miss_count)
    b, hkv, cap, d2 = kv_store.shape
    _, hq, n, d = k_act.shape
    assert d2 == 2 * d and kv_store.is_contiguous() and k_act.is_contiguous() and v_act.is_contiguous()
    assert kv_store.dtype == k_act.dtype == v_act.dtype
    if not kv_store.is_cuda and not kv_store.is_pinned():
        raise ValueError("the host [K|V] store must be pinned memory")
    check(_lib.load().lrqk_fetch_rows(kv_store.data_ptr(), cap, k_act.data_ptr(), v_act.data_ptr(), n, hit.data_ptr(),
                                      hit.shape[2], miss_slots.data_ptr(), miss_count.data_ptr(), b, hq, hkv, d, k,
                                      _dt(k_act), _stream(k_act)))


def fetch_rows_staged(ws: Workspace, kv_store: torch.Tensor, k_act: torch.Tensor, v_act: torch.Tensor,
                      hit: torch.Tensor, miss_slots: torch.Tensor, miss_count: torch.Tensor, k: int):
    """Same result as fetch_rows, through host gather + hipMemcpyAsync on the workspace's side stream
    (kv_store must be pinned host memory; waits for the stream once)."""
    _need_cuda(k_act, v_act, hit, miss_slots, miss_count)
    b, hkv, cap, d2 = kv_store.shape
    _, hq, n, d = k_act.shape
    assert d2 == 2 * d and kv_store.is_contiguous() and k_act.is_contiguous() and v_act.is_contiguous()
    assert kv_store.dtype == k_act.dtype == v_act.dtype
    if kv_store.is_cuda or not kv_store.is_pinned():
        raise ValueError("the staged fetch needs the [K|V] store in pinned host memory")
    check(_lib.load().lrqk_fetch_rows_staged(ws.handle, kv_store.data_ptr(), cap, k_act.data_ptr(), v_act.data_ptr(), n,
                                             hit.data_ptr(), hit.shape[2], miss_slots.data_ptr(),
                                             miss_count.data_ptr(), b, hq, hkv, d, k, _dt(k_act), _stream(k_act)))


def gather_rows(src: torch.Tensor, idx: torch.Tensor, dst: torch.Tensor, count: int):
    """dst[b,h,j,:] = src[b,h//g,idx[b,h,j],:] for j < count; slots whose id is negative keep their
    contents.  src [b,Hkv,l,d] on the GPU or in pinned host memory, dst [b,Hq,n,d]."""
    _need_cuda(idx, dst)
    if not src.is_cuda and not src.is_pinned():
        raise ValueError("a host source must be pinned memory")
    b, hkv, l, d = src.shape
    _, hq, n, _ = dst.shape
    # the kernel takes the row width and the element type from src alone: a source whose rows are wider than
    # the destination's (the [K|V] store, 2d wide) would be written past the end of dst
    if src.shape[-1] != dst.shape[-1] or src.dtype != dst.dtype or src.shape[0] != dst.shape[0]:
        raise ValueError(f"source rows {tuple(src.shape)} {src.dtype} do not match the destination "
                         f"{tuple(dst.shape)} {dst.dtype}: pass a K or a V source whose rows are as wide as dst")
    if hq % hkv != 0 or tuple(idx.shape[:2]) != (b, hq) or not 0 <= count <= min(idx.shape[2], n):
        raise ValueError("idx must be [b,Hq,>=count] with count slots inside dst")
    assert src.is_contiguous() and dst.is_contiguous() and idx.is_contiguous() and idx.dtype == torch.int32
    check(_lib.load().lrqk_gather_rows(src.data_ptr(), l, idx.data_ptr(), idx.shape[2], count, dst.data_ptr(), n, b, hq,
                                       hkv, d, _dt(src), _stream(dst)))


def append_token(k_new, v_new, k_act, v_act, slot: int, active_idx: Optional[torch.Tensor], token: int):
    _need_cuda(k_new, v_new, k_act, v_act)
    b, hkv = k_new.shape[:2]
    _, hq, n, d = k_act.shape
    kn, vn = k_new.reshape(b, hkv, d).contiguous(), v_new.reshape(b, hkv, d).contiguous()
    check(_lib.load().lrqk_append_token(kn.data_ptr(), vn.data_ptr(), k_act.data_ptr(), v_act.data_ptr(), n, slot,
                                        _ptr(active_idx), 0 if active_idx is None else active_idx.shape[2], token, b,
                                        hq, hkv, d, _dt(k_act), _stream(k_act)))


def flush_ring(k_act, v_act, slot0: int, count: int, kv_store: torch.Tensor, row0: int, hkv: int):
    _need_cuda(k_act, v_act)
    b, hq, n, d = k_act.shape
    cap = kv_store.shape[2]
    check(_lib.load().lrqk_flush_ring(k_act.data_ptr(), v_act.data_ptr(), n, slot0, count, kv_store.data_ptr(), cap,
                                      row0, b, hq, hkv, d, _dt(k_act), _stream(k_act)))


def attention(ws: Workspace, q: torch.Tensor, k_act: torch.Tensor, v_act: torch.Tensor,
              n_valid: Optional[int] = None) -> torch.Tensor:
    """q [b,H,1,d]; k_act,v_act [b,H,n,d] contiguous -> [b,H,1,d]."""
    _need_cuda(q, k_act, v_act)
    b, H, n, d = k_act.shape
    n_valid = n if n_valid is None else n_valid
    assert k_act.is_contiguous() and v_act.is_contiguous() and q.dtype == k_act.dtype == v_act.dtype
    qq = q.reshape(b * H, d).contiguous()
    out = torch.empty((b, H, 1, d), dtype=q.dtype, device=q.device)
    check(_lib.load().lrqk_attention(ws.handle, qq.data_ptr(), k_act.data_ptr(), v_act.data_ptr(), n, n_valid,
                                     out.data_ptr(), b * H, d, _dt(q), _stream(q)))
    return out


def attention_static(q: torch.Tensor, k_act: torch.Tensor, v_act: torch.Tensor, out: torch.Tensor,
                     n_valid: Optional[int] = None) -> torch.Tensor:
    """The same attention through the entry point that allocates nothing: no workspace, the caller
    passes ``out`` [b,H,1,d] and a contiguous q; partial results go to a fixed block inside the library."""
    _need_cuda(q, k_act, v_act, out)
    b, H, n, d = k_act.shape
    n_valid = n if n_valid is None else n_valid
    assert k_act.is_contiguous() and v_act.is_contiguous() and q.is_contiguous() and out.is_contiguous()
    assert q.dtype == k_act.dtype == v_act.dtype == out.dtype and out.numel() == b * H * d
    check(_lib.load().lrqk_attention_static(q.data_ptr(), k_act.data_ptr(), v_act.data_ptr(), n, n_valid,
                                            out.data_ptr(), b * H, d, _dt(q), _stream(q)))
    return out


def als_decode(ws: Workspace, b_q, b_k, a_k, active_idx: Optional[torch.Tensor], k_prev, n: int, q, k_new,
               max_iter: int, tol: float, append_row: int = -1) -> Tuple[torch.Tensor, torch.Tensor]:
    """In-place factor update.  b_q,b_k [b,H,r,d]; a_k [b,H,cap,r]; active_idx int32 [b,H,>=n] or None;
    k_prev [b,H,slots,d]; q [b,H,1,d]; k_new [b,Hkv,1,d].  Returns (q_hat, k_hat) [b,H,1,r]."""
    _need_cuda(b_q, b_k, a_k, k_prev, q, k_new)
    b, H, r, d = b_q.shape
    hkv = k_new.shape[1]
    cap = a_k.shape[2]
    assert b_q.is_contiguous() and b_k.is_contiguous() and a_k.is_contiguous() and k_prev.is_contiguous()
    assert b_q.dtype == b_k.dtype == a_k.dtype == k_prev.dtype == q.dtype == k_new.dtype
    qq = q.reshape(b * H, d).contiguous()
    kn = k_new.reshape(b * hkv, d).contiguous()
    q_hat = torch.empty((b, H, 1, r), dtype=b_q.dtype, device=b_q.device)
    k_hat = torch.empty((b, H, 1, r), dtype=b_q.dtype, device=b_q.device)
    check(_lib.load().lrqk_als_decode(ws.handle, b_q.data_ptr(), b_k.data_ptr(), a_k.data_ptr(), cap * r,
                                      _ptr(active_idx), 0 if active_idx is None else active_idx.shape[2],
                                      k_prev.data_ptr(), k_prev.shape[2], n, qq.data_ptr(), kn.data_ptr(), b, H, hkv, r,
                                      d, int(max_iter), float(tol), q_hat.data_ptr(), k_hat.data_ptr(), append_row,
                                      _dt(b_q), _stream(b_q)))
    return q_hat, k_hat


def als_prefill(ws: Workspace, q: torch.Tensor, k: torch.Tensor, a_q0: torch.Tensor, a_k0: torch.Tensor,
                max_iter: int, tol: float):
    """q [b,Hq,l,d], k [b,Hkv,l,d] storage dtype; a_q0,a_k0 fp32 [b,Hq,l,r] initial factors (consumed:
    they are updated in place).  Returns fp32 (A_Q, B_Q, A_K, B_K)."""
    _need_cuda(q, k, a_q0, a_k0)
    b, hq, l, d = q.shape
    hkv = k.shape[1]
    r = a_q0.shape[-1]
    assert q.is_contiguous() and k.is_contiguous() and q.dtype == k.dtype
    assert a_q0.dtype == torch.float32 and a_k0.dtype == torch.float32 and a_q0.is_contiguous() and a_k0.is_contiguous()
    assert a_q0.shape == (b, hq, l, r) and a_k0.shape == (b, hq, l, r)
    b_q = torch.empty((b, hq, r, d), dtype=torch.float32, device=q.device)
    b_k = torch.empty((b, hq, r, d), dtype=torch.float32, device=q.device)
    check(_lib.load().lrqk_als_prefill(ws.handle, q.data_ptr(), k.data_ptr(), a_q0.data_ptr(), a_k0.data_ptr(),
                                       b_q.data_ptr(), b_k.data_ptr(), b, hq, hkv, l, r, d, int(max_iter), float(tol),
                                       _dt(q), _stream(q)))
    return a_q0, b_q, a_k0, b_k


def decode_step(ws: Workspace, b_q, b_k, a_k, active_idx, k_act, v_act, kv_store, q, k_new, v_new, *, topk: int,
                lite: int, ring_slot: int, token: int, m: int, flush_row0: int, max_iter: int, tol: float,
                round_scores: bool, no_hit_miss: bool, q_hat, k_hat, attn_out=None, evict=None, miss_count=None):
    b, H, r, d = b_q.shape
    hkv = k_new.shape[1]
    cap_a = a_k.shape[2]
    qq = q.reshape(b * H, d)
    kn = k_new.reshape(b * hkv, d)
    vn = v_new.reshape(b * hkv, d)
    assert qq.is_contiguous() and kn.is_contiguous() and vn.is_contiguous()
    check(_lib.load().lrqk_decode_step(
        ws.handle, b_q.data_ptr(), b_k.data_ptr(), a_k.data_ptr(), cap_a * r, active_idx.data_ptr(), k_act.data_ptr(),
        v_act.data_ptr(), kv_store.data_ptr(), kv_store.shape[2], qq.data_ptr(), kn.data_ptr(), vn.data_ptr(), b, H, hkv,
        r, d, topk, lite, ring_slot, token, m, flush_row0, int(max_iter), float(tol),
        1 if (round_scores and b_q.dtype == torch.bfloat16) else 0, 1 if no_hit_miss else 0, q_hat.data_ptr(),
        k_hat.data_ptr(), _ptr(attn_out), _ptr(evict), _ptr(miss_count), _dt(b_q), _stream(b_q)))


def probe_bandwidth(nbytes: int, reps: int = 10, device="cuda:0"):
    """(read GB/s, copy GB/s of bytes read + bytes written) of plain streaming kernels over ``nbytes``."""
    src = torch.empty(nbytes, dtype=torch.uint8, device=device).fill_(1)
    dst = torch.empty_like(src)
    r_ms, c_ms = ctypes.c_double(), ctypes.c_double()
    check(_lib.load().lrqk_probe_bandwidth(src.data_ptr(), dst.data_ptr(), nbytes, reps, ctypes.byref(r_ms),
                                           ctypes.byref(c_ms), _stream(src)))
    return nbytes / (r_ms.value * 1e-3) / 1e9, 2 * nbytes / (c_ms.value * 1e-3) / 1e9


def probe_read_sweep(nbytes: int, reps: int = 5, device="cuda:0", slice_bytes: int = 0):
    """The plain read over ``nbytes`` in every variant (4 / 8 / 16 vectors in flight, plain / non-temporal loads,
    1 .. 8 workgroups per CU): ({(in_flight, nontemporal, grid_per_cu): GB/s}, best GB/s).  With ``slice_bytes`` a
    launch reads one slice of the buffer and the launches take the slices in turn: the rate of launches of that size."""
    src = torch.empty(nbytes, dtype=torch.uint8, device=device).fill_(1)
    sink = torch.zeros(1 << 16, dtype=torch.uint8, device=device)
    table = {}
    ms = ctypes.c_double()
    per_launch = slice_bytes or nbytes
    n = reps * (nbytes // slice_bytes) if slice_bytes else reps
    for nt in (0, 1):
        for fl in (4, 8, 16):
            for per_cu in (1, 2, 4, 8):
                check(_lib.load().lrqk_probe_read_variant(src.data_ptr(), sink.data_ptr(), nbytes, slice_bytes, min(n, 1000), fl,
                                                          nt, per_cu, ctypes.byref(ms), _stream(src)))
                table[(fl, nt, per_cu)] = per_launch / (ms.value * 1e-3) / 1e9
    return table, max(table.values())


def probe_event_pair(reps: int = 64, device="cuda:0", kernels: int = 1) -> float:
    """Microseconds that a pair of HIP events reads around ``kernels`` launches that do nothing (average of ``reps``
    pairs)."""
    us = ctypes.c_double()
    with torch.cuda.device(device):
        check(_lib.load().lrqk_probe_event_pair(reps, kernels, ctypes.byref(us),
                                                torch.cuda.current_stream().cuda_stream))
    return us.value


# --------------------------------------------------------------------------- host gathers

def d0_index_select(src: torch.Tensor, indices: torch.Tensor, threads: int = 8) -> torch.Tensor:
    """Host row gather into a new pinned tensor: out[i] = src[indices[i]].  src [N,w] CPU, indices int64 [n]."""
    if src.is_cuda or indices.is_cuda:
        raise ValueError("d0_index_select gathers host rows; tensors must be on the CPU")
    src = src.contiguous()
    idx = indices.to(torch.int64).contiguous()
    pin = torch.cuda.is_available()
    out = torch.empty((idx.shape[0], src.shape[1]), dtype=src.dtype, pin_memory=pin)
    check(_lib.load().lrqk_d0_indices_select(out.data_ptr(), src.data_ptr(), idx.data_ptr(), idx.shape[0],
                                             src.shape[1] * src.element_size(), src.shape[0], threads))
    return out


def take_along_dim_with_mask(src: torch.Tensor, indices: torch.Tensor, mask: torch.Tensor, threads: int = 8):
    """src [b,Hkv,seq,w] CPU; indices int64, mask bool [b,Hkv,g,k] CPU -> [sum(mask), w]."""
    for name, t in (("src", src), ("indices", indices), ("indices_mask", mask)):
        if t.is_cuda:
            raise RuntimeError(f"{name} must be a CPU tensor")
        if not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous")
    if indices.dtype != torch.int64:
        raise RuntimeError("indices must be int64")
    if mask.dtype != torch.bool:
        raise RuntimeError("mask must be bool")
    if src.dim() != 4 or indices.dim() != 4:
        raise RuntimeError("src [bsz, kv_heads, seq_len, hdim]; indices [bsz, kv_heads, num_groups, k]")
    if mask.shape != indices.shape:
        raise RuntimeError("shape mask != indices")
    b, hkv, seq, w = src.shape
    _, _, g, k = indices.shape
    mk = mask.view(torch.uint8)
    lib = _lib.load()
    rb = w * src.element_size()
    total = check(lib.lrqk_take_along_dim_with_mask(None, src.data_ptr(), indices.data_ptr(), mk.data_ptr(), b, hkv, g,
                                                    k, seq, rb, threads))
    out = torch.empty((total, w), dtype=src.dtype)
    if total:
        check(lib.lrqk_take_along_dim_with_mask(out.data_ptr(), src.data_ptr(), indices.data_ptr(), mk.data_ptr(), b,
                                                hkv, g, k, seq, rb, threads))
    return out
