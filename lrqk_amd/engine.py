"""Per-layer LRQK engine with the interface of LightAttentionIndicesFactory
(lrqk_attention.py:1031-1775).  This file only keeps state and decides which C-ABI entry
point to call; every computation on the decode path runs in liblrqk_hip.so.

State kept on the GPU
  B_Q, B_K        [b, Hq, r, d]          storage dtype
  _A_K            [b, Hq, capacity, r]   storage dtype, zero beyond the rows written
  Kgpu, Vgpu      [b, Hq, k+L, d]        slots 0..k-1 = selected tokens, k..k+L-1 = recent ring
  _active_idx     [b, Hq, k+L] int32     token id held by each slot
State kept in pinned host memory
  KVcpu           [b, Hkv, capacity, 2d] every flushed token, [K row | V row]
"""
from __future__ import annotations

from typing import Optional, Tuple, Union

import torch

from . import ops
from .buffers import AutoIncreaseTensor, AutoIncreaseTensorSharedKV
from .factor import InitAQAK, _ensure_tuple2, _init_AQ_AK, repeat_kv


class LightAttentionIndicesFactory:
    no_hit_miss = False

    def __init__(self, num_lite_tokens: int = 1, attn_topk: int = 128, num_key_value_groups: int = 1, r: int = 16,
                 max_iter: Union[int, Tuple[int, int]] = 2, tol: Union[float, Tuple[float, float]] = 1e-4,
                 weights: Tuple[float, float, float, float] = (1.0, 1.0, 1.0, 1.0), capacity: int = 4096,
                 init_aq_ak_method: Union[InitAQAK, str] = InitAQAK.randn, scaling_ratio: float = 1.5,
                 device: Optional[torch.device] = None, dtype: Optional[torch.dtype] = None,
                 round_scores_to_storage: bool = True):
        self.num_lite_tokens = num_lite_tokens
        self.attn_topk = attn_topk
        self.dim = 2
        self.num_key_value_groups = num_key_value_groups
        self.r = r
        self.max_iter = _ensure_tuple2(max_iter)
        self.tol = _ensure_tuple2(tol)
        self.init_aq_ak_method = init_aq_ak_method
        self.gpu_capacity = attn_topk + num_lite_tokens
        self.prefill_length = 0
        self.current_len = 0
        if isinstance(weights, float):
            self.weights = (weights,) * 4
        elif isinstance(weights, tuple):
            assert len(weights) == 4, "weights must be a tuple of length 4"
            self.weights = weights
        else:
            raise ValueError("weights must be a float or a tuple of length 4")
        if any(w != 1.0 for w in self.weights):
            raise NotImplementedError("only unit weights are implemented (the only setting the cache front door "
                                      "ever forwards, lrqk_attention.py:1811-1820)")
        # proxy scores of bf16 factors are rounded to bf16 before ranking, as the reference's
        # bf16 matmul does (lrqk_attention.py:1260-1263); False ranks on the fp32 sums
        self.round_scores_to_storage = round_scores_to_storage

        self.B_Q: Optional[torch.Tensor] = None
        self.B_K: Optional[torch.Tensor] = None
        self._A_K = AutoIncreaseTensor(capacity=capacity, dim=2, scaling_ratio=scaling_ratio, device=device, dtype=dtype)
        self.KVcpu = AutoIncreaseTensorSharedKV(capacity=capacity, dim=2, scaling_ratio=scaling_ratio, device="cpu",
                                                pin_memory=True)
        self.Kgpu: Optional[torch.Tensor] = None
        self.Vgpu: Optional[torch.Tensor] = None
        self.lite_len = 0
        self.lite_indices = [-1] * self.num_lite_tokens
        self._active_idx: Optional[torch.Tensor] = None  # int32 [b,Hq,k+L]
        self._hit_len = 0
        self.verbose = False
        self.ws = ops.Workspace()
        # injected initial factors (fp32 [b,Hq,l,r]) for reproducible `randn` initialisation
        self.init_factors: Optional[Tuple[torch.Tensor, torch.Tensor]] = None
        # per-step results kept for inspection / statistics
        self.last_q_hat = None
        self.last_k_hat = None
        self.last_evict = None        # uint8 [b,Hq,k]
        self.last_miss_count = None   # int32 [b,Hq]
        self.last_attn = None
        self.attn_in_step = False     # compute attention inside the fused step (uses the step's q)
        self._fetch_mode = "direct"
        # rows per head of the device-side victim cache of evicted K/V rows (0 = off); None = 4 * attn_topk
        self.victim_rows: Optional[int] = None
        # 8-bit copy of the A_K rows read by the scan (bounds + exact rescoring of the rows that may pass)
        self.use_score_index = True
        # True: the decode step's factor update runs in fp64 from state kept between steps (iterates equal to an
        # fp64 evaluation to rounding; one more launch per step); False: over the active rows in fp32
        self.use_factor_state = False

    # ------------------------------------------------------------------ small accessors
    @property
    def victim_rows_effective(self) -> int:
        """Rows per head the victim cache is created with (the library's limit is 32767)."""
        return min(4 * self.attn_topk, 32767) if self.victim_rows is None else self.victim_rows

    @property
    def fetch_mode(self) -> str:
        """'direct' (the fetch kernel reads the pinned store) or 'staged' (host gather into pinned staging +
        hipMemcpyAsync on a side stream + scatter, the way lrqk_attention.py:1597-1608 moves its misses)."""
        return self._fetch_mode

    @fetch_mode.setter
    def fetch_mode(self, mode: str):
        self.ws.set_fetch_mode(mode)
        self._fetch_mode = mode

    def __len__(self):
        return self.current_len

    def _lite_view(self, src):
        return src[:, 0:src.shape[1]:self.num_key_value_groups, self.attn_topk:self.attn_topk + self.num_lite_tokens, :]

    @property
    def Klite(self):
        return self._lite_view(self.Kgpu)

    @property
    def Vlite(self):
        return self._lite_view(self.Vgpu)

    @property
    def Kgpu_topk_area(self):
        return self.Kgpu.narrow(self.dim, 0, self.attn_topk)

    @property
    def Vgpu_topk_area(self):
        return self.Vgpu.narrow(self.dim, 0, self.attn_topk)

    @property
    def A_K(self):
        return self._A_K.tensor()

    @property
    def hit_indices(self) -> Optional[torch.Tensor]:
        """Token ids of the selected slots, int64 [b,Hq,k,1] (a copy of the device table)."""
        if self._active_idx is None:
            return None
        return self._active_idx[:, :, :self._hit_len].to(torch.int64).unsqueeze(-1)

    @hit_indices.setter
    def hit_indices(self, value: torch.Tensor):
        v = value.reshape(value.shape[0], value.shape[1], -1)
        self._hit_len = v.shape[2]
        self._active_idx[:, :, :self._hit_len] = v.to(torch.int32)
        self.ws.factor_state(self.use_factor_state)   # the kept sums describe the old ids

    @property
    def A_K_hitted(self):
        if self._active_idx is None:
            return self._A_K.tensor()
        return self._A_K.take_along_dim(self.hit_indices)

    def _get_A_K_hitted_with_lite(self):
        """lrqk_attention.py:1156-1171 (gather on the full-capacity, zero-initialised buffer)."""
        return self._A_K.take_along_dim(self._active_idx.to(torch.int64).unsqueeze(-1))

    @property
    def Kgpu_hitted(self):
        if self._active_idx is None:
            return self.Kgpu
        return self.Kgpu[:, :, :min(self._hit_len, self.attn_topk), :]

    def sync_cache(self, B_Q: torch.Tensor, A_K: torch.Tensor, B_K: torch.Tensor):
        """lrqk_attention.py:1208-1233"""
        self.B_Q = B_Q
        self._A_K.append(A_K)
        self.B_K = B_K
        # rows of A_K were written behind the library's back: whatever the scan had indexed is dropped
        self.ws.score_index(self.use_score_index)
        self.ws.factor_state(self.use_factor_state)
        return self

    def _is_overridden(self, name: str) -> bool:
        return getattr(type(self), name) is not getattr(LightAttentionIndicesFactory, name)

    # ------------------------------------------------------------------ overridable stages
    def compute_hit_indices(self, query_states: torch.Tensor, key_states: torch.Tensor) -> torch.Tensor:
        """lrqk_attention.py:1235-1273.  query_states [b,H,1,r]; key_states [b,H,m,r] (may be a
        narrow view of the factor buffer) -> int64 [b,H,min(k,m),1], ascending."""
        b, H, m, r = key_states.shape
        base, cap = _as_head_strided(key_states)
        out = ops.score_select(self.ws, base, query_states, m, self.attn_topk, self.round_scores_to_storage,
                               head_rows=cap)
        return out.to(torch.int64).unsqueeze(-1)

    def only_indices_in_cpu(self, now_indices: torch.Tensor, new_indices: torch.Tensor):
        """lrqk_attention.py:1275-1315 -> (updated int64 [b,H,k,1], replaced-slot mask bool [b,H,k])."""
        b, H = now_indices.shape[:2]
        hit = now_indices.reshape(b, H, -1).to(torch.int32).contiguous()
        new = new_indices.reshape(b, H, -1).to(torch.int32).contiguous()
        evict, slots, count = ops.diff(new, hit)
        self._last_slots, self._last_count = slots, count
        return hit.to(torch.int64).unsqueeze(-1), evict.bool()

    def fetch_by_hit(self, dst: torch.Tensor, src: torch.Tensor, hit_indices: torch.Tensor,
                     dst_mask: Optional[torch.Tensor] = None):
        """lrqk_attention.py:1317-1383.  dst [b,Hq,<=k,d] must be the topk area of Kgpu or Vgpu
        (a narrow view); src [b,Hkv,seq,d] on the GPU or in pinned host memory: a K or a V source whose rows
        are as wide as dst's (not the 2d-wide [K|V] store: such a source is refused); with dst_mask only the
        slots it marks are written."""
        b, H = hit_indices.shape[:2]
        idx = hit_indices.reshape(b, H, -1).to(device=dst.device, dtype=torch.int32)
        count = idx.shape[2]
        full = self.Kgpu if dst.data_ptr() == self.Kgpu.data_ptr() else self.Vgpu
        assert dst.data_ptr() == full.data_ptr(), "dst must be the topk area of Kgpu or Vgpu"
        if not src.is_cuda:
            # host source (:1351-1381): every listed row, or with dst_mask only the slots it marks; the
            # kernel reads the pinned rows through their device mapping and skips negative ids
            if not (src.is_pinned() and src.is_contiguous()):
                raise ValueError("a host source must be contiguous pinned memory")
            if dst_mask is not None:
                idx = torch.where(dst_mask.reshape(b, H, -1).to(dst.device), idx, torch.full_like(idx, -1))
        ops.gather_rows(src if not src.is_cuda else src.contiguous(), idx.contiguous(), full, count)
        self.ws.factor_state(self.use_factor_state)   # rows of the active set changed
        return dst if count >= self.attn_topk else dst.narrow(2, 0, count)

    # ------------------------------------------------------------------ prefill
    @torch.inference_mode()
    def prefill(self, query_states: torch.Tensor, key_states: torch.Tensor, value_states: torch.Tensor):
        """lrqk_attention.py:1385-1504.  query_states [b,Hq,l,d]; key/value_states [b,Hkv,l,d]."""
        bsz, nheads, seq_len, hdim = query_states.shape
        assert seq_len >= self.attn_topk, "seq_len must be larger than attn_topk"
        k, L, g = self.attn_topk, self.num_lite_tokens, self.num_key_value_groups
        dev, dt = query_states.device, query_states.dtype
        key_states = key_states.contiguous()
        value_states = value_states.contiguous()
        self.Kgpu = torch.zeros((bsz, nheads, self.gpu_capacity, hdim), dtype=dt, device=dev)
        self.Vgpu = torch.zeros((bsz, nheads, self.gpu_capacity, hdim), dtype=dt, device=dev)
        self._active_idx = torch.full((bsz, nheads, self.gpu_capacity), -1, dtype=torch.int32, device=dev)
        self.prefill_length = seq_len
        self.current_len = seq_len
        # a new sequence: whatever the victim cache holds belongs to the previous one
        self.ws.victim_cache(self.victim_rows_effective)

        from .factor import cast_lrqk_prefill
        A_Q, B_Q, A_K, B_K = cast_lrqk_prefill(query_states, key_states, r=self.r, lambda_Q=self.weights[0],
                                               lambda_K=self.weights[1], max_iter=self.max_iter[0], tol=self.tol[0],
                                               init_method=self.init_aq_ak_method, init_factors=self.init_factors,
                                               workspace=self.ws)
        self.init_factors = None
        self.sync_cache(B_Q, A_K, B_K)

        if seq_len <= self.gpu_capacity:
            # k <= l <= k+L: everything stays resident, the first k tokens are the selected set
            self.KVcpu.append(key_states.narrow(2, 0, k), value_states.narrow(2, 0, k))
            rem = seq_len - k
            self.lite_len = rem
            self.lite_indices = list(range(k, k + rem)) + [-1] * (L - rem)
            if rem == L:
                # A prompt of exactly k + L tokens fills the ring.  The reference leaves lite_len = L here
                # (lrqk_attention.py:1449-1452) and its next _append indexes slot L (:1188): an IndexError.  The
                # full ring is flushed instead, which is the state the reference is in when the same tokens
                # have arrived one by one (:1192-1196).
                self.KVcpu.append(key_states.narrow(2, k, L), value_states.narrow(2, k, L))
                self.lite_len = 0
            self.Kgpu.narrow(2, 0, seq_len).copy_(repeat_kv(key_states, g))
            self.Vgpu.narrow(2, 0, seq_len).copy_(repeat_kv(value_states, g))
            self._active_idx[:, :, :seq_len] = torch.arange(seq_len, dtype=torch.int32, device=dev)
            self._hit_len = k
        else:
            self._store_prompt(key_states, value_states)
            # the rows are scanned where they will live (same values as A_K, which sync_cache copied there): the
            # score index that this first scan builds then stays valid for the decode steps
            hit = self.compute_hit_indices(query_states=A_Q[:, :, -1:, :],
                                           key_states=self._A_K.data.narrow(2, 0, seq_len - L))
            self._hit_len = hit.shape[2]
            self._active_idx[:, :, :self._hit_len] = hit[..., 0].to(torch.int32)
            self.fetch_by_hit(dst=self.Kgpu_topk_area, src=key_states, hit_indices=hit)
            self.fetch_by_hit(dst=self.Vgpu_topk_area, src=value_states, hit_indices=hit)
            lb = seq_len - L
            self.lite_indices = list(range(lb, seq_len))
            self.lite_len = 0
            self.Kgpu[:, :, k:k + L, :] = repeat_kv(key_states.narrow(2, lb, L), g)
            self.Vgpu[:, :, k:k + L, :] = repeat_kv(value_states.narrow(2, lb, L), g)
            self._active_idx[:, :, k:] = torch.arange(lb, seq_len, dtype=torch.int32, device=dev)
        self.last_A_Q_row = A_Q[:, :, -1:, :]

    def _store_prompt(self, key_states: torch.Tensor, value_states: torch.Tensor):
        """The prompt's rows into the host store (what ``KVcpu.append`` does, lrqk_attention.py:959-963), written
        by a kernel straight into the pinned block as [K|V] rows: a host-side ``copy_`` into the interleaved
        layout goes through a staging copy and took 155 ms for a 128K prompt of 8 kv heads against 11 ms."""
        b, hkv, length, d = key_states.shape
        if self.KVcpu.dtype is None:
            self.KVcpu.dtype = key_states.dtype
        if self.KVcpu.device is None:
            self.KVcpu.device = torch.device("cpu")
        if not (self.KVcpu.pin_memory and key_states.is_cuda):
            self.KVcpu.append(key_states, value_states)
            return
        row0 = self.KVcpu.extend((b, hkv, 0, 2 * d), length)
        ops.flush_ring(key_states, value_states, 0, length, self.KVcpu.data, row0, hkv)

    # ------------------------------------------------------------------ decode
    def _bookkeep_append(self) -> Tuple[int, int, int]:
        """The counter updates of _append (lrqk_attention.py:1188-1196).  Returns (ring slot,
        token id, first store row to flush to or -1)."""
        slot, token = self.lite_len, self.current_len
        self.lite_indices[slot] = token
        self.lite_len += 1
        self.current_len += 1
        flush_row0 = -1
        if self.lite_len >= self.num_lite_tokens:
            b, H, n, d = self.Kgpu.shape
            flush_row0 = self.KVcpu.extend((b, H // self.num_key_value_groups, 0, 2 * d), self.num_lite_tokens)
            self.lite_len = 0
        return slot, token, flush_row0

    @torch.inference_mode()
    def decode(self, query_states: torch.Tensor, key_states: torch.Tensor, value_states: torch.Tensor):
        """lrqk_attention.py:1506-1613.  query_states [b,Hq,1,d]; key/value_states [b,Hkv,1,d].
        Returns (Kgpu, Vgpu) [b,Hq,k+L,d] (views of the persistent buffers)."""
        k, L = self.attn_topk, self.num_lite_tokens
        b, H, n, d = self.Kgpu.shape
        hkv = key_states.shape[1]
        q = query_states.contiguous()
        kn = key_states.contiguous()
        vn = value_states.contiguous()
        slot, token, flush_row0 = self._bookkeep_append()
        # room for the new k_hat row (the kernel writes it); the buffer stays zero beyond it
        row = self._A_K.extend(None, 1)
        assert row == token
        a_k = self._A_K.data
        q_hat = torch.empty((b, H, 1, self.r), dtype=a_k.dtype, device=a_k.device)
        k_hat = torch.empty_like(q_hat)
        self.last_q_hat, self.last_k_hat = q_hat, k_hat

        if self.current_len <= self.gpu_capacity:
            # growing-prefix branch (lrqk_attention.py:1526-1545): no selection yet
            self.ws.factor_state(self.use_factor_state)
            ops.append_token(kn, vn, self.Kgpu, self.Vgpu, k + slot, self._active_idx, token)
            if flush_row0 >= 0:
                ops.flush_ring(self.Kgpu, self.Vgpu, k, L, self.KVcpu.data, flush_row0, hkv)
            qh, kh = ops.als_decode(self.ws, self.B_Q, self.B_K, a_k, None, self.Kgpu, self.current_len - 1, q, kn,
                                    self.max_iter[1], self.tol[1], append_row=token)
            q_hat.copy_(qh)
            k_hat.copy_(kh)
            return self.Kgpu.narrow(2, 0, self.current_len), self.Vgpu.narrow(2, 0, self.current_len)

        m = self.lite_indices[self.lite_len] - 1
        custom = self._is_overridden("compute_hit_indices") or self._is_overridden("only_indices_in_cpu")
        if m < k or custom:
            return self._decode_staged(q, kn, vn, slot, token, flush_row0, m, q_hat, k_hat)

        evict = torch.empty((b, H, k), dtype=torch.uint8, device=a_k.device)
        miss_count = torch.empty((b, H), dtype=torch.int32, device=a_k.device)
        attn = torch.empty((b, H, 1, d), dtype=q.dtype, device=q.device) if self.attn_in_step else None
        ops.decode_step(self.ws, self.B_Q, self.B_K, a_k, self._active_idx, self.Kgpu, self.Vgpu, self.KVcpu.data, q,
                        kn, vn, topk=k, lite=L, ring_slot=slot, token=token, m=m, flush_row0=flush_row0,
                        max_iter=self.max_iter[1], tol=self.tol[1], round_scores=self.round_scores_to_storage,
                        no_hit_miss=self.no_hit_miss, q_hat=q_hat, k_hat=k_hat, attn_out=attn, evict=evict,
                        miss_count=miss_count)
        self.last_evict, self.last_miss_count, self.last_attn = evict, miss_count, attn
        return self.Kgpu, self.Vgpu

    def _decode_staged(self, q, kn, vn, slot, token, flush_row0, m, q_hat, k_hat):
        """The same step stage by stage through the overridable methods (used when a subclass
        replaces a stage, and while fewer than k candidates exist)."""
        k, L = self.attn_topk, self.num_lite_tokens
        hkv = kn.shape[1]
        a_k = self._A_K.data
        self.ws.factor_state(self.use_factor_state)   # this step changes the active set stage by stage
        ops.append_token(kn, vn, self.Kgpu, self.Vgpu, k + slot, self._active_idx, token)
        if flush_row0 >= 0:
            ops.flush_ring(self.Kgpu, self.Vgpu, k, L, self.KVcpu.data, flush_row0, hkv)
        qh, kh = ops.als_decode(self.ws, self.B_Q, self.B_K, a_k, self._active_idx, self.Kgpu, self.gpu_capacity, q, kn,
                                self.max_iter[1], self.tol[1], append_row=token)
        q_hat.copy_(qh)
        k_hat.copy_(kh)
        new = self.compute_hit_indices(query_states=q_hat, key_states=self.A_K.narrow(2, 0, m))
        if self.no_hit_miss:
            new32 = new[..., 0].to(torch.int32).contiguous()
            evict, slots, count = ops.diff(new32, self._active_idx, k=new32.shape[2], replace_all=True)
            self._hit_len = new32.shape[2]
        else:
            now = self.hit_indices
            if new.shape[2] != now.shape[2]:
                raise ValueError("shape mismatch: the resident set and the new selection differ in size")
            updated, mask = self.only_indices_in_cpu(now, new)
            self.hit_indices = updated
            evict = mask.to(torch.uint8).contiguous()
            slots, count = _slots_from_mask(evict)
        self.last_evict, self.last_miss_count = evict, count
        if self._fetch_mode == "staged":
            ops.fetch_rows_staged(self.ws, self.KVcpu.data, self.Kgpu, self.Vgpu, self._active_idx, slots, count,
                                  evict.shape[2])
        else:
            ops.fetch_rows(self.KVcpu.data, self.Kgpu, self.Vgpu, self._active_idx, slots, count, evict.shape[2])
        self.last_attn = ops.attention(self.ws, q, self.Kgpu, self.Vgpu) if self.attn_in_step else None
        return self.Kgpu, self.Vgpu

    # ------------------------------------------------------------------ statistics
    def miss_stats(self):
        """(missed rows, selected rows, host->GPU bytes) of the last decode step."""
        if self.last_miss_count is None:
            return 0, 0, 0
        n_miss = int(self.last_miss_count.sum())
        d = self.Kgpu.shape[-1]
        return n_miss, self.last_miss_count.numel() * self.attn_topk, n_miss * 2 * d * self.Kgpu.element_size()


def _as_head_strided(t: torch.Tensor):
    """Accept [b,H,m,r] views whose rows are contiguous and whose heads are a fixed number of
    rows apart; return (tensor positioned at element 0, rows between heads)."""
    b, H, m, r = t.shape
    if t.stride(3) != 1 or t.stride(2) != r:
        t = t.contiguous()
    hs = t.stride(1) if H > 1 else (t.stride(0) if b > 1 else m * r)
    if hs % r != 0 or (b > 1 and H > 1 and t.stride(0) != H * hs) or hs < m * r:
        t = t.contiguous()
        hs = m * r
    return t, hs // r


def _slots_from_mask(evict: torch.Tensor):
    """evict u8 [b,H,k] -> (miss_slots int32 [b,H,k] ascending slots first, miss_count int32 [b,H])."""
    b, H, k = evict.shape
    order = torch.argsort(1 - evict.to(torch.int32), dim=-1, stable=True).to(torch.int32)
    return order.contiguous(), evict.sum(-1, dtype=torch.int32).contiguous()


class LightAttentionIndicesOffloadPrefill(LightAttentionIndicesFactory):
    """Between a layer's prefill and its first decode, park the active set and the key
    factors in pinned host memory (lrqk_attention.py:1616-1680).  The copies run on a side
    stream and are ordered by events in both directions."""

    def prefill(self, query_states, key_states, value_states):
        super().prefill(query_states, key_states, value_states)
        dev = query_states.device
        self.stream_temp = torch.cuda.Stream(dev)
        ready = torch.cuda.Event()
        ready.record(torch.cuda.current_stream(dev))
        self._parked = {}
        with torch.cuda.stream(self.stream_temp):
            self.stream_temp.wait_event(ready)
            for name, t in (("Kgpu", self.Kgpu), ("Vgpu", self.Vgpu), ("A_K", self._A_K.data),
                            ("idx", self._active_idx)):
                host = torch.empty(t.shape, dtype=t.dtype, pin_memory=True)
                host.copy_(t, non_blocking=True)
                t.record_stream(self.stream_temp)
                self._parked[name] = host
            self._parked_done = torch.cuda.Event()
            self._parked_done.record(self.stream_temp)
        self.Kgpu = self.Vgpu = self._active_idx = None
        self._A_K.data = None

    def _restore(self, dev):
        if getattr(self, "_parked", None) is None:
            return
        with torch.cuda.stream(self.stream_temp):
            self.stream_temp.wait_event(self._parked_done)
            restored = {n: h.to(dev, non_blocking=True) for n, h in self._parked.items()}
            back = torch.cuda.Event()
            back.record(self.stream_temp)
        torch.cuda.current_stream(dev).wait_event(back)
        self.Kgpu, self.Vgpu = restored["Kgpu"], restored["Vgpu"]
        self._A_K.data, self._active_idx = restored["A_K"], restored["idx"]
        for t in restored.values():
            t.record_stream(torch.cuda.current_stream(dev))
        self._held = self._parked  # keep the pinned sources alive until the copies ran
        self._parked = None

    def decode(self, query_states, key_states, value_states):
        self._restore(query_states.device)
        return super().decode(query_states, key_states, value_states)


class LightAttentionIndicesNoHitMiss(LightAttentionIndicesFactory):
    """Ablation: no resident-set bookkeeping, all k rows are refetched every step
    (lrqk_attention.py:1683-1775)."""
    no_hit_miss = True
