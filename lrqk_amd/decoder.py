"""A Llama-shaped decoder stack around the LRQK cache, for end-to-end tokens/s.

Only the call pattern matters here: every layer calls ``cache.update(q, k, v, layer)`` exactly
as the reference's patched attention does (lrqk_attention.py:2254-2290, 2326-2344) -- raw K/V
and ordinary causal attention over the prompt, the active set ``[b,Hq,k+L,d]`` and exact
single-query attention per decoded token.  Projections, norms, rotary embedding, SwiGLU and the
prompt attention are plain PyTorch-ROCm library calls on random-initialised weights; the
cache path (factorisation, selection, fetch, decode attention) is the HIP library.

``cache=None`` runs the same module with a dense K/V cache; with ``k + lite`` at least as long as
the whole sequence the LRQK run returns every cached token (the growing-prefix branch,
lrqk_attention.py:1526-1545) and must produce the same tokens.
"""
from __future__ import annotations

import math
import time
from dataclasses import dataclass
from typing import List, Optional, Tuple

import torch
import torch.nn.functional as F

from . import ops
from .cache import DynamicLRQKCache


@dataclass
class DecoderConfig:
    layers: int = 32
    hidden: int = 4096
    heads: int = 32
    kv_heads: int = 8
    head_dim: int = 128
    intermediate: int = 14336
    vocab: int = 128256
    rope_theta: float = 5e5
    rms_eps: float = 1e-5


LLAMA3_8B = DecoderConfig()


def _rms(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    v = x.float()
    v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
    return (v * w.float()).to(x.dtype)


class LlamaShapeDecoder:
    def __init__(self, cfg: DecoderConfig = LLAMA3_8B, dtype=torch.bfloat16, device="cuda:0", seed: int = 0,
                 mlp_chunk: int = 16384, context_scale: float = 0.0):
        """``context_scale`` > 0 adds a fixed direction of that length (in units of an embedding's length) to every
        token embedding.  With random weights and random ids the hidden states of successive positions are
        unrelated, so every decode step selects a fresh set of tokens; a shared component makes successive
        queries (and all keys) correlated, as the residual stream of a trained model does, and the selection then
        drifts slowly from step to step -- the regime the cache is built for."""
        self.cfg, self.dtype, self.device = cfg, dtype, torch.device(device)
        self.mlp_chunk = mlp_chunk
        self.context_scale = context_scale
        g = torch.Generator(device=self.device).manual_seed(seed)

        def w(*shape, std=0.02):
            return (torch.randn(shape, generator=g, device=self.device, dtype=torch.float32) * std).to(dtype)

        c = cfg
        self.embed = w(c.vocab, c.hidden)
        ctx = torch.randn((c.hidden,), generator=g, device=self.device, dtype=torch.float32)
        self.context = (ctx / ctx.norm() * (0.02 * math.sqrt(c.hidden)) * context_scale).to(dtype)
        self.lm_head = w(c.hidden, c.vocab)
        self.final_norm = torch.ones(c.hidden, dtype=dtype, device=self.device)
        self.layers = []
        for _ in range(c.layers):
            self.layers.append(dict(
                n1=torch.ones(c.hidden, dtype=dtype, device=self.device),
                n2=torch.ones(c.hidden, dtype=dtype, device=self.device),
                wq=w(c.hidden, c.heads * c.head_dim), wk=w(c.hidden, c.kv_heads * c.head_dim),
                wv=w(c.hidden, c.kv_heads * c.head_dim), wo=w(c.heads * c.head_dim, c.hidden),
                wg=w(c.hidden, c.intermediate), wu=w(c.hidden, c.intermediate), wd=w(c.intermediate, c.hidden)))
        half = c.head_dim // 2
        self.inv_freq = 1.0 / (c.rope_theta ** (torch.arange(0, half, device=self.device, dtype=torch.float32) / half))
        self.ws = ops.Workspace()
        self.dense: Optional[List[Tuple[torch.Tensor, torch.Tensor]]] = None
        self.progress = None   # optional callable(str), called once per layer while the prompt is processed
        self.path_events = None  # a list: decode steps append an event pair around each layer's cache path

    # ------------------------------------------------------------------ pieces
    def _rope(self, x: torch.Tensor, pos0: int) -> torch.Tensor:
        """x [b,H,s,d]; rotate-half convention, positions pos0 .. pos0+s-1."""
        s, d = x.shape[2], x.shape[3]
        ang = torch.arange(pos0, pos0 + s, device=x.device, dtype=torch.float32)[:, None] * self.inv_freq[None, :]
        cos, sin = torch.cos(ang), torch.sin(ang)
        x1, x2 = x[..., :d // 2].float(), x[..., d // 2:].float()
        return torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1).to(x.dtype)

    def _mlp(self, L, x: torch.Tensor) -> torch.Tensor:
        out = torch.empty_like(x)
        flat, oflat = x.view(-1, x.shape[-1]), out.view(-1, x.shape[-1])
        for i in range(0, flat.shape[0], self.mlp_chunk):
            t = flat[i:i + self.mlp_chunk]
            oflat[i:i + self.mlp_chunk] = (F.silu(t @ L["wg"]) * (t @ L["wu"])) @ L["wd"]
        return out

    def new_cache(self, r=32, num_active_tokens=2048, lite_tokens=64, max_iter=(2, 2), tol=(1e-2, 1e-2),
                  max_sequence_length=4096) -> DynamicLRQKCache:
        return DynamicLRQKCache(r=r, num_active_tokens=num_active_tokens, lite_tokens=lite_tokens, max_iter=max_iter,
                                tol=tol, max_sequence_length=max_sequence_length,
                                num_key_value_groups=self.cfg.heads // self.cfg.kv_heads)

    # ------------------------------------------------------------------ one forward over s new positions
    @torch.inference_mode()
    def forward(self, ids: torch.Tensor, pos0: int, cache: Optional[DynamicLRQKCache]) -> torch.Tensor:
        """ids [b,s] -> logits of the last position [b,vocab]."""
        c = self.cfg
        b, s = ids.shape
        x = self.embed[ids]
        if self.context_scale:
            x = x + self.context
        if cache is None and self.dense is None:
            self.dense = [None] * c.layers
        for li, L in enumerate(self.layers):
            hcur = _rms(x, L["n1"], c.rms_eps)
            q = (hcur @ L["wq"]).view(b, s, c.heads, c.head_dim).transpose(1, 2)
            k = (hcur @ L["wk"]).view(b, s, c.kv_heads, c.head_dim).transpose(1, 2)
            v = (hcur @ L["wv"]).view(b, s, c.kv_heads, c.head_dim).transpose(1, 2).contiguous()
            q, k = self._rope(q, pos0).contiguous(), self._rope(k, pos0).contiguous()
            if cache is None:
                if self.dense[li] is None:
                    self.dense[li] = (k, v)
                else:
                    self.dense[li] = (torch.cat([self.dense[li][0], k], 2), torch.cat([self.dense[li][1], v], 2))
                K, V = self.dense[li]
                o = F.scaled_dot_product_attention(q, K, V, is_causal=s > 1, enable_gqa=True)
            elif s > 1:
                cache.update(q, k, v, li)   # factorises the prompt; the prompt itself attends densely
                o = F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
            else:
                eng = cache.lwattn[li]
                eng.attn_in_step = True
                eng.last_attn = None
                if self.path_events is not None:
                    e0 = torch.cuda.Event(enable_timing=True)
                    e0.record()
                K, V = cache.update(q, k, v, li)
                if eng.last_attn is not None:
                    o = eng.last_attn
                else:   # prefix / edge branches return a view of the first n slots of the persistent buffers
                    o = ops.attention(self.ws, q, eng.Kgpu, eng.Vgpu, n_valid=K.shape[2])
                if self.path_events is not None:
                    e1 = torch.cuda.Event(enable_timing=True)
                    e1.record()
                    self.path_events.append((e0, e1))
            x = x + o.transpose(1, 2).reshape(b, s, c.heads * c.head_dim) @ L["wo"]
            x = x + self._mlp(L, _rms(x, L["n2"], c.rms_eps))
            if s > 1 and self.progress is not None:
                self.progress(f"prompt: layer {li + 1}/{c.layers}")
        last = _rms(x[:, -1], self.final_norm, c.rms_eps)
        return (last @ self.lm_head).float()

    @torch.inference_mode()
    def generate(self, ids: torch.Tensor, new_tokens: int, cache: Optional[DynamicLRQKCache]):
        """Greedy decoding.  Returns (tokens [b,new_tokens], prefill seconds, decode seconds, per-step seconds)."""
        self.dense = None
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        tok = self.forward(ids, 0, cache).argmax(-1)
        torch.cuda.synchronize()
        t_prefill = time.perf_counter() - t0
        out = [tok]
        steps = []
        pos = ids.shape[1]
        t0 = time.perf_counter()
        for _ in range(new_tokens - 1):
            t1 = time.perf_counter()
            tok = self.forward(tok[:, None], pos, cache).argmax(-1)
            out.append(tok)
            pos += 1
            steps.append(time.perf_counter() - t1)
        torch.cuda.synchronize()
        t_decode = time.perf_counter() - t0
        return torch.stack(out, 1), t_prefill, t_decode, steps
