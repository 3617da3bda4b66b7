"""Growable and pre-allocated token buffers (interface of lrqk_attention.py:844-1028).

The layouts are part of the kernel contract: the rank-r key factors live on the GPU as
``[b, Hq, capacity, r]`` and the full-precision store lives in pinned host memory as
``[b, Hkv, capacity, 2*d]`` with the K row followed by the V row.  Buffers are
zero-initialised up to their capacity: the decode step gathers the not-yet-written row of
the newest token and relies on reading zeros there.
"""
from __future__ import annotations

from typing import Optional

import torch


class AutoIncreaseTensor:
    """Buffer that grows by ``scaling_ratio`` along ``dim`` (lrqk_attention.py:844-957)."""

    def __init__(self, capacity: int = 4096, dim: int = 0, scaling_ratio: float = 1.5,
                 device: Optional[torch.device] = None, dtype: Optional[torch.dtype] = None,
                 pin_memory: bool = False):
        self.capacity = capacity
        self.dim = dim
        self.scaling_ratio = scaling_ratio
        self.device = device
        self.dtype = dtype
        self.data: Optional[torch.Tensor] = None
        self.current_len = 0
        self.pin_memory = pin_memory

    # -- allocation policy (first allocation :877-889, growth :892-920)
    def _alloc(self, shape):
        pin = bool(self.pin_memory) and torch.cuda.is_available()
        return torch.zeros(shape, device=self.device, dtype=self.dtype, pin_memory=pin)

    def _ensure(self, like_shape, length: int):
        target = self.current_len + length
        if self.data is None:
            cap = max(self.capacity, int(length * self.scaling_ratio))
            shape = list(like_shape)
            shape[self.dim] = cap
            self.data = self._alloc(shape)
            self.capacity = cap
        elif target >= self.capacity:
            cap = self.capacity
            while cap <= target:
                cap = int(cap * self.scaling_ratio)
            shape = list(self.data.shape)
            shape[self.dim] = cap
            grown = self._alloc(shape)
            if self.pin_memory and torch.cuda.is_available():
                # kernels may still be writing flushed rows into (or fetching rows from) the old
                # pinned block; the host copy below and the release of the block must wait
                torch.cuda.synchronize()
            if self.current_len:
                grown.narrow(self.dim, 0, self.current_len).copy_(self.data.narrow(self.dim, 0, self.current_len))
            self.data = grown
            self.capacity = cap

    @torch.inference_mode()
    def append(self, x: torch.Tensor):
        if self.device is None:
            self.device = x.device
        if self.dtype is None:
            self.dtype = x.dtype
        length = x.size(self.dim)
        self._ensure(x.shape, length)
        self.data.narrow(self.dim, self.current_len, length).copy_(x)
        self.current_len += length

    @torch.inference_mode()
    def extend(self, like_shape, length: int) -> int:
        """Make room for ``length`` more entries exactly as ``append`` would, without writing
        them (a kernel fills the rows).  Returns the index of the first new entry."""
        self._ensure(like_shape, length)
        first = self.current_len
        self.current_len += length
        return first

    def has_data(self):
        return self.data is not None

    @property
    def shape(self) -> torch.Size:
        s = list(self.data.shape)
        s[self.dim] = self.current_len
        return torch.Size(s)

    def tensor(self) -> torch.Tensor:
        return self.data.narrow(self.dim, 0, self.current_len)

    def __len__(self):
        return self.current_len

    def __getitem__(self, idx):
        if self.data is None:
            raise IndexError("Cache is empty")
        return self.tensor()[idx]

    def take_along_dim(self, indices: torch.Tensor, dim: int = None, out=None) -> torch.Tensor:
        """Gather on the FULL-capacity buffer (lrqk_attention.py:952-956)."""
        if self.data is None:
            raise IndexError("Cache is empty")
        return torch.take_along_dim(self.data, indices, self.dim if dim is None else dim, out=out)


class AutoIncreaseTensorSharedKV(AutoIncreaseTensor):
    """K and V rows side by side on the last dim (lrqk_attention.py:959-963)."""

    def _alloc(self, shape):
        # Rows at and beyond current_len are never read (every access goes through a token id below it or
        # through tensor()), so the store is not cleared: clearing 0.8 GB of pinned memory is 4 ms of a
        # 128K layer prefill.  (The factor buffer keeps the zero fill: it is gathered at full capacity.)
        pin = bool(self.pin_memory) and torch.cuda.is_available()
        return torch.empty(shape, device=self.device, dtype=self.dtype, pin_memory=pin)

    @torch.inference_mode()
    def append(self, k: torch.Tensor, v: torch.Tensor):
        if self.dtype is None:
            self.dtype = k.dtype
        if self.device is None:
            self.device = torch.device("cpu")
        length = k.size(self.dim)
        d = k.size(-1)
        shape = list(k.shape)
        shape[-1] = 2 * d
        self._ensure(shape, length)
        dst = self.data.narrow(self.dim, self.current_len, length)
        dst.narrow(-1, 0, d).copy_(k)
        dst.narrow(-1, d, d).copy_(v)
        self.current_len += length


class PreAllocatedTensor:
    """Bounded buffer along ``dim`` (interface of lrqk_attention.py:966-1011: ``capacity``, ``dim``,
    ``dtype``, ``device``, ``data``, ``current_len``; ``append`` past the capacity raises ``ValueError``).
    Storage appears with the first piece and takes its shape, dtype and device from it unless given."""

    def __init__(self, capacity: int, dim: int, dtype: torch.dtype = None, device: torch.device = None):
        self.capacity, self.dim = capacity, dim
        self.dtype, self.device = dtype, device
        self.data, self.current_len = None, 0

    @classmethod
    def from_tensor(cls, capacity: int, dim: int, data: torch.Tensor):
        buf = cls(capacity, dim, dtype=data.dtype, device=data.device)
        buf.append(data)
        return buf

    def _window(self, start: int, length: int) -> torch.Tensor:
        return self.data.narrow(self.dim, start, length)

    def append(self, x: torch.Tensor):
        self.dtype = x.dtype if self.dtype is None else self.dtype
        self.device = x.device if self.device is None else self.device
        if self.data is None:
            full = [self.capacity if ax == self.dim else size for ax, size in enumerate(x.shape)]
            self.data = torch.empty(full, dtype=self.dtype, device=self.device)
        end = self.current_len + x.shape[self.dim]
        if end > self.capacity:
            raise ValueError("Not enough capacity to store the tensor")
        self._window(self.current_len, end - self.current_len).copy_(x)
        self.current_len = end

    def has_data(self):
        return self.data is not None

    def tensor(self) -> torch.Tensor:
        return self._window(0, self.current_len)

    def __len__(self):
        return self.current_len

    def __getitem__(self, idx):
        return self.tensor()[idx]


class _CacheQKV:
    """The pieces of a prompt that is still shorter than the active set (interface of
    lrqk_attention.py:1014-1028: members ``Q``, ``K``, ``V``; ``append`` returns what has been
    collected so far; ``len`` is the number of positions held)."""

    _NAMES = ("Q", "K", "V")

    def __init__(self, capacity: int, dim: int, dtype: torch.dtype = None, device: torch.device = None):
        for name in self._NAMES:
            setattr(self, name, PreAllocatedTensor(capacity, dim, dtype, device))

    def append(self, Q: torch.Tensor, K: torch.Tensor, V: torch.Tensor):
        held = []
        for name, piece in zip(self._NAMES, (Q, K, V)):
            buf = getattr(self, name)
            buf.append(piece)
            held.append(buf.tensor())
        return tuple(held)

    def __len__(self):
        return len(self.Q)
