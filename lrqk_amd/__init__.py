"""MI355X-native LRQK decode path: the reference's cache / engine interface backed by
hand-written gfx950 kernels (liblrqk_hip.so)."""
from .buffers import AutoIncreaseTensor, AutoIncreaseTensorSharedKV, PreAllocatedTensor, _CacheQKV
from .cache import DynamicLRQKCache
from .engine import (LightAttentionIndicesFactory, LightAttentionIndicesNoHitMiss,
                     LightAttentionIndicesOffloadPrefill)
from .factor import InitAQAK, cast_lrqk_decode, cast_lrqk_prefill, repeat_kv

__all__ = [
    "AutoIncreaseTensor", "AutoIncreaseTensorSharedKV", "PreAllocatedTensor", "_CacheQKV", "DynamicLRQKCache",
    "LightAttentionIndicesFactory", "LightAttentionIndicesNoHitMiss", "LightAttentionIndicesOffloadPrefill",
    "InitAQAK", "cast_lrqk_decode", "cast_lrqk_prefill", "repeat_kv",
]
