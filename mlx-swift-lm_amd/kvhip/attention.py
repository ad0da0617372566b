"""`attentionWithCacheUpdate` (AttentionUtils.swift:37-95) over libkvhip caches."""
from __future__ import annotations

from .cache import MaskMode, QuantizedKVCache


def attention_with_cache_update(queries, keys, values, cache, scale, mask=None):
    """Update `cache` with the new keys/values and attend; returns [B,Hq,L,Dv].

    Quantized caches take the `updateQuantized` + `quantizedScaledDotProductAttention`
    branch (AttentionUtils.swift:72-85), others `update` + fused SDPA (:86-93); both
    run as one C-ABI call, kvhip_cache_update_attend.
    """
    if cache is None:
        raise ValueError("a kvhip cache is required; cache-less attention is outside this path")
    return cache.update_attend(queries, keys, values, scale, mask or MaskMode.none())


def quantized_scaled_dot_product_attention(queries, cache: QuantizedKVCache, scale, mask=None):
    """`quantizedScaledDotProductAttention` (KVCache.swift:2351-2447) over the rows
    `cache` already holds (the quantized tuples stay in device pages)."""
    return cache.attend(queries, scale, mask or MaskMode.none())
