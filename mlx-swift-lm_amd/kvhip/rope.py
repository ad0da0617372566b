"""Rotary position embedding in front of the cache write.

`RoPE` mirrors the layer the reference's models hold (`MLXNN.RoPE(dimensions:traditional:base:scale:)`
and the `freqs`-carrying variants `Llama3RoPE`, `YarnRoPE`, `SuScaledRoPE`, RoPEUtils.swift:86-160,
SuScaledRoPE.swift:8-70, all ending in `MLXFast.RoPE`); `apply_rotary_position` is
`applyRotaryPosition(_:to:offset:)` (RoPEApplication.swift:62-74) for queries, and
`attention_with_rope_and_cache_update` is the call sequence of an attention layer
(Llama.swift:58-70) with the key rotation folded into the append kernel.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib as L
from .cache import MaskMode, _DT, _ptr, _stream


class RoPE:
    def __init__(self, dims, traditional=False, base=10000.0, scale=1.0, freqs=None):
        self.dims, self.traditional, self.base, self.scale = int(dims), bool(traditional), float(base), float(scale)
        self.freqs = None if freqs is None else torch.as_tensor(freqs, dtype=torch.float32).to("cuda").contiguous()
        if self.freqs is not None:
            assert self.freqs.numel() == self.dims // 2

    def to_c(self):
        r = L.Rope(self.dims, int(self.traditional), self.base, self.scale,
                   self.freqs.data_ptr() if self.freqs is not None else None)
        return r, self.freqs

    def __call__(self, x, offset=0):
        return apply_rotary_position(self, x, offset)


def apply_rotary_position(rope, x, offset=None):
    """x [B,H,L,D] rotated at positions offset + l; `offset` is None (0), an int, a cache
    (its `ropeOffset`) or an int32 tensor [B] (`RoPEOffset.batch`)."""
    lib = L.load()
    x = x.contiguous()
    B, H, Lq, D = x.shape
    out = torch.empty_like(x)
    r, keep = rope.to_c()
    bo = None
    if offset is None:
        pos = 0
    elif torch.is_tensor(offset):
        bo, pos = offset.to(device="cuda", dtype=torch.int32).contiguous(), 0
    elif hasattr(offset, "rope_offset"):
        pos = offset.rope_offset
    else:
        pos = int(offset)
    L.check(lib.kvhip_rope_apply(C.byref(r), _ptr(x), _ptr(out), B, H, Lq, D, _DT[x.dtype], int(pos),
                                 _ptr(bo) if bo is not None else None, _stream()))
    del keep
    return out


def attention_with_rope_and_cache_update(rope, queries, keys, values, cache, scale, mask=None, batch_offsets=None):
    """Rotate queries and keys at the cache's `ropeOffset`, write the cache, attend
    (Llama.swift:58-70 + AttentionUtils.swift:37-95): one launch for the queries, one fused
    rotate-and-append (or rotate-quantize-append) for the keys and values, one for attention."""
    offset = batch_offsets if batch_offsets is not None else cache.rope_offset
    q = apply_rotary_position(rope, queries, offset)
    cache.update_rope(rope, keys, values, batch_offsets)
    return cache.attend(q, scale, mask or MaskMode.none())
