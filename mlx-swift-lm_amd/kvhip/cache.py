"""Host-side mirror of the reference's cache classes over libkvhip.

Class and member names follow Libraries/MLXLMCommon/KVCache.swift
(`KVCacheSimple` :391, `RotatingKVCache` :541, `QuantizedKVCache` :923); the
arrays are torch tensors on the GPU, used only as device memory.  Every method
is a thin call into the C ABI: the cached rows never leave the device unless a
caller asks for `state`, `fetch()` or `logical_view()`.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib as L

_DT = {torch.float16: L.F16, torch.bfloat16: L.BF16, torch.float32: L.F32}
_TORCH = {L.F16: torch.float16, L.BF16: torch.bfloat16, L.F32: torch.float32, L.U32: torch.int32,
          L.BOOL: torch.bool}


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return C.c_void_p(t.data_ptr())


class MaskMode:
    """`MLXFast.ScaledDotProductAttentionMaskMode`: .none / .causal / .array(mask),
    plus .window -- createCausalMask evaluated from indices inside the kernel."""

    def __init__(self, mode, array=None, offset=0, window=0, lengths=None, left_pad=None, plan=None):
        self.mode, self._array, self._plan = mode, array, plan
        self.offset, self.window, self.lengths, self.left_pad = offset, window, lengths, left_pad

    @property
    def array(self):
        """The boolean array of an `.array` mask; a mask planned by `make_mask` and evaluated from
        indices builds it (on the device) only when somebody asks for it."""
        if self._array is None and self._plan is not None:
            p = self._plan
            buf = torch.empty((p.rows, p.cols), dtype=torch.uint8, device="cuda")
            L.check(L.load().kvhip_mask_materialize(C.byref(p), _ptr(buf), _stream()))
            self._array = buf.bool()
        return self._array

    @staticmethod
    def none():
        return MaskMode(L.MASK_NONE)

    @staticmethod
    def causal():
        return MaskMode(L.MASK_CAUSAL)

    @staticmethod
    def from_array(a):
        return MaskMode(L.MASK_ARRAY, array=a)

    @staticmethod
    def window_mask(offset, window=0, lengths=None, left_pad=None):
        return MaskMode(L.MASK_WINDOW, offset=offset, window=window, lengths=lengths, left_pad=left_pad)

    def to_c(self, B, Hq, Lq):
        m = L.Mask()
        m.mode = self.mode
        keep = []
        if self.mode == L.MASK_ARRAY:
            a = self.array
            if a.dtype == torch.bool:
                a8 = a.to(torch.uint8).contiguous()
                m.dtype = L.BOOL
            else:
                a8 = a.contiguous()
                m.dtype = _DT[a.dtype]
            while a8.dim() < 4:
                a8 = a8.unsqueeze(0)
            assert a8.shape[2] == Lq, "mask query extent"
            assert a8.shape[0] in (1, B) and a8.shape[1] in (1, Hq)
            st = a8.stride()
            m.stride_b = 0 if a8.shape[0] == 1 else st[0]
            m.stride_h = 0 if a8.shape[1] == 1 else st[1]
            m.stride_l = st[2]
            m.key_len = a8.shape[3]
            m.data = a8.data_ptr()
            keep.append(a8)
        elif self.mode == L.MASK_WINDOW:
            m.offset, m.window = int(self.offset), int(self.window or 0)
            for name in ("lengths", "left_pad"):
                t = getattr(self, name)
                if t is not None:
                    t = t.to(device="cuda", dtype=torch.int32).contiguous()
                    setattr(m, name, t.data_ptr())
                    keep.append(t)
        return m, keep


class _Cache:
    kind = None

    def __init__(self, handle=None, **cfg):
        L.init()
        self._lib = L.load()
        if handle is None:
            c = L.Config(kind=self.kind, step=cfg.get("step", 0), max_size=cfg.get("max_size", 0),
                         keep=cfg.get("keep", 0), group_size=cfg.get("group_size", 0), bits=cfg.get("bits", 0))
            h = C.c_void_p()
            L.check(self._lib.kvhip_cache_create(C.byref(c), C.byref(h)))
            handle = h
        self._h = handle
        self._shape = None  # (B, Hkv, Dk, Dv, torch dtype) once known

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.kvhip_cache_free(h)

    # ---- protocol surface -------------------------------------------------
    @property
    def offset(self):
        return self._lib.kvhip_cache_offset(self._h)

    @offset.setter
    def offset(self, v):
        L.check(self._lib.kvhip_cache_set_offset(self._h, int(v)))

    @property
    def rope_offset(self):
        """`ropeOffset` (KVCache.swift:190): `.scalar(offset)`, read before the write."""
        return self.offset

    @property
    def max_size(self):
        v = self._lib.kvhip_cache_max_size(self._h)
        return None if v < 0 else v

    @property
    def capacity(self):
        return self._lib.kvhip_cache_capacity(self._h)

    @property
    def device_rows(self):
        """Rows the device pages allocated so far can hold."""
        return self._lib.kvhip_cache_device_rows(self._h)

    @property
    def slot_span(self):
        """Device slots a decode launch walks (one past the highest slot holding a presented row)."""
        return self._lib.kvhip_cache_slot_span(self._h)

    @property
    def presented_length(self):
        return self._lib.kvhip_cache_presented_length(self._h)

    @property
    def is_trimmable(self):
        return bool(self._lib.kvhip_cache_is_trimmable(self._h, 0))

    def is_trimmable_after(self, positions):
        return bool(self._lib.kvhip_cache_is_trimmable(self._h, int(positions)))

    def trim(self, n):
        return self._lib.kvhip_cache_trim(self._h, int(n))

    def prepare(self, lengths=None):
        """`prepare(lengths:)` (KVCache.swift:96-99): a hook for batched caches; these three
        kinds keep the protocol's empty default (:114-116)."""

    def finalize(self):
        """`finalize()` (KVCache.swift:102, default :118): nothing transient to clear."""

    def inner_state(self):
        """`innerState()` (KVCache.swift:400-402, :572-574, :939-948): the arrays `eval(cache)`
        materialises.  The rows already live on the device; their export is `state`."""
        return self.state

    def eval(self):
        """`eval(cache)` (LLMModel.swift:52-58): wait for the work enqueued on the current stream."""
        L.check(self._lib.kvhip_sync(_stream()))

    def reserve(self, B, Hkv, Dk, Dv, dtype, tokens):
        L.check(self._lib.kvhip_cache_reserve(self._h, B, Hkv, Dk, Dv, _DT[dtype], int(tokens)))

    def _note_shape(self, keys, values):
        B, H, _, Dk = keys.shape
        self._shape = (B, H, Dk, values.shape[3], keys.dtype)

    def _update(self, keys, values):
        assert keys.is_cuda and values.is_cuda and keys.dtype == values.dtype
        keys, values = keys.contiguous(), values.contiguous()
        B, H, Lq, Dk = keys.shape
        L.check(self._lib.kvhip_cache_update(self._h, _ptr(keys), _ptr(values), B, H, Lq, Dk,
                                             values.shape[3], _DT[keys.dtype], _stream()))
        self._note_shape(keys, values)

    def update_rope(self, rope, keys, values, batch_offsets=None):
        """`update` / `updateQuantized` of keys that still need their rotary embedding: the
        rotation runs inside the append kernel, at positions starting from this cache's
        `ropeOffset` (its offset before the write) or from `batch_offsets` [B] (int32)."""
        assert keys.is_cuda and values.is_cuda and keys.dtype == values.dtype
        keys, values = keys.contiguous(), values.contiguous()
        B, H, Lq, Dk = keys.shape
        r, keep = rope.to_c()
        bo = None if batch_offsets is None else batch_offsets.to(device="cuda", dtype=torch.int32).contiguous()
        L.check(self._lib.kvhip_cache_update_rope(self._h, C.byref(r), _ptr(bo) if bo is not None else None,
                                                  _ptr(keys), _ptr(values), B, H, Lq, Dk, values.shape[3],
                                                  _DT[keys.dtype], _stream()))
        self._note_shape(keys, values)
        del keep

    def _check_query_dtype(self, q, k=None):
        # the C entry points carry no dtype for queries / out: they are read as the cache's dtype
        want = k.dtype if k is not None else (self._shape[4] if self._shape else q.dtype)
        if q.dtype != want or (k is not None and self._shape and k.dtype != self._shape[4]):
            raise TypeError(f"queries are {q.dtype}, keys {k.dtype if k is not None else want}, "
                            f"the cache holds {self._shape[4] if self._shape else want}")

    def attend(self, queries, scale, mask=None, out=None, static_scratch=False):
        """Attention of `queries` [B,Hq,L,D] over what the cache presents.  With `static_scratch` the
        call goes through the allocation-free entry point (`kvhip_cache_attend_static`); pass `out`
        too if the caller must not allocate at all."""
        q = queries.contiguous()
        self._check_query_dtype(q)
        B, Hq, Lq, D = q.shape
        Dv = self._shape[3]
        if out is None:
            out = torch.empty((B, Hq, Lq, Dv), dtype=q.dtype, device=q.device)
        assert out.is_contiguous() and tuple(out.shape) == (B, Hq, Lq, Dv) and out.dtype == q.dtype
        mask = mask or MaskMode.none()
        m, keep = mask.to_c(B, Hq, Lq)
        fn = self._lib.kvhip_cache_attend_static if static_scratch else self._lib.kvhip_cache_attend
        L.check(fn(self._h, _ptr(q), B, Hq, Lq, D, float(scale), C.byref(m), _ptr(out), _stream()))
        del keep
        return out

    def update_attend(self, queries, keys, values, scale, mask=None):
        """`attentionWithCacheUpdate` for this cache (AttentionUtils.swift:37-95)."""
        q, k, v = queries.contiguous(), keys.contiguous(), values.contiguous()
        self._check_query_dtype(q, k)
        B, Hq, Lq, D = q.shape
        H = k.shape[1]
        out = torch.empty((B, Hq, Lq, v.shape[3]), dtype=q.dtype, device=q.device)
        mask = mask or MaskMode.none()
        m, keep = mask.to_c(B, Hq, Lq)
        L.check(self._lib.kvhip_cache_update_attend(self._h, _ptr(q), _ptr(k), _ptr(v), B, Hq, H, Lq, D,
                                                    v.shape[3], _DT[k.dtype], float(scale), C.byref(m),
                                                    _ptr(out), _stream()))
        self._note_shape(k, v)
        del keep
        return out

    def make_mask(self, n, window_size=None, return_array=False):
        """`makeMask(n:windowSize:returnArray:)`; array masks are built on the device."""
        p = L.MaskPlan()
        L.check(self._lib.kvhip_cache_mask_plan(self._h, int(n), int(window_size or 0), int(return_array), C.byref(p)))
        if p.mode == L.MASK_NONE:
            return MaskMode.none()
        if p.mode == L.MASK_CAUSAL:
            return MaskMode.causal()
        if not p.rolled:
            # createCausalMask(n, offset, windowSize) (KVCache.swift:253-275) is a function of the
            # indices: the kernels evaluate it in place, and `.array` materialises it on demand
            return MaskMode(L.MASK_WINDOW, offset=p.offset, window=p.window, plan=p)
        shape = (p.cols,)
        buf = torch.empty(shape, dtype=torch.uint8, device="cuda")
        L.check(self._lib.kvhip_mask_materialize(C.byref(p), _ptr(buf), _stream()))
        return MaskMode.from_array(buf.bool())

    # ---- state / metaState ---------------------------------------------------
    @property
    def state(self):
        n = self._lib.kvhip_cache_state_count(self._h)
        out = []
        for i in range(n):
            shape = (C.c_int64 * 4)()
            dt = C.c_int32()
            L.check(self._lib.kvhip_cache_state_desc(self._h, i, C.byref(shape), C.byref(dt)))
            t = torch.empty(tuple(shape), dtype=_TORCH[dt.value], device="cuda")
            L.check(self._lib.kvhip_cache_state_export(self._h, i, _ptr(t), _stream()))
            out.append(t)
        return out

    @state.setter
    def state(self, arrays):
        arrays = [a.contiguous() for a in arrays]
        n = len(arrays)
        ptrs = (C.c_void_p * max(n, 1))(*[a.data_ptr() for a in arrays])
        shapes = (C.c_int64 * (4 * max(n, 1)))(*[d for a in arrays for d in a.shape])
        dts = (C.c_int32 * max(n, 1))(*[L.U32 if a.dtype in (torch.int32, torch.uint32) else _DT[a.dtype] for a in arrays])
        L.check(self._lib.kvhip_cache_state_import(self._h, n, ptrs, shapes, dts, _stream()))
        torch.cuda.current_stream().synchronize()
        if self.kind == L.KIND_QUANTIZED:
            bits = self.bits
            self._shape = (arrays[0].shape[0], arrays[0].shape[1], arrays[0].shape[3] * 32 // bits,
                           arrays[3].shape[3] * 32 // bits, arrays[1].dtype)
        else:
            self._shape = (arrays[0].shape[0], arrays[0].shape[1], arrays[0].shape[3], arrays[1].shape[3],
                           arrays[0].dtype)

    @property
    def meta_state(self):
        out = []
        buf = C.create_string_buffer(64)
        for i in range(self._lib.kvhip_cache_meta_count(self._h)):
            L.check(self._lib.kvhip_cache_meta_get(self._h, i, buf, 64))
            out.append(buf.value.decode())
        return out

    @meta_state.setter
    def meta_state(self, values):
        arr = (C.c_char_p * len(values))(*[v.encode() for v in values])
        L.check(self._lib.kvhip_cache_meta_set(self._h, len(values), arr))

    def copy(self):
        h = C.c_void_p()
        L.check(self._lib.kvhip_cache_copy(self._h, _stream(), C.byref(h)))
        new = type(self).__new__(type(self))
        _Cache.__init__(new, handle=h)
        new._shape = self._shape
        return new


class KVCacheSimple(_Cache):
    """`KVCacheSimple` (KVCache.swift:391-538)."""
    kind = L.KIND_SIMPLE

    def __init__(self, step=256, handle=None):
        super().__init__(handle=handle, step=step)

    def update(self, keys, values, fetch=True):
        """`update(keys:values:)`: returns all cached keys/values (copied out of the
        page layout when `fetch` is true; attention does not need that copy)."""
        self._update(keys, values)
        return self.fetch() if fetch else None

    def fetch(self):
        B, H, Dk, Dv, dt = self._shape
        n = self.presented_length
        k = torch.empty((B, H, n, Dk), dtype=dt, device="cuda")
        v = torch.empty((B, H, n, Dv), dtype=dt, device="cuda")
        L.check(self._lib.kvhip_cache_fetch(self._h, _ptr(k), _ptr(v), _stream()))
        return k, v

    def to_quantized(self, group_size=64, bits=4):
        h = C.c_void_p()
        L.check(self._lib.kvhip_cache_to_quantized(self._h, group_size, bits, _stream(), C.byref(h)))
        q = QuantizedKVCache.__new__(QuantizedKVCache)
        _Cache.__init__(q, handle=h)
        q._shape = self._shape
        return q


class RotatingKVCache(KVCacheSimple):
    """`RotatingKVCache` (KVCache.swift:541-900)."""
    kind = L.KIND_ROTATING

    def __init__(self, max_size, keep=0, step=256, handle=None):
        _Cache.__init__(self, handle=handle, max_size=max_size, keep=keep, step=step)

    @property
    def idx(self):
        return self._lib.kvhip_cache_idx(self._h)

    def logical_view(self, tail):
        """`logicalView(tail:)` (KVCache.swift:631-658); None before the first write."""
        if self._shape is None or self._lib.kvhip_cache_state_count(self._h) == 0:
            return None
        n = C.c_int64()
        L.check(self._lib.kvhip_cache_logical_view(self._h, int(tail), C.byref(n), None, None, _stream()))
        B, H, Dk, Dv, dt = self._shape
        k = torch.empty((B, H, n.value, Dk), dtype=dt, device="cuda")
        v = torch.empty((B, H, n.value, Dv), dtype=dt, device="cuda")
        if n.value:
            L.check(self._lib.kvhip_cache_logical_view(self._h, int(tail), C.byref(n), _ptr(k), _ptr(v), _stream()))
        return k, v


class QuantizedKVCache(_Cache):
    """`QuantizedKVCache` (KVCache.swift:923-1210), affine mode."""
    kind = L.KIND_QUANTIZED

    def __init__(self, group_size=64, bits=8, handle=None):
        super().__init__(handle=handle, group_size=group_size, bits=bits)

    @property
    def group_size(self):
        return self._lib.kvhip_cache_group_size(self._h)

    @property
    def bits(self):
        return self._lib.kvhip_cache_bits(self._h)

    def update(self, keys, values):
        raise RuntimeError("`update` was called on `QuantizedKVCache`. Use `updateQuantized` instead.")

    def update_quantized(self, keys, values, fetch=True):
        """`updateQuantized(keys:values:)`: ((wq, scales, biases), (wq, scales, biases))."""
        self._update(keys, values)
        return self.get_quantized_state() if fetch else None

    def get_quantized_state(self):
        s = self.state
        if not s:
            return None
        n = self.offset
        s = [a[:, :, :n] for a in s]
        return (s[0], s[1], s[2]), (s[3], s[4], s[5])

    def to_unquantized(self):
        h = C.c_void_p()
        L.check(self._lib.kvhip_cache_to_unquantized(self._h, _stream(), C.byref(h)))
        s = KVCacheSimple.__new__(KVCacheSimple)
        _Cache.__init__(s, handle=h)
        s._shape = self._shape
        return s


def resolved_kv_quantization_group_size(requested, key_head_dim, value_head_dim):
    """`resolvedKVQuantizationGroupSize` (KVCache.swift:902-920)."""
    g = L.load().kvhip_resolved_group_size(requested, key_head_dim, value_head_dim)
    return g or None


class KVCacheConfigurationError(ValueError):
    """`KVCacheConfigurationError` (KVCacheConfiguration.swift:256): an invalid capacity or window."""


def make_attention_kv_cache(max_kv_size=None):
    """`makeAttentionKVCache(parameters:)` (CacheConfiguration.swift:291-296) for the legacy
    `maxKVSize` request: a ring of that capacity that keeps min(4, maxKVSize - 1) leading
    tokens (KVCachePlan.swift:455-462), else an unbounded `KVCacheSimple`."""
    if max_kv_size is None:
        return KVCacheSimple()
    if max_kv_size <= 0:
        raise KVCacheConfigurationError(f"invalid KV cache capacity {max_kv_size}")
    return RotatingKVCache(int(max_kv_size), keep=min(4, max(0, int(max_kv_size) - 1)))


def make_sliding_window_kv_cache(window, max_kv_size=None):
    """`makeSlidingWindowKVCache(parameters:window:)` (CacheConfiguration.swift:312-317): the
    architecture's window capped by the legacy `maxKVSize`, no pinned prefix."""
    if window <= 0:
        raise KVCacheConfigurationError(f"invalid sliding window {window}")
    if max_kv_size is not None and max_kv_size <= 0:
        raise KVCacheConfigurationError(f"invalid KV cache capacity {max_kv_size}")
    return RotatingKVCache(int(min(window, max_kv_size) if max_kv_size is not None else window))


def make_prompt_cache(num_layers, max_kv_size=None):
    """`makePromptCacheWithLayerCount(numLayers:maxKVSize:)` (KVCache.swift:2281-2290): one cache
    per layer."""
    return [make_attention_kv_cache(max_kv_size) for _ in range(num_layers)]


def create_attention_mask(n, cache=None, window_size=None, return_array=False):
    """`createAttentionMask(h:cache:windowSize:returnArray:)` (KVCache.swift:359-380) for `n` new
    positions (`h.dim(1)`): the cache's own `makeMask` when there is one, else the cache-less rule."""
    if cache is not None:
        return cache.make_mask(n, window_size, return_array)
    if n == 1:
        return MaskMode.none()
    if return_array or (window_size is not None and n > window_size):
        plan = L.MaskPlan(mode=L.MASK_ARRAY, rows=n, cols=n, offset=0, window=int(window_size or 0))
        return MaskMode(L.MASK_WINDOW, offset=0, window=int(window_size or 0), plan=plan)
    return MaskMode.causal()


def can_trim_prompt_cache(caches):
    """`canTrimPromptCache` (KVCache.swift:2293-2295)."""
    return all(c.is_trimmable for c in caches)


def trim_prompt_cache(caches, num_tokens):
    """`trimPromptCache` (KVCache.swift:2302-2306)."""
    if not caches or not can_trim_prompt_cache(caches):
        return 0
    for c in caches[1:]:
        c.trim(num_tokens)
    return caches[0].trim(num_tokens)


def resolve_affine_scheme(scheme):
    """`resolveAffineScheme` (KVCache.swift:2455-2461): (bits, group size) or None."""
    return {"affine4": (4, 64), "affine8": (8, 64)}.get(scheme)


def maybe_affine_quantize_kv_cache(caches, bits, group_size, compression_start):
    """`maybeAffineQuantizeKVCache` (KVCache.swift:2500-2520): every `KVCacheSimple` whose offset
    has passed `compression_start` is replaced, in place in the list, by its quantized form (one
    bulk quantize kernel on the device); a cache whose head dims fit no supported group size
    stays as it is.  Returns False while some cache is still waiting for the threshold."""
    awaits = False
    for i, c in enumerate(caches):
        if type(c) is not KVCacheSimple:
            continue
        if not c.offset > compression_start:
            awaits = True
            continue
        try:
            caches[i] = c.to_quantized(group_size, bits)
        except L.KVHipError:
            pass
    return not awaits


def affine_quantize(w, group_size=64, bits=4):
    """`MLX.quantized(w, groupSize:, bits:)` on the device: (wq int32-as-u32, scales, biases)."""
    L.init()
    w = w.contiguous()
    D = w.shape[-1]
    rows = w.numel() // D
    wq = torch.empty(w.shape[:-1] + (D * bits // 32,), dtype=torch.int32, device=w.device)
    s = torch.empty(w.shape[:-1] + (D // group_size,), dtype=w.dtype, device=w.device)
    b = torch.empty_like(s)
    L.check(L.load().kvhip_affine_quantize(_ptr(w), rows, D, group_size, bits, _DT[w.dtype], _ptr(wq),
                                           _ptr(s), _ptr(b), _stream()))
    return wq, s, b


def affine_dequantize(wq, scales, biases, group_size=64, bits=4):
    """`MLX.dequantized` on the device."""
    L.init()
    wq, scales, biases = wq.contiguous(), scales.contiguous(), biases.contiguous()
    D = wq.shape[-1] * 32 // bits
    rows = wq.numel() // wq.shape[-1]
    out = torch.empty(wq.shape[:-1] + (D,), dtype=scales.dtype, device=wq.device)
    L.check(L.load().kvhip_affine_dequantize(_ptr(wq), _ptr(scales), _ptr(biases), rows, D, group_size, bits,
                                             _DT[scales.dtype], _ptr(out), _stream()))
    return out
