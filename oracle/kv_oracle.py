"""CPU oracle for the KV-cache hot path (TEST INFRASTRUCTURE ONLY).

This module is a checker: it restates, on the CPU with numpy, what the
reference computes for `KVCacheSimple`, `RotatingKVCache`, `QuantizedKVCache`,
the mask builders and (quantized) scaled-dot-product attention. Only `tests/`,
`__graft_entry__.smoke()` and the `cpu_baseline` leg of `bench.py` may import
it. Nothing in the product path (the HIP library and its host mirror) touches
it.

All arrays are numpy float32 whose values are representable in the logical
dtype `T` ("float16", "bfloat16" or "float32"); `round_to` is applied wherever
the reference materialises an array of dtype `T`.

Reference files restated here (paths relative to the reference checkout):
  Libraries/MLXLMCommon/KVCache.swift
  Libraries/MLXLMCommon/AttentionUtils.swift
  Libraries/MLXLMCommon/RotatingStagedKVCache.swift

Parity status of each function
------------------------------
* Cache bookkeeping (offset, idx, capacity, ring order, trim, state shapes,
  metaState strings, mask mode choice, createCausalMask truth table,
  logicalView): fully specified by the Swift source and pinned by the
  integer known answers of the reference's own tests (tests/test_oracle_kat.py).
* `affine_quantize` / `affine_dequantize`: the arithmetic lives in the
  third-party dependency ml-explore/mlx-swift (pinned 0.31.6 ..< 0.32.0,
  Package.swift:64 -> MLX core, CPU backend: `quantize<T, U>` in
  mlx/backend/cpu/quantized.cpp), whose sources are absent from the reference
  checkout.  The published loop is restated; it is pinned by known answers
  worked out by hand from that loop (tests/quantizer_kats.py: float32 scale
  versus the stored T-rounded one, round-half-to-even for q0 and the codes, the
  1e-7 floor on a non-constant group, the strict magnitude comparison, both
  clamps), by closed forms, invariants and an independent scalar implementation
  (oracle/kv_oracle.c).  No output of MLX itself is held by the reference for
  packed codes or scale / bias bits, so against the MLX binary this stays
  **parity unpinned**; against the published algorithm it is pinned.
  The packing of 3-, 5- and 6-bit codes (8 / 8 / 4 codes in 3 / 5 / 3 bytes, low
  code first) is likewise restated from that file and pinned only by byte patterns
  worked out by hand (tests/test_oracle_kat.py) and by the pack / unpack round trip:
  **parity unpinned** against the MLX binary.
* `sdpa`, `quantized_sdpa`, `softmax_last`, `_apply_mask`, `round_to`: what they compute -- which query
  heads share a kv head, the lower-right alignment of `.causal` with fewer queries than keys, how
  [L,T], [B,1,L,T] and [B,Hq,L,T] masks broadcast, exclusion against addition, the float16 / bfloat16
  rounding itself -- is pinned against an implementation that shares no code with this file: torch's CPU
  `scaled_dot_product_attention` on the dequantised cache, `torch.softmax` and torch's dtype casts
  (tests/test_oracle_kat.py, float32 to 1e-5; the 16-bit paths inside the stated tolerance of it).
* `quantized_matmul` / `softmax_last` rounding points and accumulation order inside MLX:
  **parity unpinned** (tolerance-level only).  `softmax(precise: false)`, which
  KVCache.swift:2416 calls, accumulates in the input dtype on MLX's CPU backend
  (`softmax<T, AccT = T>`, mlx/backend/cpu/softmax.cpp); this oracle exponentiates
  and sums in float32 and rounds the normalised probabilities to T once.  For
  float16 / bfloat16 inputs that is the more accurate of the two and differs from
  MLX's own output by about one unit in the last place of T per probability; the
  attention bound (max-abs 1e-2, mean-abs 1e-3) is a tolerance, not a bit pattern.
"""

from __future__ import annotations

import numpy as np

DTYPES = ("float16", "bfloat16", "float32")


# --------------------------------------------------------------------------
# dtype helpers
# --------------------------------------------------------------------------

def _bf16_bits(x32: np.ndarray) -> np.ndarray:
    """float32 -> bfloat16 bit pattern (round to nearest even), NaN kept quiet."""
    u = np.ascontiguousarray(x32, dtype=np.float32).view(np.uint32)
    rounding = ((u >> 16) & 1) + np.uint32(0x7FFF)
    r = ((u + rounding) >> 16).astype(np.uint16)
    nan = np.isnan(x32)
    if np.any(nan):
        r = np.where(nan, np.uint16(0x7FC0), r)
    return r


def to_bits(x32: np.ndarray, dtype: str) -> np.ndarray:
    """Bit pattern of `x32` in dtype `T` (uint16 for 16-bit types, uint32 for f32)."""
    x32 = np.asarray(x32, dtype=np.float32)
    if dtype == "float16":
        return x32.astype(np.float16).view(np.uint16)
    if dtype == "bfloat16":
        return _bf16_bits(x32)
    if dtype == "float32":
        return np.ascontiguousarray(x32).view(np.uint32)
    raise ValueError(dtype)


def from_bits(bits: np.ndarray, dtype: str) -> np.ndarray:
    if dtype == "float16":
        return np.asarray(bits, dtype=np.uint16).view(np.float16).astype(np.float32)
    if dtype == "bfloat16":
        return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)
    if dtype == "float32":
        return np.asarray(bits, dtype=np.uint32).view(np.float32)
    raise ValueError(dtype)


def round_to(x32: np.ndarray, dtype: str) -> np.ndarray:
    """Round float32 values to dtype `T` and return them as float32."""
    x32 = np.asarray(x32, dtype=np.float32)
    if dtype == "float32":
        return x32
    return from_bits(to_bits(x32, dtype), dtype)


def finfo_min(dtype: str) -> np.float32:
    """`MLXArray.maskFill(for:)` == finfo(dtype).min (KVCache.swift:2401, :2442)."""
    if dtype == "float16":
        return np.float32(-65504.0)
    if dtype == "bfloat16":
        return np.float32(-3.3895313892515355e38)
    return np.float32(np.finfo(np.float32).min)


# --------------------------------------------------------------------------
# MLX affine quantization (third-party arithmetic, restated)
# --------------------------------------------------------------------------

def affine_quantize(w: np.ndarray, group_size: int, bits: int, dtype: str):
    """`MLX.quantized(w, groupSize:, bits:)`, affine mode, CPU backend.

    Call sites: KVCache.swift:506,508,975,1069,1070. Per group of `group_size`
    consecutive elements of the last axis, all in float32:

        w_max, w_min          (initialised to -inf / +inf)
        mask  = |w_min| > |w_max|
        scale = max((w_max - w_min) / (2^bits - 1), 1e-7);  scale = mask ? scale : -scale
        edge  = mask ? w_min : w_max
        q0    = rint(edge / scale)                          (half to even)
        if q0 != 0: scale = edge / q0, bias = edge   else: bias = 0
        code  = clamp(rint((w - bias) / scale), 0, 2^bits - 1)   with the float32 scale/bias
        scales = T(scale), biases = T(bias)

    Packing: for 2, 4 and 8 bits element k of each run of 32/bits codes occupies
    bits [k*bits, (k+1)*bits) of one uint32 word.  For 3, 5 and 6 bits MLX packs
    8 / 8 / 4 codes, low code first, into a 24 / 40 / 24-bit integer stored as
    3 / 5 / 3 little-endian bytes; the row's bytes are then read as uint32 words.
    Both are the same thing: the row is a little-endian bit stream in which code j
    occupies bits [j*bits, (j+1)*bits), and `pack_codes` builds exactly that.
    Returns (wq uint32 [..., D*bits/32], scales f32-as-T [..., D/group_size],
    biases likewise).
    """
    assert bits in (2, 3, 4, 5, 6, 8), "MLX's affine code widths"
    w = np.asarray(w, dtype=np.float32)
    D = w.shape[-1]
    assert D % group_size == 0
    G = D // group_size
    g = w.reshape(w.shape[:-1] + (G, group_size))
    n_bins = np.float32((1 << bits) - 1)
    eps = np.float32(1e-7)
    with np.errstate(divide="ignore", invalid="ignore"):
        w_max = g.max(axis=-1)
        w_min = g.min(axis=-1)
        mask = np.abs(w_min) > np.abs(w_max)
        scale = np.maximum((w_max - w_min) / n_bins, eps).astype(np.float32)
        scale = np.where(mask, scale, -scale).astype(np.float32)
        edge = np.where(mask, w_min, w_max).astype(np.float32)
        q0 = np.rint(edge / scale).astype(np.float32)
        nz = q0 != 0
        safe_q0 = np.where(nz, q0, np.float32(1))
        scale = np.where(nz, (edge / safe_q0).astype(np.float32), scale).astype(np.float32)
        bias = np.where(nz, edge, np.float32(0)).astype(np.float32)
        q = np.rint((g - bias[..., None]) / scale[..., None]).astype(np.float32)
    q = np.minimum(np.maximum(q, np.float32(0)), n_bins)
    codes = q.astype(np.uint32).reshape(w.shape[:-1] + (D,))
    return pack_codes(codes, bits), round_to(scale, dtype), round_to(bias, dtype)


def pack_codes(codes: np.ndarray, bits: int) -> np.ndarray:
    """codes [..., D] (each < 2^bits) -> uint32 [..., D*bits/32]: code j at bits [j*bits, (j+1)*bits)
    of the row read as a little-endian bit stream (see `affine_quantize`)."""
    codes = np.asarray(codes, dtype=np.uint32)
    D = codes.shape[-1]
    assert (D * bits) % 32 == 0
    if 32 % bits == 0:
        per = 32 // bits
        c = codes.reshape(codes.shape[:-1] + (D // per, per))
        shifts = (np.arange(per, dtype=np.uint32) * np.uint32(bits))
        return np.bitwise_or.reduce(c << shifts, axis=-1).astype(np.uint32)
    one = ((codes[..., None] >> np.arange(bits, dtype=np.uint32)) & np.uint32(1)).astype(np.uint8)
    stream = np.packbits(one.reshape(codes.shape[:-1] + (D * bits,)), axis=-1, bitorder="little")
    return np.ascontiguousarray(stream).view("<u4").astype(np.uint32)


def unpack_codes(wq: np.ndarray, bits: int) -> np.ndarray:
    wq = np.asarray(wq, dtype=np.uint32)
    if 32 % bits == 0:
        per = 32 // bits
        shifts = (np.arange(per, dtype=np.uint32) * np.uint32(bits))
        c = (wq[..., None] >> shifts) & np.uint32((1 << bits) - 1)
        return c.reshape(wq.shape[:-1] + (wq.shape[-1] * per,))
    stream = np.ascontiguousarray(wq.astype("<u4")).view(np.uint8)
    one = np.unpackbits(stream, axis=-1, bitorder="little")
    D = wq.shape[-1] * 32 // bits
    one = one.reshape(wq.shape[:-1] + (D, bits)).astype(np.uint32)
    return (one << np.arange(bits, dtype=np.uint32)).sum(axis=-1).astype(np.uint32)


def _dequant_f32(wq, scales, biases, group_size, bits):
    """scale_T * code + bias_T evaluated in float32 (not rounded)."""
    codes = unpack_codes(wq, bits).astype(np.float32)
    D = codes.shape[-1]
    G = D // group_size
    c = codes.reshape(codes.shape[:-1] + (G, group_size))
    out = scales[..., None].astype(np.float32) * c
    if biases is not None:
        out = out + biases[..., None].astype(np.float32)
    return out.reshape(codes.shape).astype(np.float32)


def affine_dequantize(wq, scales, biases, group_size, bits, dtype):
    """`MLX.dequantized` (KVCache.swift:1197,1200): T(scale*code + bias)."""
    return round_to(_dequant_f32(wq, scales, biases, group_size, bits), dtype)


def quantized_matmul(x, wq, scales, biases, transpose, group_size, bits, dtype):
    """`MLX.quantizedMM` (KVCache.swift:2387, :2419).

    transpose=True : y[..., m, n] = sum_k x[..., m, k] * w^[..., n, k]
    transpose=False: y[..., m, n] = sum_k x[..., m, k] * w^[..., k, n]
    Accumulated in float32, result rounded to T (accumulation order inside MLX
    is backend specific: tolerance-level parity only).
    """
    w = _dequant_f32(wq, scales, biases, group_size, bits)
    if transpose:
        y = np.matmul(x.astype(np.float32), np.swapaxes(w, -1, -2))
    else:
        y = np.matmul(x.astype(np.float32), w)
    return round_to(y, dtype)


def softmax_last(x: np.ndarray, dtype: str) -> np.ndarray:
    """`softmax(scores, axis: -1)` (KVCache.swift:2416): float32 inside, T out.

    MLX's CPU backend accumulates in T when `precise` is false (the default the
    reference uses); accumulating in float32 here is a deliberate choice, stated in
    the module header: tolerance-level parity only."""
    x = x.astype(np.float32)
    m = x.max(axis=-1, keepdims=True)
    e = np.exp(x - m, dtype=np.float32)
    s = e.sum(axis=-1, keepdims=True, dtype=np.float32)
    return round_to(e / s, dtype)


# --------------------------------------------------------------------------
# masks
# --------------------------------------------------------------------------

def create_causal_mask(n, offset, window_size=None, lengths=None):
    """`createCausalMask` (KVCache.swift:253-275). Bool [n, offset+n] or [B,1,n,offset+n]."""
    rinds = np.arange(offset + n, dtype=np.int32)
    linds = np.arange(offset, offset + n, dtype=np.int32) if offset != 0 else rinds
    linds = linds[:, None]
    rinds = rinds[None, :]
    mask = linds >= rinds
    if window_size is not None:
        mask = mask & (linds < rinds + window_size)
    if lengths is not None:
        lengths = np.asarray(lengths)[:, None, None, None]
        mask = mask & (rinds < lengths)
    return mask


class Mask:
    """`MLXFast.ScaledDotProductAttentionMaskMode` (.none / .causal / .array)."""

    def __init__(self, mode, array=None):
        assert mode in ("none", "causal", "array")
        self.mode = mode
        self.array = array

    NONE = None
    CAUSAL = None

    def __repr__(self):
        if self.mode == "array":
            return f"Mask(array {self.array.shape} {self.array.dtype})"
        return f"Mask({self.mode})"


Mask.NONE = Mask("none")
Mask.CAUSAL = Mask("causal")


def base_make_mask(offset, n, window_size, return_array):
    """`BaseKVCache.makeMask` (KVCache.swift:236-250)."""
    if n == 1:
        return Mask.NONE
    if return_array or (window_size is not None and n > window_size):
        return Mask("array", create_causal_mask(n, offset, window_size))
    return Mask.CAUSAL


# --------------------------------------------------------------------------
# attention
# --------------------------------------------------------------------------

def _apply_mask(scores, mask: Mask, dtype, n_repeats, fill):
    """Mask application on scores [B,Hkv,r,L,T] (5-D) or [B,H,L,T] (4-D)."""
    if mask is None or mask.mode == "none":
        return scores
    L, T = scores.shape[-2], scores.shape[-1]
    if mask.mode == "causal":
        qi = np.arange(L) + (T - L)
        ki = np.arange(T)
        cm = qi[:, None] >= ki[None, :]
        return np.where(cm, scores, fill).astype(np.float32)
    m = mask.array
    if scores.ndim == 5 and m.ndim == 4:
        m = np.expand_dims(m, -3)
    if m.dtype == np.bool_:
        return np.where(m, scores, fill).astype(np.float32)
    return round_to(scores + m.astype(np.float32), dtype)


def quantized_sdpa(queries, qkeys, qvalues, scale, mask, group_size, bits, dtype):
    """`quantizedScaledDotProductAttention` (KVCache.swift:2351-2447).

    queries [B,Hq,L,D] (f32-as-T); qkeys/qvalues = (wq, scales, biases) with
    leading dims [B,Hkv,T,...]. Every intermediate the reference materialises
    (scaled queries, scores, softmax weights, output) is rounded to T.
    """
    B, Hq, L, D = queries.shape
    Hkv = qkeys[0].shape[-3]
    r = Hq // Hkv
    q = round_to(queries.astype(np.float32) * np.float32(scale), dtype)
    kw, ks, kb = qkeys
    vw, vs, vb = qvalues
    if r > 1:
        q = q.reshape(B, Hkv, r, L, D)
        kw, ks, vw, vs = (np.expand_dims(a, -3) for a in (kw, ks, vw, vs))
        kb = None if kb is None else np.expand_dims(kb, -3)
        vb = None if vb is None else np.expand_dims(vb, -3)
    scores = quantized_matmul(q, kw, ks, kb, True, group_size, bits, dtype)
    scores = _apply_mask(scores, mask, dtype, r, finfo_min(dtype))
    p = softmax_last(scores, dtype)
    out = quantized_matmul(p, vw, vs, vb, False, group_size, bits, dtype)
    if r > 1:
        out = out.reshape(B, Hq, L, out.shape[-1])
    return out


def sdpa(queries, keys, values, scale, mask, dtype):
    """`MLXFast.scaledDotProductAttention` (AttentionUtils.swift:46,59,87).

    Fused op of the third-party runtime: float32 inside, one rounding to T at
    the output. GQA by head repetition; `.causal` aligns query i with key
    T-L+i; bool masks exclude (score -> -inf), other masks are added.
    """
    B, Hq, L, D = queries.shape
    Hkv, T = keys.shape[1], keys.shape[2]
    r = Hq // Hkv
    q = queries.astype(np.float32).reshape(B, Hkv, r, L, D)
    k = keys.astype(np.float32)[:, :, None]
    v = values.astype(np.float32)[:, :, None]
    scores = np.matmul(q * np.float32(scale), np.swapaxes(k, -1, -2))
    neg_inf = np.float32(-np.inf)
    if mask is not None and mask.mode == "causal":
        qi = np.arange(L) + (T - L)
        cm = qi[:, None] >= np.arange(T)[None, :]
        scores = np.where(cm, scores, neg_inf)
    elif mask is not None and mask.mode == "array":
        m = mask.array
        if m.ndim == 4:
            # [B or 1, Hq or 1, L, T] -> split the head axis into (Hkv, r)
            if m.shape[1] == 1:
                m = m[:, :, None]
            else:
                m = m.reshape(m.shape[0], Hkv, r, m.shape[2], m.shape[3])
        if m.dtype == np.bool_:
            scores = np.where(m, scores, neg_inf)
        else:
            scores = scores + m.astype(np.float32)
    scores = scores.astype(np.float32)
    mx = scores.max(axis=-1, keepdims=True)
    e = np.exp(scores - mx, dtype=np.float32)
    p = e / e.sum(axis=-1, keepdims=True, dtype=np.float32)
    out = np.matmul(p, v).reshape(B, Hq, L, values.shape[-1])
    return round_to(out, dtype)


# --------------------------------------------------------------------------
# caches
# --------------------------------------------------------------------------

class KVCacheSimple:
    """`KVCacheSimple` (KVCache.swift:391-538)."""

    def __init__(self, dtype="float16"):
        self.keys = None
        self.values = None
        self.offset = 0
        self.step = 256
        self.dtype = dtype

    max_size = None

    def update(self, keys, values):
        # KVCache.swift:404-447
        prev = self.offset
        S = keys.shape[2]
        reset = self.keys is None or (prev + S) > self.keys.shape[2]
        if reset:
            B, H, _, Dk = keys.shape
            Dv = values.shape[3]
            n_steps = (self.step + S - 1) // self.step
            new_k = np.zeros((B, H, n_steps * self.step, Dk), np.float32)
            new_v = np.zeros((B, H, n_steps * self.step, Dv), np.float32)
            if self.keys is not None:
                ck, cv = self.keys, self.values
                if prev % self.step != 0:
                    ck, cv = ck[:, :, :prev], cv[:, :, :prev]
                self.keys = np.concatenate([ck, new_k], axis=2)
                self.values = np.concatenate([cv, new_v], axis=2)
            else:
                self.keys, self.values = new_k, new_v
        self.offset += S
        self.keys[:, :, prev:self.offset] = keys
        self.values[:, :, prev:self.offset] = values
        return self.keys[:, :, :self.offset], self.values[:, :, :self.offset]

    @property
    def capacity(self):
        return 0 if self.keys is None else self.keys.shape[2]

    def get_state(self):
        # KVCache.swift:449-460
        if self.keys is None:
            return []
        return [self.keys[:, :, :self.offset], self.values[:, :, :self.offset]]

    def set_state(self, arrays):
        # KVCache.swift:461-468
        assert len(arrays) == 2
        self.keys = np.array(arrays[0], np.float32)
        self.values = np.array(arrays[1], np.float32)
        self.offset = self.keys.shape[2]

    def get_meta_state(self):
        return [""]  # KVCache.swift:207-214

    is_trimmable = True

    def is_trimmable_after(self, positions):
        return True

    def trim(self, n):
        t = min(self.offset, n)  # KVCache.swift:474-478
        self.offset -= t
        return t

    def make_mask(self, n, window_size=None, return_array=False):
        return base_make_mask(self.offset, n, window_size, return_array)

    def copy(self):
        new = KVCacheSimple(self.dtype)
        new.step = self.step
        s = self.get_state()
        if s:
            new.set_state([a.copy() for a in s])
        return new

    def to_quantized(self, group_size=64, bits=4):
        # KVCache.swift:486-523
        if self.keys is not None:
            ck = self.keys[:, :, :self.offset]
            cv = self.values[:, :, :self.offset]
            eff = resolved_group_size(group_size, ck.shape[3], cv.shape[3])
            if eff is None:
                raise ValueError("KV cache quantization requires head dimensions divisible by 32/64/128")
            qc = QuantizedKVCache(eff, bits, self.dtype)
            qc.offset = self.offset
            qk = affine_quantize(ck, eff, bits, self.dtype)
            qv = affine_quantize(cv, eff, bits, self.dtype)
            qc.set_state(list(qk) + list(qv))
            return qc
        qc = QuantizedKVCache(group_size, bits, self.dtype)
        qc.offset = self.offset
        return qc


class RotatingKVCache:
    """`RotatingKVCache` (KVCache.swift:541-900)."""

    def __init__(self, max_size, keep=0, step=256, dtype="float16"):
        self.max_cache_size = max_size
        self.keep = keep
        self.step = step
        self.keys = None
        self.values = None
        self.offset = 0
        self.idx = 0
        self.capacity_origin = "modelNative"
        self.dtype = dtype

    @property
    def max_size(self):
        return self.max_cache_size

    def _trim(self, trim_size, a, append=None):
        # KVCache.swift:576-590
        if trim_size > 0:
            parts = [a[:, :, :self.keep], a[:, :, trim_size + self.keep:]]
        else:
            parts = [a]
        if append is not None:
            parts.append(append)
        return np.concatenate(parts, axis=2)

    def _temporal_order(self, a):
        # KVCache.swift:592-606
        if self.idx == a.shape[2]:
            return a
        if self.idx < self.offset:
            return np.concatenate(
                [a[:, :, :self.keep], a[:, :, self.idx:], a[:, :, self.keep:self.idx]], axis=2)
        return a[:, :, :self.idx]

    def logical_view(self, tail):
        # KVCache.swift:631-658
        if self.keys is None:
            return None
        ok, ov = self._temporal_order(self.keys), self._temporal_order(self.values)
        available = ok.shape[2]
        requested = min(max(tail, 0), available)
        bound = max(requested, min(self.keep, available))
        trim_size = available - bound
        if trim_size <= 0:
            return ok, ov
        if self.keep == 0:
            return ok[:, :, trim_size:], ov[:, :, trim_size:]
        return self._trim(trim_size, ok), self._trim(trim_size, ov)

    def _update_concat(self, keys, values):
        # KVCache.swift:660-682
        if self.keys is None:
            self.keys = np.array(keys, np.float32)
            self.values = np.array(values, np.float32)
        else:
            self.keys = self._temporal_order(self.keys)
            self.values = self._temporal_order(self.values)
            self.idx = self.keys.shape[2]
            trim_size = self.idx - self.max_cache_size + 1
            self.keys = self._trim(trim_size, self.keys, keys)
            self.values = self._trim(trim_size, self.values, values)
        self.offset += keys.shape[2]
        self.idx = self.keys.shape[2]
        return self.keys, self.values

    def _update_in_place(self, keys, values):
        # KVCache.swift:684-740
        B, H, S, Dk = keys.shape
        Dv = values.shape[3]
        prev = self.offset
        M = self.max_cache_size
        if self.keys is None or (prev >= self.keys.shape[2] and self.keys.shape[2] < M):
            new_size = min(self.step, M - prev)
            new_k = np.zeros((B, H, new_size, Dk), np.float32)
            new_v = np.zeros((B, H, new_size, Dv), np.float32)
            if self.keys is not None:
                self.keys = np.concatenate([self.keys, new_k], axis=2)
                self.values = np.concatenate([self.values, new_v], axis=2)
            else:
                self.keys, self.values = new_k, new_v
            self.idx = prev
        trim_size = self.keys.shape[2] - M
        if trim_size > 0:
            self.keys = self._trim(trim_size, self.keys)
            self.values = self._trim(trim_size, self.values)
            self.idx = M
        if self.idx == M:
            self.idx = self.keep
        self.keys[:, :, self.idx:self.idx + S] = keys
        self.values[:, :, self.idx:self.idx + S] = values
        self.offset += S
        self.idx += S
        if self.offset < M:
            return self.keys[:, :, :self.offset], self.values[:, :, :self.offset]
        return self.keys, self.values

    def update(self, keys, values):
        # KVCache.swift:742-750
        if keys.shape[2] == 1:
            return self._update_in_place(keys, values)
        return self._update_concat(keys, values)

    def get_state(self):
        # KVCache.swift:752-763
        if self.keys is None:
            return []
        if self.offset < self.keys.shape[2]:
            return [self.keys[:, :, :self.offset], self.values[:, :, :self.offset]]
        return [self.keys, self.values]

    def set_state(self, arrays):
        assert len(arrays) == 2
        self.keys = np.array(arrays[0], np.float32)
        self.values = np.array(arrays[1], np.float32)

    def get_meta_state(self):
        # KVCache.swift:775-781
        return [str(self.keep), str(self.max_cache_size), str(self.step), str(self.offset),
                str(self.idx), self.capacity_origin]

    def set_meta_state(self, v):
        # KVCache.swift:782-815
        if len(v) not in (5, 6):
            raise ValueError("RotatingKVCache metaState must have 5 or 6 values")
        if v[1] == "None":
            raise ValueError("RotatingKVCache requires a non-nil maxSize")
        keep, max_size, step, offset, idx = int(v[0]), int(v[1]), int(v[2]), int(v[3]), int(v[4])
        self.keep, self.max_cache_size, self.step = keep, max_size, step
        self.offset, self.idx = offset, idx
        if len(v) == 6:
            if v[5] not in ("modelNative", "requested"):
                raise ValueError("Invalid RotatingKVCache capacity origin")
            self.capacity_origin = v[5]
        else:
            self.capacity_origin = "modelNative"

    @property
    def is_trimmable(self):
        return self.is_trimmable_after(0)

    def is_trimmable_after(self, positions):
        return self.offset + positions < self.max_cache_size  # KVCache.swift:821-823

    def trim(self, n):
        t = min(self.offset, n)  # KVCache.swift:826-831
        self.offset -= t
        self.idx -= t
        return t

    def make_mask(self, n, window_size=None, return_array=False):
        # KVCache.swift:834-871
        M = self.max_cache_size
        if n > 1:
            actual = window_size if window_size is not None else M
            capped = min(M - 1, self.offset)
            if capped + n > actual or return_array:
                return Mask("array", create_causal_mask(n, capped, actual))
            return Mask.CAUSAL
        if window_size is None:
            return Mask.NONE
        if self.offset >= window_size and M > window_size:
            cur = self.idx
            if cur >= M:
                cur = 0
            mask_size = self.offset + 1 if self.offset < M else M
            mask = np.arange(mask_size) >= (mask_size - window_size)
            return Mask("array", np.roll(mask, cur + 1))
        return Mask.NONE

    def copy(self):
        new = RotatingKVCache(self.max_cache_size, self.keep, self.step, self.dtype)
        s = self.get_state()
        if s:
            new.set_state([a.copy() for a in s])
        new.set_meta_state(self.get_meta_state())
        return new

    def to_quantized(self, group_size=64, bits=4):
        raise ValueError("RotatingKVCache quantization is not implemented")  # KVCache.swift:894-899


def resolved_group_size(requested, key_head_dim, value_head_dim):
    """`resolvedKVQuantizationGroupSize` (KVCache.swift:902-920)."""
    requested = max(1, requested)
    compatible = [g for g in (32, 64, 128) if key_head_dim % g == 0 and value_head_dim % g == 0]
    if not compatible:
        return None
    return min(compatible, key=lambda g: (abs(g - requested), g))


class QuantizedKVCache:
    """`QuantizedKVCache` (KVCache.swift:923-1210), affine mode."""

    def __init__(self, group_size=64, bits=8, dtype="float16"):
        self.keys = None    # [wq, scales, biases]
        self.values = None
        self.offset = 0
        self.step = 256
        self.group_size = group_size
        self.bits = bits
        self.dtype = dtype

    max_size = None

    def _init_quant(self, dim, shape):
        # KVCache.swift:971-978: quantized(zeros) -> scales are T(-1e-7), not 0
        return list(affine_quantize(np.zeros(tuple(shape) + (dim,), np.float32),
                                    self.group_size, self.bits, self.dtype))

    @staticmethod
    def _expand(t, shape):
        # KVCache.swift:981-989
        return [np.concatenate([a, np.zeros(tuple(shape) + (a.shape[-1],), a.dtype)], axis=-2)
                for a in t]

    def update_quantized(self, keys, values):
        # KVCache.swift:1011-1102
        B, H, S, Dk = keys.shape
        Dv = values.shape[3]
        prev = self.offset
        eff = resolved_group_size(self.group_size, Dk, Dv)
        if (eff is not None and eff != self.group_size and self.keys is None
                and self.values is None and self.offset == 0):
            self.group_size = eff
        if eff is None:
            raise ValueError("KV cache quantization requires head dimensions divisible by 32/64/128")
        if self.keys is None or (prev + S) > self.keys[0].shape[-2]:
            new_steps = ((self.step + S - 1) // self.step) * self.step
            shape = (B, H, new_steps)
            if self.keys is not None:
                if prev % self.step != 0:
                    self.keys = [a[:, :, :prev] for a in self.keys]
                    self.values = [a[:, :, :prev] for a in self.values]
                self.keys = self._expand(self.keys, shape)
                self.values = self._expand(self.values, shape)
            else:
                self.keys = self._init_quant(Dk, shape)
                self.values = self._init_quant(Dv, shape)
        self.offset += S
        qk = affine_quantize(keys, self.group_size, self.bits, self.dtype)
        qv = affine_quantize(values, self.group_size, self.bits, self.dtype)
        for i in range(3):
            self.keys[i][:, :, prev:self.offset] = qk[i]
            self.values[i][:, :, prev:self.offset] = qv[i]
        return (tuple(a[:, :, :self.offset] for a in self.keys),
                tuple(a[:, :, :self.offset] for a in self.values))

    def update(self, keys, values):
        raise RuntimeError("`update` was called on `QuantizedKVCache`. Use `updateQuantized` instead.")

    @property
    def capacity(self):
        return 0 if self.keys is None else self.keys[0].shape[2]

    def get_quantized_state(self):
        if self.keys is None:
            return None
        return (tuple(a[:, :, :self.offset] for a in self.keys),
                tuple(a[:, :, :self.offset] for a in self.values))

    def get_state(self):
        # KVCache.swift:1113-1130
        if self.keys is None:
            return []
        return [a[:, :, :self.offset] for a in self.keys] + [a[:, :, :self.offset] for a in self.values]

    def set_state(self, arrays):
        # KVCache.swift:1131-1146 (offset is NOT touched)
        if len(arrays) == 6:
            self.keys = [np.array(a) for a in arrays[:3]]
            self.values = [np.array(a) for a in arrays[3:]]
        else:
            raise ValueError("QuantizedKVCache state must have exactly 6 or 4 arrays")

    def get_meta_state(self):
        return [str(self.step), str(self.offset), str(self.group_size), str(self.bits)]

    def set_meta_state(self, v):
        # KVCache.swift:1148-1166
        if len(v) != 4:
            raise ValueError("QuantizedKVCache metaState must have exactly 4 values")
        self.offset, self.group_size, self.bits = int(v[1]), int(v[2]), int(v[3])

    is_trimmable = True

    def is_trimmable_after(self, positions):
        return True

    def trim(self, n):
        t = min(self.offset, n)
        self.offset -= t
        return t

    def make_mask(self, n, window_size=None, return_array=False):
        return base_make_mask(self.offset, n, window_size, return_array)

    def copy(self):
        new = QuantizedKVCache(self.group_size, self.bits, self.dtype)
        s = self.get_state()
        if s:
            new.set_state([a.copy() for a in s])
        new.set_meta_state(self.get_meta_state())
        return new

    def to_unquantized(self):
        # KVCache.swift:1188-1209
        simple = KVCacheSimple(self.dtype)
        simple.offset = self.offset
        if self.keys is not None:
            k = [a[:, :, :self.offset] for a in self.keys]
            v = [a[:, :, :self.offset] for a in self.values]
            simple.set_state([
                affine_dequantize(k[0], k[1], k[2], self.group_size, self.bits, self.dtype),
                affine_dequantize(v[0], v[1], v[2], self.group_size, self.bits, self.dtype)])
        return simple


class RotatingStagedKVCache:
    """`RotatingStagedKVCache` (RotatingStagedKVCache.swift:12-132)."""

    def __init__(self, live: RotatingKVCache):
        self.live = live
        self.staged_keys = None
        self.staged_values = None

    @property
    def staged_count(self):
        return 0 if self.staged_keys is None else self.staged_keys.shape[2]

    @property
    def offset(self):
        return self.live.offset + self.staged_count

    @property
    def max_size(self):
        return self.live.max_size

    def update(self, keys, values):
        if self.staged_keys is None:
            self.staged_keys, self.staged_values = np.array(keys), np.array(values)
        else:
            self.staged_keys = np.concatenate([self.staged_keys, keys], axis=2)
            self.staged_values = np.concatenate([self.staged_values, values], axis=2)
        bound = min(self.live.offset, self.live.max_size - 1)
        view = self.live.logical_view(bound) if bound > 0 else None
        if view is None:
            return self.staged_keys, self.staged_values
        return (np.concatenate([view[0], self.staged_keys], axis=2),
                np.concatenate([view[1], self.staged_values], axis=2))

    def make_mask(self, n, window_size=None, return_array=False):
        return self.live.make_mask(n, window_size, return_array)

    def commit(self, retaining):
        sk, sv = self.staged_keys, self.staged_values
        self.staged_keys = self.staged_values = None
        if sk is None:
            return
        keep = min(max(retaining, 0), sk.shape[2])
        if keep > 0:
            self.live.update(sk[:, :, :keep], sv[:, :, :keep])

    is_trimmable = False

    def trim(self, n):
        return 0


def attention_with_cache_update(queries, keys, values, cache, scale, mask, dtype):
    """`attentionWithCacheUpdate` (AttentionUtils.swift:37-95), non-Turbo branches."""
    if cache is None:
        return sdpa(queries, keys, values, scale, mask, dtype)
    if isinstance(cache, QuantizedKVCache):
        qk, qv = cache.update_quantized(keys, values)
        return quantized_sdpa(queries, qk, qv, scale, mask, cache.group_size, cache.bits, dtype)
    ck, cv = cache.update(keys, values)
    return sdpa(queries, ck, cv, scale, mask, dtype)


def trim_prompt_cache(caches, num_tokens):
    """`trimPromptCache` (KVCache.swift:2302-2306)."""
    if not caches or not all(c.is_trimmable for c in caches):
        return 0
    for c in caches[1:]:
        c.trim(num_tokens)
    return caches[0].trim(num_tokens)
