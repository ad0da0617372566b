"""Edge cases and error paths through the C ABI on the device: empty caches, shape and mask
mismatches, single-row and tile-boundary lengths, fully padded batch rows, growth across
pages, and the largest row counts the decode kernels take."""
import numpy as np
import pytest
import torch

import kvhip
from kvhip import _lib as L
from oracle import kv_oracle as O
from tests.util import NAME, err_stats, np32, randn

pytestmark = pytest.mark.gpu


def test_error_paths_are_loud_and_leave_the_cache_usable():
    rng = np.random.default_rng(0)
    c = kvhip.KVCacheSimple()
    _, q = randn(rng, (1, 4, 1, 64), torch.float16)
    with pytest.raises(kvhip.KVHipError):           # attention over an empty cache
        c._shape = (1, 2, 64, 64, torch.float16)
        c.attend(q, 0.125)
    _, k = randn(rng, (1, 2, 5, 64), torch.float16)
    c.update(k, k, fetch=False)
    with pytest.raises(kvhip.KVHipError):           # other head dim
        c.update(k[..., :32].contiguous(), k[..., :32].contiguous(), fetch=False)
    with pytest.raises(kvhip.KVHipError):           # other dtype
        c.update(k.to(torch.bfloat16), k.to(torch.bfloat16), fetch=False)
    with pytest.raises(kvhip.KVHipError):           # query heads not a multiple of kv heads
        c.attend(torch.zeros((1, 3, 1, 64), dtype=torch.float16, device="cuda"), 0.125)
    with pytest.raises(kvhip.KVHipError):           # array mask of the wrong key extent
        c.attend(q, 0.125, kvhip.MaskMode.from_array(torch.ones((1, 4), dtype=torch.bool, device="cuda")))
    lib = kvhip.load()
    assert lib.kvhip_cache_update(c._h, None, None, 1, 2, 1, 64, 64, L.F16, None) < 0   # null rows
    assert lib.kvhip_cache_update(c._h, k.data_ptr(), k.data_ptr(), 1, 2, 0, 64, 64, L.F16, None) < 0  # no rows
    assert lib.kvhip_last_error_message() is not None
    assert c.offset == 5 and c.trim(100) == 5 and c.offset == 0 and c.trim(1) == 0
    c.update(k, k, fetch=False)                     # still usable: rows are overwritten after the trim
    out = c.attend(q, 0.125)
    assert torch.isfinite(out).all() and c.offset == 5
    with pytest.raises(RuntimeError):
        kvhip.QuantizedKVCache().update(k, k)      # KVCache.swift:1106-1110
    with pytest.raises(kvhip.KVHipError):
        kvhip.RotatingKVCache(0)                    # needs a positive maxSize


@pytest.mark.parametrize("T", [1, 2, 63, 64, 65, 255, 256, 257, 513])
@pytest.mark.parametrize("quant", [None, (64, 4), (64, 8)])
def test_lengths_around_tile_and_page_boundaries(T, quant):
    """A tile is 64 tokens, a page 256: lengths just below, at and above them, built by one
    bulk write plus single-token appends, decode (L = 1) and a 3-token causal step."""
    rng = np.random.default_rng(T)
    dtype, name = torch.float16, "float16"
    B, Hkv, r, D = 2, 2, 4, 64
    if quant:
        c, o = kvhip.QuantizedKVCache(*quant), O.QuantizedKVCache(*quant, name)
    else:
        c, o = kvhip.KVCacheSimple(), O.KVCacheSimple(name)
    upd = (lambda cc, a, b: cc.update_quantized(a, b, fetch=False)) if quant else (lambda cc, a, b: cc.update(a, b, fetch=False))
    oupd = (lambda oc, a, b: oc.update_quantized(a, b)) if quant else (lambda oc, a, b: oc.update(a, b))
    first = max(T - 2, 1)
    for n in [first] + [1] * (T - first):
        k, kd = randn(rng, (B, Hkv, n, D), dtype)
        v, vd = randn(rng, (B, Hkv, n, D), dtype)
        upd(c, kd, vd)
        oupd(o, k, v)
    assert c.offset == o.offset == T
    for Lq, mask, om in ((1, None, O.Mask.NONE), (3, kvhip.MaskMode.causal(), O.Mask.CAUSAL)):
        k, kd = randn(rng, (B, Hkv, Lq, D), dtype)
        v, vd = randn(rng, (B, Hkv, Lq, D), dtype)
        q, qd = randn(rng, (B, Hkv * r, Lq, D), dtype)
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, D ** -0.5, mask)
        ref = O.attention_with_cache_update(q, k, v, o, D ** -0.5, om, name)
        mx, mean = err_stats(np32(out), ref)
        assert mx <= 1e-2 and mean <= 1e-3, (T, quant, Lq, mx, mean)


def test_query_rows_per_kv_head_at_the_decode_limit():
    """Quantized caches: r * L = 16 rows still run on the split-sequence kernels, 17 go to the
    prefill tile.  Full-precision caches: 8 rows still do, 9 go to the prefill tile (faster there).
    All agree with the oracle."""
    rng = np.random.default_rng(3)
    dtype, name = torch.float16, "float16"
    B, Hkv, D, T0 = 1, 2, 128, 300
    lib = kvhip.load()
    for quant in (None, (64, 4)):
        for r, Lq in ((16, 1), (4, 4), (1, 16), (1, 17), (17, 1), (8, 1), (2, 4), (1, 8), (9, 1), (3, 3)):
            family = (1 if r * Lq <= 16 else 3) if quant else (2 if r * Lq <= 8 else 3)
            if quant:
                c, o = kvhip.QuantizedKVCache(*quant), O.QuantizedKVCache(*quant, name)
            else:
                c, o = kvhip.KVCacheSimple(), O.KVCacheSimple(name)
            k, kd = randn(rng, (B, Hkv, T0, D), dtype)
            v, vd = randn(rng, (B, Hkv, T0, D), dtype)
            (c.update_quantized if quant else c.update)(kd, vd, fetch=False)
            (o.update_quantized if quant else o.update)(k, v)
            k, kd = randn(rng, (B, Hkv, Lq, D), dtype)
            v, vd = randn(rng, (B, Hkv, Lq, D), dtype)
            q, qd = randn(rng, (B, Hkv * r, Lq, D), dtype)
            mask, om = (None, O.Mask.NONE) if Lq == 1 else (kvhip.MaskMode.causal(), O.Mask.CAUSAL)
            out = kvhip.attention_with_cache_update(qd, kd, vd, c, D ** -0.5, mask)
            fam = lib.kvhip_last_attend_kernel()
            assert fam == family, (quant, r, Lq, fam)
            ref = O.attention_with_cache_update(q, k, v, o, D ** -0.5, om, name)
            mx, mean = err_stats(np32(out), ref)
            assert mx <= 1e-2 and mean <= 1e-3, (quant, r, Lq, mx, mean)


def test_ragged_batch_with_an_all_padding_row():
    """Left padding that covers a whole batch row: the quantized path fills masked scores with
    finfo.min, so such a row comes out as the plain average of V (KVCache.swift:2396-2447); the
    other rows see only their own tokens."""
    rng = np.random.default_rng(5)
    dtype, name = torch.float16, "float16"
    B, Hkv, r, D, T, Lq = 3, 2, 4, 128, 200, 2
    c, o = kvhip.QuantizedKVCache(64, 4), O.QuantizedKVCache(64, 4, name)
    k, kd = randn(rng, (B, Hkv, T, D), dtype)
    v, vd = randn(rng, (B, Hkv, T, D), dtype)
    c.update_quantized(kd, vd, fetch=False)
    o.update_quantized(k, v)
    q, qd = randn(rng, (B, Hkv * r, Lq, D), dtype)
    pad = np.array([0, 137, T], dtype=np.int32)          # row 2 is all padding
    mask = kvhip.MaskMode.window_mask(T - Lq, 0, left_pad=torch.from_numpy(pad))
    out = c.attend(qd, D ** -0.5, mask)
    li = np.arange(T - Lq, T)[:, None]
    kj = np.arange(T)[None, :]
    m = (li >= kj)[None, None] & (kj[None, None] >= pad[:, None, None, None])
    ref = O.quantized_sdpa(q, *o.get_quantized_state(), D ** -0.5, O.Mask("array", m), 64, 4, name)
    mx, mean = err_stats(np32(out), ref)
    assert np.isfinite(np32(out)).all() and mx <= 1e-2 and mean <= 1e-3, (mx, mean)


def test_growth_across_many_pages_keeps_every_row():
    """Appends of irregular sizes over 9 pages with a copy() in the middle: the state equals the
    oracle's bit for bit, so page appends and device-to-device copies lose nothing."""
    rng = np.random.default_rng(8)
    dtype, name = torch.bfloat16, "bfloat16"
    c, o = kvhip.QuantizedKVCache(64, 8), O.QuantizedKVCache(64, 8, name)
    for i, n in enumerate([7, 250, 1, 300, 64, 129, 511, 3, 1000]):
        k, kd = randn(rng, (1, 2, n, 64), dtype)
        v, vd = randn(rng, (1, 2, n, 64), dtype)
        c.update_quantized(kd, vd, fetch=False)
        o.update_quantized(k, v)
        if i == 4:
            c, o = c.copy(), o.copy()
    st, ost = c.state, o.get_state()
    assert c.offset == o.offset == 2265
    for i, (a, b) in enumerate(zip(st, ost)):
        got = np32(a)
        if i % 3 == 0:
            assert np.array_equal(got, b), i
        else:
            assert np.array_equal(O.to_bits(got, name), O.to_bits(b, name)), i


def test_protocol_hooks_with_empty_defaults():
    """`prepare(lengths:)`, `finalize()`, `innerState()`, `ropeOffset` (KVCache.swift:46-120)."""
    rng = np.random.default_rng(3)
    for c in (kvhip.KVCacheSimple(), kvhip.RotatingKVCache(32), kvhip.QuantizedKVCache(64, 4)):
        assert c.inner_state() == [] and c.rope_offset == 0
        c.prepare(lengths=[3, 4])
        _, k = randn(rng, (1, 2, 5, 64), torch.float16)
        (c.update_quantized if isinstance(c, kvhip.QuantizedKVCache) else c.update)(k, k)
        c.eval()
        c.finalize()
        assert c.rope_offset == c.offset == 5
        assert [tuple(a.shape) for a in c.inner_state()] == [tuple(a.shape) for a in c.state]


def test_create_attention_mask_with_and_without_a_cache():
    """`createAttentionMask` (KVCache.swift:359-380): delegates to the cache, else the cache-less rule."""
    assert kvhip.create_attention_mask(1).mode == L.MASK_NONE
    assert kvhip.create_attention_mask(5).mode == L.MASK_CAUSAL
    m = kvhip.create_attention_mask(5, window_size=3)
    assert np.array_equal(m.array.cpu().numpy(), O.create_causal_mask(5, 0, 3))
    m = kvhip.create_attention_mask(4, return_array=True)
    assert np.array_equal(m.array.cpu().numpy(), O.create_causal_mask(4, 0, None))
    c = kvhip.KVCacheSimple()
    c.offset = 9
    m = kvhip.create_attention_mask(3, c, window_size=2)
    assert np.array_equal(m.array.cpu().numpy(), O.create_causal_mask(3, 9, 2))
    r = kvhip.RotatingKVCache(8)
    assert kvhip.can_trim_prompt_cache([c, r]) and kvhip.can_trim_prompt_cache([])
    r.meta_state = ["0", "8", "256", "9", "1"]
    assert not kvhip.can_trim_prompt_cache([c, r]) and kvhip.trim_prompt_cache([c, r], 2) == 0


def test_cache_factories():
    """`makeAttentionKVCache` / `makeSlidingWindowKVCache` / `makePromptCacheWithLayerCount`
    (CacheConfiguration.swift:291-317, KVCache.swift:2281-2290) for the legacy `maxKVSize` request."""
    assert isinstance(kvhip.make_attention_kv_cache(), kvhip.KVCacheSimple)
    r = kvhip.make_attention_kv_cache(4096)
    assert isinstance(r, kvhip.RotatingKVCache) and r.max_size == 4096 and r.meta_state[:2] == ["4", "4096"]
    assert kvhip.make_attention_kv_cache(3).meta_state[:2] == ["2", "3"]      # keep = min(4, maxKVSize - 1)
    assert kvhip.make_attention_kv_cache(1).meta_state[:2] == ["0", "1"]
    w = kvhip.make_sliding_window_kv_cache(1024, max_kv_size=512)
    assert w.max_size == 512 and w.meta_state[0] == "0"
    assert kvhip.make_sliding_window_kv_cache(1024).max_size == 1024
    for bad in (lambda: kvhip.make_attention_kv_cache(0), lambda: kvhip.make_sliding_window_kv_cache(0),
                lambda: kvhip.make_sliding_window_kv_cache(8, max_kv_size=-1)):
        with pytest.raises(kvhip.KVCacheConfigurationError):
            bad()
    caches = kvhip.make_prompt_cache(3, max_kv_size=64)
    assert len(caches) == 3 and all(c.max_size == 64 for c in caches)


@pytest.mark.parametrize("kind", ["simple", "quantized", "rotating"])
@pytest.mark.parametrize("Lq", [1, 4, 40])
def test_inputs_at_odd_element_offsets(kind, Lq):
    """Keys, values and queries that start one element into an allocation (contiguous views, 2-byte
    aligned only): same cache state and outputs, bit for bit, as from 256-byte aligned copies."""
    g = torch.Generator(device="cuda")
    g.manual_seed(3)
    B, Hq, Hkv, D, T0 = 2, 8, 2, 128, 300
    dtype = torch.float16

    def odd(*shape):
        n = int(np.prod(shape))
        flat = torch.randn(n + 1, generator=g, device="cuda").to(dtype)
        v = flat[1:].view(*shape)
        assert v.data_ptr() % 4 == 2 and v.is_contiguous()
        return v

    def make():
        if kind == "simple":
            return kvhip.KVCacheSimple()
        if kind == "rotating":
            return kvhip.RotatingKVCache(256, keep=4)
        return kvhip.QuantizedKVCache(64, 4)

    k0, v0, k1, v1, q = odd(B, Hkv, T0, D), odd(B, Hkv, T0, D), odd(B, Hkv, Lq, D), odd(B, Hkv, Lq, D), odd(B, Hq, Lq, D)
    outs, states = [], []
    for aligned in (False, True):
        f = (lambda t: t.clone()) if aligned else (lambda t: t)
        c = make()
        upd = c.update_quantized if kind == "quantized" else c.update
        upd(f(k0), f(v0), fetch=False)
        upd(f(k1), f(v1), fetch=False)
        mask = kvhip.MaskMode.none() if Lq == 1 else kvhip.MaskMode.causal()
        outs.append(c.attend(f(q), D ** -0.5, mask))
        states.append([a.clone() for a in c.state])
    assert torch.equal(outs[0], outs[1])
    assert len(states[0]) == len(states[1]) and all(torch.equal(a, b) for a, b in zip(*states))
