"""GPU parity of the matrix-core decode kernel for full-precision caches at larger
sizes (several pages, several spans) for KVCacheSimple and RotatingKVCache."""
import numpy as np
import pytest
import torch

import kvhip
from oracle import c_oracle as CO
from oracle import kv_oracle as O
from tests.util import NAME, bits_equal, dev, err_stats, np32, randn

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D,Hq,Hkv", [(128, 8, 2), (64, 4, 4), (256, 4, 2)])
def test_simple_decode_grow(dtype, D, Hq, Hkv):
    """BASELINE config 2 scaled down: append one token per step, SDPA over everything cached,
    checked against the C restatement of the fused SDPA at several lengths."""
    rng = np.random.default_rng(D)
    B = 2
    name = NAME[dtype]
    c = kvhip.KVCacheSimple()
    T0 = 1500
    ch = np.ones(D, np.float32)
    ch[rng.integers(0, D, size=max(1, D // 100))] = 8.0  # outlier channels
    k = O.round_to(rng.standard_normal((B, Hkv, T0, D)).astype(np.float32) * 0.5 * ch, name)
    v = O.round_to(rng.standard_normal((B, Hkv, T0, D)).astype(np.float32) * 0.5 * ch, name)
    c.update(dev(k, dtype), dev(v, dtype), fetch=False)
    scale = 1.0 / np.sqrt(D)
    for step in range(6):
        kn = O.round_to(rng.standard_normal((B, Hkv, 1, D)).astype(np.float32) * 0.5 * ch, name)
        vn = O.round_to(rng.standard_normal((B, Hkv, 1, D)).astype(np.float32) * 0.5 * ch, name)
        q, qd = randn(rng, (B, Hq, 1, D), dtype)
        out = kvhip.attention_with_cache_update(qd, dev(kn, dtype), dev(vn, dtype), c, scale)
        k = np.concatenate([k, kn], 2)
        v = np.concatenate([v, vn], 2)
        ref = CO.sdpa(q, k, v, scale, None, name)
        mx, mean = err_stats(np32(out), ref)
        assert mx <= 1e-2 and mean <= 1e-3, (step, mx, mean)
    # a speculative-style multi-token step with a causal mask (4 query rows per head)
    kn, knd = randn(rng, (B, Hkv, 4, D), dtype)
    q, qd = randn(rng, (B, Hq, 4, D), dtype)
    out = kvhip.attention_with_cache_update(qd, knd, knd, c, scale, kvhip.MaskMode.causal())
    k = np.concatenate([k, kn], 2)
    v = np.concatenate([v, kn], 2)
    ref = CO.sdpa(q, k, v, scale, "causal", name)
    mx, mean = err_stats(np32(out), ref)
    assert mx <= 1e-2 and mean <= 1e-3, (mx, mean)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,Hkv,T0", [(32, 8, 333), (64, 8, 70), (16, 8, 900)])
def test_simple_decode_many_pairs(dtype, B, Hkv, T0):
    """128 (batch, kv-head) pairs and more: with 256 a single span covers a pair's sequence and
    the decode kernel writes the output rows itself, with fewer the merge kernel runs."""
    rng = np.random.default_rng(B + T0)
    D, r = 128, 4
    name = NAME[dtype]
    scale = 1.0 / np.sqrt(D)
    c = kvhip.KVCacheSimple()
    k, kd = randn(rng, (B, Hkv, T0, D), dtype)
    v, vd = randn(rng, (B, Hkv, T0, D), dtype)
    c.update(kd, vd, fetch=False)
    for Lq, mask, om in ((1, kvhip.MaskMode.none(), None), (2, kvhip.MaskMode.causal(), "causal")):
        kn, knd = randn(rng, (B, Hkv, Lq, D), dtype)
        vn, vnd = randn(rng, (B, Hkv, Lq, D), dtype)
        q, qd = randn(rng, (B, Hkv * r, Lq, D), dtype)
        out = kvhip.attention_with_cache_update(qd, knd, vnd, c, scale, mask)
        k, v = np.concatenate([k, kn], 2), np.concatenate([v, vn], 2)
        ref = CO.sdpa(q, k, v, scale, om, name)
        mx, mean = err_stats(np32(out), ref)
        assert mx <= 1e-2 and mean <= 1e-3, (Lq, mx, mean)
        assert kvhip.load().kvhip_last_attend_kernel() == 2  # matrix-core full-precision decode


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_rotating_decode_after_wrap(dtype):
    """Ring of 1024 (keep 4), D 256: chunked prefill wraps it, then single-token decode over
    the full window, with and without the rolled window mask."""
    rng = np.random.default_rng(7)
    B, Hq, Hkv, D, M = 2, 4, 2, 256, 1024
    name = NAME[dtype]
    scale = 1.0 / np.sqrt(D)
    c = kvhip.RotatingKVCache(M, keep=4)
    o = O.RotatingKVCache(M, keep=4, dtype=name)
    for i in range(6):
        k, kd = randn(rng, (B, Hkv, 256, D), dtype)
        v, vd = randn(rng, (B, Hkv, 256, D), dtype)
        c.update(kd, vd, fetch=False)
        o.update(k, v)
    for i in range(30):
        k, kd = randn(rng, (B, Hkv, 1, D), dtype)
        v, vd = randn(rng, (B, Hkv, 1, D), dtype)
        q, qd = randn(rng, (B, Hq, 1, D), dtype)
        w = M if i % 2 == 0 else 512  # 512 < maxSize: rolled single-token window mask
        mask = c.make_mask(1, w, False)
        om = o.make_mask(1, w, False)
        assert (mask.mode == 0) == (om.mode == "none")
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
        ref = O.attention_with_cache_update(q, k, v, o, scale, om, name)
        mx, mean = err_stats(np32(out), ref)
        assert mx <= 1e-2 and mean <= 1e-3, (i, mx, mean)
        assert c.meta_state == o.get_meta_state()


@pytest.mark.parametrize("dtype,D,B,Hq,Hkv", [(torch.float16, 128, 2, 8, 2), (torch.bfloat16, 64, 1, 4, 4), (torch.bfloat16, 256, 2, 4, 2),
                                              (torch.float16, 256, 1, 8, 2), (torch.float16, 96, 1, 4, 2)])
@pytest.mark.parametrize("kind", ["simple", "ring"])
def test_single_token_steps_write_their_row_inside_the_decode_kernel(kind, dtype, D, B, Hq, Hkv):
    """`attentionWithCacheUpdate` with one new token and no mask on a 16-bit full-precision cache has no append
    launch: the decode kernel copies the new row into its slot (KVCacheSimple: the next row; RotatingKVCache: the
    slot of the in-place step, past the wrap as well).  After every run of steps the cache's state must equal
    the oracle's bit for bit -- across 64-token tiles, pages, trims and ring wraps -- and every output the
    oracle's within the bound.  Head size 96 has no decode kernel: there the row goes through the append kernel."""
    rng = np.random.default_rng(D + B)
    name = NAME[dtype]
    if kind == "simple":
        cache, ocache = kvhip.KVCacheSimple(), O.KVCacheSimple(name)
    else:
        cache, ocache = kvhip.RotatingKVCache(300, keep=4), O.RotatingKVCache(300, keep=4, dtype=name)
    scale = D ** -0.5
    for start, steps, trim in [(1, 9, 0), (60, 10, 3), (250, 12, 0), (290, 25, 2), (700, 6, 0)]:
        n = start - ocache.offset
        if n > 0:
            k, kd = randn(rng, (B, Hkv, n, D), dtype)
            v, vd = randn(rng, (B, Hkv, n, D), dtype)
            cache.update(kd, vd, fetch=False)
            ocache.update(k, v)
        for _ in range(steps):
            q, qd = randn(rng, (B, Hq, 1, D), dtype)
            k, kd = randn(rng, (B, Hkv, 1, D), dtype)
            v, vd = randn(rng, (B, Hkv, 1, D), dtype)
            got = kvhip.attention_with_cache_update(qd, kd, vd, cache, scale)
            assert kvhip.load().kvhip_last_attend_kernel() == (3 if D == 96 else 2)
            ref = O.attention_with_cache_update(q, k, v, ocache, scale, O.Mask.NONE, name)
            mx, mean = err_stats(np32(got), ref)
            assert mx <= 1e-2 and mean <= 1e-3, (ocache.offset, mx, mean)
            assert cache.offset == ocache.offset and cache.meta_state == ocache.get_meta_state()
        for a, b in zip(cache.state, ocache.get_state()):
            assert bits_equal(a, b, dtype), (kind, start)
        assert cache.trim(trim) == ocache.trim(trim)
