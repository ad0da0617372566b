"""Drawn schedules against the oracle: appends of drawn widths, trims, copies, state round trips, conversions and
decode sequences, each case a seed.  The fixed schedules of the other files pin the cases the reference's own tests
name; these walk combinations nobody wrote down (one of them found that a cache trimmed back to empty could not
export its state)."""
import numpy as np
import pytest
import torch

import kvhip
from oracle import kv_oracle as O
from tests.test_gpu_cache import check_quantized_state, drive_pair, positioned
from tests.util import NAME, check_attention, err_stats, exact_attention, np32, presented_f64, randn

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", range(30))
def test_quantized_append_trim_convert(seed):
    """Codes and (scale, bias) pairs bit for bit after a drawn schedule, and after `toQuantized` of the same rows."""
    rng = np.random.default_rng(9000 + seed)
    dtype = [torch.float16, torch.bfloat16][seed % 2]
    Dk, Dv, gss = [(64, 64, [32, 64]), (96, 96, [32]), (128, 128, [32, 64, 128]), (256, 256, [64, 128]),
                   (192, 128, [32, 64])][seed % 5]
    gs, bits = int(rng.choice(gss)), int(rng.choice([4, 8, 4, 8, 3, 6]))
    B, H = int(rng.integers(1, 4)), int(rng.integers(1, 4))
    cache, oc = kvhip.QuantizedKVCache(gs, bits), O.QuantizedKVCache(gs, bits, NAME[dtype])
    c, o = kvhip.KVCacheSimple(), O.KVCacheSimple(NAME[dtype])
    for _ in range(int(rng.integers(3, 8))):
        L = int(rng.choice([1, 2, 5, 63, 64, 65, 128, 130, 257, 400]))
        k, kd = randn(rng, (B, H, L, Dk), dtype, float(rng.choice([0.1, 1.0, 30.0])))
        v, vd = randn(rng, (B, H, L, Dv), dtype, float(rng.choice([0.1, 1.0, 30.0])))
        cache.update_quantized(kd, vd, fetch=False)
        oc.update_quantized(k, v)
        c.update(kd, vd, fetch=False)
        o.update(k, v)
        t = int(rng.choice([0, 0, 1, 3, 70]))
        assert cache.trim(t) == oc.trim(t) and c.trim(t) == o.trim(t)
    check_quantized_state(cache, oc, dtype)
    if c.offset > 0:
        check_quantized_state(c.to_quantized(gs, bits), o.to_quantized(gs, bits), dtype)


@pytest.mark.parametrize("seed", range(30))
def test_ring_updates_trims_copies_and_restores(seed):
    """Every update's presentation and metaState equal the reference's buffers through drawn widths (single
    tokens, chunks up to twice the ring), trims, copies and state / metaState restores."""
    rng = np.random.default_rng(7000 + seed)
    M = int(rng.choice([5, 8, 16, 33, 64, 100, 300]))
    keep = min(int(rng.choice([0, 1, 2, 4])), M - 1)
    step = int(rng.choice([256, 3, 16]))
    dtype = [torch.float16, torch.bfloat16, torch.float32][seed % 3]
    c, o = kvhip.RotatingKVCache(M, keep=keep, step=step), O.RotatingKVCache(M, keep=keep, step=step, dtype=NAME[dtype])
    pos = 0
    for _ in range(int(rng.integers(5, 60))):
        L = int(rng.choice([1, 1, 1, 1, 2, 3, M // 2 + 1, M, M + 3, 2 * M + 1]))
        (k, v), _ = positioned(pos, pos + L, D=4)
        k, v = O.round_to(k, NAME[dtype]), O.round_to(v, NAME[dtype])  # (positions past 256 / 2048 are not exact in 16 bits)
        drive_pair(c, o, k, v, dtype)
        pos += L
        assert c.is_trimmable == o.is_trimmable
        act = int(rng.integers(0, 10))
        if act == 0 and o.is_trimmable:
            t = int(rng.integers(0, 4))
            assert c.trim(t) == o.trim(t) and c.meta_state == o.get_meta_state()
            pos = o.offset
        elif act == 1:
            st = c.state
            assert all(np.array_equal(np32(a), b) for a, b in zip(st, o.get_state()))
            fresh = kvhip.RotatingKVCache(M)
            fresh.state = st
            fresh.meta_state = c.meta_state
            c = fresh
        elif act == 2:
            c = c.copy()


@pytest.mark.parametrize("seed", range(36))
def test_decode_sequences_through_the_dispatcher(seed):
    """A prompt, then single tokens and small chunks through `attentionWithCacheUpdate` (the steps whose row the
    decode kernel writes itself, the ring's gather, trims in between): every step's output against the oracle's."""
    rng = np.random.default_rng(11000 + seed)
    kind = ["simple", "rotating", "quantized"][seed % 3]
    dtype = [torch.float16, torch.bfloat16][(seed // 3) % 2]
    if kind == "quantized":
        Dk, Dv, gs = [(64, 64, 64), (128, 128, 64), (128, 128, 32), (96, 96, 32), (256, 256, 64), (192, 128, 64)][int(rng.integers(6))]
        bits = int(rng.choice([4, 8]))
        c, o = kvhip.QuantizedKVCache(gs, bits), O.QuantizedKVCache(gs, bits, NAME[dtype])
    else:
        Dk, Dv = [(64, 64), (128, 128), (256, 256), (96, 96), (80, 80), (192, 128)][int(rng.integers(6))]
        if kind == "simple":
            c, o = kvhip.KVCacheSimple(), O.KVCacheSimple(NAME[dtype])
        else:
            M, keep = int(rng.choice([64, 100, 300])), int(rng.choice([0, 4]))
            c, o = kvhip.RotatingKVCache(M, keep=keep), O.RotatingKVCache(M, keep=keep, dtype=NAME[dtype])
    B, Hkv, r = int(rng.integers(1, 4)), int(rng.choice([1, 2, 4])), int(rng.choice([1, 2, 4, 8]))
    scale = Dk ** -0.5
    steps = [int(rng.choice([1, 40, 70, 200, 330]))] + [int(rng.choice([1, 1, 1, 1, 1, 2, 4, 16])) for _ in range(int(rng.integers(4, 30)))]
    for i, Lq in enumerate(steps):
        k, kd = randn(rng, (B, Hkv, Lq, Dk), dtype)
        v, vd = randn(rng, (B, Hkv, Lq, Dv), dtype)
        q, qd = randn(rng, (B, Hkv * r, Lq, Dk), dtype)
        if Lq == 1 and rng.random() < 0.7:
            mask, om = kvhip.MaskMode.none(), O.Mask.NONE
        else:
            mask, om = kvhip.MaskMode.causal(), O.Mask.CAUSAL
        out = np32(kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask))
        ref = O.attention_with_cache_update(q, k, v, o, scale, om, NAME[dtype])
        assert c.offset == o.offset and np.isfinite(out).all()
        # outside the 1e-2 / 1e-3 bound only where a float64 evaluation shows the device as close to exact as the oracle
        check_attention(out, ref, dtype, f"step {i} L={Lq} T={c.offset}", lambda: exact_attention(q, *presented_f64(o), scale, om))
        if kind != "rotating" and rng.random() < 0.15:
            t = int(rng.integers(0, 5))
            assert c.trim(t) == o.trim(t)


@pytest.mark.parametrize("seed", range(24))
def test_make_mask_between_drawn_updates(seed):
    """`makeMask(n:windowSize:returnArray:)` (KVCache.swift:236-275, 834-871) of a ring or a simple cache at drawn
    offsets: the same mode as the reference's, and the same array where it gives one."""
    from kvhip import _lib as L
    rng = np.random.default_rng(13000 + seed)
    M = int(rng.choice([5, 8, 16, 33, 64]))
    if seed % 4 != 3:
        keep = min(int(rng.choice([0, 1, 4])), M - 1)
        c, o = kvhip.RotatingKVCache(M, keep=keep), O.RotatingKVCache(M, keep=keep)
    else:
        c, o = kvhip.KVCacheSimple(), O.KVCacheSimple("float16")
    pos = 0
    for it in range(int(rng.integers(1, 40))):
        n = int(rng.choice([1, 1, 2, 5, M, M + 2]))
        w = [None, 1, 3, M // 2, M, 2 * M][int(rng.integers(6))]
        ra = bool(rng.integers(2))
        m, om = c.make_mask(n, w, ra), o.make_mask(n, w, ra)
        what = f"update {it}, offset {o.offset}, n {n}, window {w}, returnArray {ra}"
        if om.mode == "array":
            assert np.array_equal(m.array.cpu().numpy(), om.array), what
        else:
            assert m.mode == (L.MASK_NONE if om.mode == "none" else L.MASK_CAUSAL), what
        Lw = int(rng.choice([1, 1, 1, 2, M // 2 + 1, M + 1]))
        (k, v), _ = positioned(pos, pos + Lw, D=4)
        drive_pair(c, o, k, v, torch.float16)
        pos += Lw


@pytest.mark.parametrize("seed", range(24))
def test_prompt_cache_files_of_drawn_cache_lists(seed, tmp_path):
    """`savePromptCache` / `loadPromptCache` (KVCache.swift:1797-2249) over lists of caches of drawn kinds, dtypes,
    head sizes and histories (never written, written, trimmed, trimmed back to empty): the loaded caches hold the
    same state and metaState, and both lists continue alike."""
    rng = np.random.default_rng(15000 + seed)
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)

    def rand(shape, dtype):
        return torch.randn(*shape, generator=g, device="cuda").to(dtype)

    caches = []
    for _ in range(int(rng.integers(1, 6))):
        kind = int(rng.integers(3))
        dtype = [torch.float16, torch.bfloat16, torch.float32][int(rng.integers(3))]
        B, H = int(rng.integers(1, 3)), int(rng.integers(1, 3))
        Dk, Dv = [(64, 64), (128, 128), (96, 96), (192, 128), (64, 32)][int(rng.integers(5))]
        if kind == 0:
            c = kvhip.KVCacheSimple()
        elif kind == 1:
            c = kvhip.RotatingKVCache(int(rng.choice([8, 33, 64])), keep=int(rng.choice([0, 2])))
        else:
            c = kvhip.QuantizedKVCache(int(rng.choice([32, 64])), int(rng.choice([2, 3, 4, 5, 6, 8])))
        for _ in range(int(rng.integers(0, 4))):
            L = int(rng.choice([1, 3, 40, 70]))
            (c.update_quantized if kind == 2 else c.update)(rand((B, H, L, Dk), dtype), rand((B, H, L, Dv), dtype), fetch=False)
            if kind != 1 and rng.random() < 0.3:
                c.trim(int(rng.choice([1, 2, 1000])))
        caches.append((c, kind, dtype, B, H, Dk, Dv))
    url = str(tmp_path / "drawn.safetensors")
    kvhip.save_prompt_cache(url, [c[0] for c in caches], {"seed": str(seed)})
    loaded, meta = kvhip.load_prompt_cache(url)
    assert meta.get("seed") == str(seed) and len(loaded) == len(caches)
    for (c, kind, dtype, B, H, Dk, Dv), r in zip(caches, loaded):
        assert type(r) is type(c) and r.meta_state == c.meta_state and r.offset == c.offset
        a, b = c.state, r.state
        assert len(a) == len(b) and all(torch.equal(x, y) for x, y in zip(a, b))
        k, v = rand((B, H, 2, Dk), dtype), rand((B, H, 2, Dv), dtype)
        (c.update_quantized if kind == 2 else c.update)(k, v, fetch=False)
        (r.update_quantized if kind == 2 else r.update)(k, v, fetch=False)
        assert r.meta_state == c.meta_state and all(torch.equal(x, y) for x, y in zip(c.state, r.state))
