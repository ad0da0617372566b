"""Growth of the page store through the C ABI, never pre-sized with `reserve`: new pages come from a
further allocation and are entered into the cache's page table, so nothing that was written moves
(the reference re-concatenates its buffers on growth: KVCache.swift:419-435, :704-728, :981-989).
Contents, offsets and capacities are compared with the oracle across page, allocation and page-table
boundaries, and on a stream other than the default one."""

import numpy as np
import pytest
import torch

import kvhip
from oracle import c_oracle as CO
from oracle import kv_oracle as O
from tests.util import NAME, bits_equal, dev, err_stats, np32, randn

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_simple_cache_grows_from_empty_one_token_per_step(dtype):
    """configs[1]'s write pattern at a reduced shape: one token per step from 0 to 1300 rows (five
    reference growth steps of 256, and as many page appends here), attention checked on the way."""
    rng = np.random.default_rng(17)
    B, Hq, H, D = 2, 8, 2, 128
    c = kvhip.KVCacheSimple()
    o = O.KVCacheSimple(NAME[dtype])
    scale = D ** -0.5
    grown = []
    for t in range(1300):
        rows_before = c.device_rows
        k, kd = randn(rng, (B, H, 1, D), dtype, 0.5)
        v, vd = randn(rng, (B, H, 1, D), dtype, 0.5)
        if t in (255, 256, 257, 511, 512, 1024, 1299):
            q, qd = randn(rng, (B, Hq, 1, D), dtype)
            got = np32(c.update_attend(qd, kd, vd, scale))
            ref = O.attention_with_cache_update(q, k, v, o, scale, O.Mask.NONE, NAME[dtype])
            mx, mean = err_stats(got, ref)
            assert mx <= 1e-2 and mean <= 1e-3, (t, mx, mean)
        else:
            c.update(kd, vd, fetch=False)
            o.update(k, v)
        assert (c.offset, c.capacity) == (o.offset, o.capacity)
        if c.device_rows != rows_before:
            grown.append((t, c.device_rows))
    # device pages were added on the way (1, 2, 3, 5, 8 pages), never pre-sized
    assert grown == [(0, 256), (256, 512), (512, 768), (768, 1280), (1280, 2048)], grown
    gk, gv = c.fetch()
    ok, ov = o.keys[:, :, :o.offset], o.values[:, :, :o.offset]
    assert np.array_equal(np32(gk), ok) and np.array_equal(np32(gv), ov)


def test_quantized_cache_grows_across_allocations():
    """B32 x 8 kv heads, D 128, 4 bits (configs[2]'s shape), grown in ragged appends to 9100 rows with no
    reserve: six allocations back its pages.  Rows written before each growth must still be there
    afterwards (two (batch row, kv head) pairs against the CPU quantizer, all rows; every pair's first
    and last rows against the device's standalone quantizer)."""
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    B, H, D, GS, BITS = 32, 8, 128, 64, 4
    c = kvhip.QuantizedKVCache(GS, BITS)
    kept_k, kept_v, first, last = [], [], None, None
    total = 0
    for L in (1000, 1, 1, 3000, 97, 1, 2900, 2100):
        k = torch.randn(B, H, L, D, generator=g, device="cuda").half()
        v = (torch.randn(B, H, L, D, generator=g, device="cuda") * 3).half()
        c.update_quantized(k, v, fetch=False)
        total += L
        assert c.offset == total
        kept_k.append(k[[0, 31]][:, [0, 7]].cpu())
        kept_v.append(v[[0, 31]][:, [0, 7]].cpu())
        if first is None:
            first = (k[:, :, :2].clone(), v[:, :, :2].clone())
        last = (k[:, :, -2:].clone(), v[:, :, -2:].clone())
    st = c.state
    assert st[0].shape[2] == total == 9100
    for plane, kept in ((0, kept_k), (3, kept_v)):
        src = torch.cat(kept, dim=2).float().numpy()
        wq, s, b = CO.affine_quantize(src, GS, BITS, "float16")
        sub = [a[[0, 31]][:, [0, 7]] for a in st[plane:plane + 3]]
        assert np.array_equal(np32(sub[0]), wq)
        assert bits_equal(sub[1], s, torch.float16) and bits_equal(sub[2], b, torch.float16)
    for plane, idx in ((0, 0), (3, 1)):
        for rows, sl in ((first, slice(0, 2)), (last, slice(total - 2, total))):
            wq, s, b = kvhip.affine_quantize(rows[idx], GS, BITS)
            assert torch.equal(st[plane][:, :, sl], wq)
            assert torch.equal(st[plane + 1][:, :, sl], s) and torch.equal(st[plane + 2][:, :, sl], b)


def test_cache_outgrows_its_page_table():
    """The page table starts with room for 64 pages (16384 rows); growing past that replaces it with a
    larger one whose old entries are copied on the stream.  Contents and later appends must be
    unaffected, for a full-precision and a quantized cache."""
    rng = np.random.default_rng(23)
    for make, omake, quant in ((kvhip.KVCacheSimple, lambda: O.KVCacheSimple("float16"), False),
                               (lambda: kvhip.QuantizedKVCache(64, 8), lambda: O.QuantizedKVCache(64, 8, "float16"), True)):
        c, o = make(), omake()
        for L in (300, 1, 7000, 1, 1, 9000, 497, 1, 20000, 3):
            k, kd = randn(rng, (1, 2, L, 64), torch.float16)
            v, vd = randn(rng, (1, 2, L, 64), torch.float16)
            if quant:
                c.update_quantized(kd, vd, fetch=False)
                o.update_quantized(k, v)
            else:
                c.update(kd, vd, fetch=False)
                o.update(k, v)
        assert c.offset == o.offset == 36804
        for i, (a, b) in enumerate(zip(c.state, o.get_state())):
            if quant and i % 3 == 0:
                assert np.array_equal(np32(a), b)
            else:
                assert bits_equal(a, b, torch.float16)
        q, qd = randn(rng, (1, 4, 1, 64), torch.float16)
        got = np32(c.attend(qd, 0.125))
        if quant:
            ref = O.quantized_sdpa(q, *o.get_quantized_state(), 0.125, O.Mask.NONE, 64, 8, "float16")
        else:
            ref = O.sdpa(q, o.keys[:, :, :o.offset], o.values[:, :, :o.offset], 0.125, O.Mask.NONE, "float16")
        mx, mean = err_stats(got, ref)
        assert mx <= 1e-2 and mean <= 1e-3, (mx, mean)


def test_ring_with_staged_rows_grows_without_losing_the_window():
    """A ring whose staged round needs more spare slots than its pages hold grows by appending a page."""
    rng = np.random.default_rng(29)
    ring = kvhip.RotatingKVCache(256, keep=2)
    o = O.RotatingKVCache(256, keep=2, dtype="float16")
    for L in (200, 1, 1, 100, 1):
        k, kd = randn(rng, (1, 2, L, 64), torch.float16)
        ring.update(kd, kd, fetch=False)
        o.update(k, k)
    before = [a.clone() for a in ring.state]
    staged = kvhip.RotatingStagedKVCache(ring)
    k, kd = randn(rng, (1, 2, 300, 64), torch.float16)      # more than the ring's spare slots
    pk, _ = staged.update(kd, kd)
    assert staged.staged_count == 300
    assert torch.equal(pk[:, :, -300:], kd)
    assert all(torch.equal(a, b) for a, b in zip(ring.state, before))
    staged.commit(0)
    assert all(torch.equal(a, b) for a, b in zip(ring.state, before))
    assert ring.meta_state == o.get_meta_state()


def test_reserve_then_append_on_another_stream():
    """`reserve` zero-fills its pages on the default stream and waits for that fill, so a first append
    on a non-blocking stream cannot be overtaken by it."""
    rng = np.random.default_rng(31)
    side = torch.cuda.Stream()
    for _ in range(3):
        c = kvhip.QuantizedKVCache(64, 4)
        c.reserve(8, 8, 128, 128, torch.float16, 40000)        # 0.37 GB to clear
        k, kd = randn(rng, (8, 8, 70, 128), torch.float16)
        o = O.QuantizedKVCache(64, 4, "float16")
        o.update_quantized(k, k)
        with torch.cuda.stream(side):
            c.update_quantized(kd, kd, fetch=False)
            st = c.state
        side.synchronize()
        for i, (a, b) in enumerate(zip(st, o.get_state())):
            assert np.array_equal(np32(a), b) if i % 3 == 0 else bits_equal(a, b, torch.float16)


def test_created_grown_and_freed_caches_reuse_their_memory_without_a_blocking_call():
    # A serving loop that never calls kvhip_sync / kvhip_cache_reserve: caches are created, grown page by page,
    # read and dropped while their work may still be in flight.  Their pages go to the library's free list once the
    # work behind them has finished and later caches are served from it, so the device's free memory settles
    # instead of shrinking by one cache per iteration.
    g = torch.Generator(device="cuda")
    g.manual_seed(0)
    B, H, D = 4, 8, 128
    k = torch.randn(B, H, 2048, D, generator=g, device="cuda").half()
    q = torch.randn(B, 32, 1, D, generator=g, device="cuda").half()
    one = torch.randn(B, H, 1, D, generator=g, device="cuda").half()
    per_cache = 2 * B * H * 6144 * D * 2
    outs = []

    def serve():
        c = kvhip.KVCacheSimple()
        for _ in range(3):               # grows by slabs: 2048, 4096, 6144 rows
            c.update(k, k, fetch=False)
        outs.append(c.update_attend(q, one, one, D ** -0.5))
        del c                            # kvhip_cache_free with the stream possibly still busy

    for _ in range(4):
        serve()
    torch.cuda.current_stream().synchronize()   # torch's own wait: the library is not told
    free_mid = torch.cuda.mem_get_info()[0]
    for _ in range(24):
        serve()
    torch.cuda.current_stream().synchronize()
    free_end = torch.cuda.mem_get_info()[0]
    assert free_mid - free_end < 3 * per_cache, (free_mid - free_end, per_cache)
    assert all(torch.isfinite(o).all() for o in outs)
    # and the answers do not depend on whose memory a cache got
    assert all(torch.equal(outs[0], o) for o in outs[1:])


def test_dequantize_first_scratch_is_one_buffer_per_stream():
    """A large prompt chunk over a quantized cache runs over scratch pages the cache is dequantized into.  The scratch
    is taken from the pool at the call and retired behind it, and a call may take a buffer retired on its own stream
    without waiting for it: twelve layers' calls enqueued back to back, three rounds of them with no wait in between,
    hold one scratch buffer, not thirty-six -- and every layer's result is what it is when computed alone."""
    g = torch.Generator(device="cuda")
    g.manual_seed(3)
    B, Hkv, r, D, T, Lq = 1, 8, 4, 128, 4096, 1024
    lib = kvhip.load()
    caches = []
    for _ in range(12):
        c = kvhip.QuantizedKVCache(64, 4)
        c.update_quantized(torch.randn(B, Hkv, T, D, generator=g, device="cuda").half(), torch.randn(B, Hkv, T, D, generator=g, device="cuda").half(), fetch=False)
        caches.append(c)
    q = torch.randn(B, Hkv * r, Lq, D, generator=g, device="cuda").half()
    outs = [torch.empty_like(q) for _ in caches]
    scratch = B * Hkv * T * 2 * D * 2
    causal = kvhip.MaskMode.causal()
    alone = []
    for c in caches:                       # each layer alone (this also brings the pool to its working size)
        alone.append(c.attend(q, D ** -0.5, causal))
        assert lib.kvhip_last_attend_kernel() == 4
        torch.cuda.current_stream().synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        for c, o in zip(caches, outs):
            c.attend(q, D ** -0.5, causal, out=o)
    torch.cuda.current_stream().synchronize()
    free_after = torch.cuda.mem_get_info()[0]
    assert free_before - free_after < 2 * scratch, (free_before - free_after, scratch)
    assert all(torch.equal(a, o) for a, o in zip(alone, outs))


def test_dequantize_first_on_two_streams():
    """Calls on different streams never share a scratch buffer that is still in use: two caches attended in turn on
    two streams (default priority), ten times each with nothing waited for, give what each gives alone."""
    g = torch.Generator(device="cuda")
    g.manual_seed(4)
    B, Hkv, r, D, T, Lq = 1, 8, 4, 128, 4096, 1024
    lib = kvhip.load()
    caches, alone = [], []
    q = torch.randn(B, Hkv * r, Lq, D, generator=g, device="cuda").half()
    causal = kvhip.MaskMode.causal()
    for _ in range(2):
        c = kvhip.QuantizedKVCache(64, 4)
        c.update_quantized(torch.randn(B, Hkv, T, D, generator=g, device="cuda").half(), torch.randn(B, Hkv, T, D, generator=g, device="cuda").half(), fetch=False)
        caches.append(c)
        alone.append(c.attend(q, D ** -0.5, causal))
        assert lib.kvhip_last_attend_kernel() == 4
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [[torch.empty_like(q) for _ in range(10)] for _ in range(2)]
    for i in range(10):
        for k in range(2):
            with torch.cuda.stream(streams[k]):
                caches[k].attend(q, D ** -0.5, causal, out=outs[k][i])
    for st in streams:
        st.synchronize()
    for k in range(2):
        assert all(torch.equal(alone[k], o) for o in outs[k])
