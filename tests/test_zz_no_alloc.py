"""The allocation-free attention entry point (`kvhip_cache_attend_static`) against the ordinary one
(`kvhip_cache_attend`) through the C ABI: same kernels, scratch in the library's fixed device array
instead of the cache's own workspace.  Two calls in a row share that array, the second on a smaller
input, and each must reproduce the ordinary entry point's output bit for bit."""
import numpy as np
import pytest
import torch

import kvhip
from kvhip import _lib as L

pytestmark = pytest.mark.gpu


def filled(kind, B, Hkv, T, D, dtype, seed, **kw):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    cache = kind(**kw)
    k = torch.randn(B, Hkv, T, D, generator=g, device="cuda").to(dtype)
    v = torch.randn(B, Hkv, T, D, generator=g, device="cuda").to(dtype)
    if isinstance(cache, kvhip.QuantizedKVCache):
        cache.update_quantized(k, v, fetch=False)
    else:
        cache.update(k, v, fetch=False)
    return cache, g


def both(cache, q, scale, mask=None):
    want = cache.attend(q, scale, mask)
    family = kvhip.load().kvhip_last_attend_kernel()
    got = torch.full_like(want, float("nan"))
    cache.attend(q, scale, mask, out=got, static_scratch=True)
    assert kvhip.load().kvhip_last_attend_kernel() == family
    torch.cuda.synchronize()
    return got, want, family


def test_static_scratch_matches_the_allocating_entry_point_twice_in_a_row():
    # first call: many spans per (batch row, kv head) pair, so the partials fill a large part of the array
    big, g = filled(kvhip.QuantizedKVCache, 2, 2, 9000, 128, torch.float16, 1, group_size=64, bits=4)
    q = torch.randn(2, 8, 1, 128, generator=g, device="cuda").half()
    got, want, family = both(big, q, 128 ** -0.5)
    assert family == 1
    assert torch.equal(got, want)
    # second call, smaller input, 16-row kernel with a ragged index mask: must not see the first call's partials
    small, g = filled(kvhip.QuantizedKVCache, 3, 2, 700, 128, torch.float16, 2, group_size=64, bits=4)
    q = torch.randn(3, 8, 4, 128, generator=g, device="cuda").half()
    pad = torch.tensor([0, 100, 650], dtype=torch.int32, device="cuda")
    mask = kvhip.MaskMode.window_mask(700 - 4, 0, left_pad=pad)
    got, want, family = both(small, q, 128 ** -0.5, mask)
    assert family == 1
    assert torch.equal(got, want)
    # and the first cache again, after the array has held something else
    q = torch.randn(2, 8, 1, 128, generator=g, device="cuda").half()
    got, want, _ = both(big, q, 128 ** -0.5)
    assert torch.equal(got, want)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_static_scratch_full_precision_and_ring(dtype):
    c, g = filled(kvhip.KVCacheSimple, 2, 4, 3000, 128, dtype, 3)
    q = torch.randn(2, 8, 1, 128, generator=g, device="cuda").to(dtype)
    got, want, family = both(c, q, 0.09)
    assert family == 2 and torch.equal(got, want)
    ring, g = filled(kvhip.RotatingKVCache, 1, 2, 300, 64, dtype, 4, max_size=256, keep=4)
    for _ in range(5):
        k = torch.randn(1, 2, 1, 64, generator=g, device="cuda").to(dtype)
        ring.update(k, k, fetch=False)
    q = torch.randn(1, 4, 1, 64, generator=g, device="cuda").to(dtype)
    got, want, _ = both(ring, q, 0.125)
    assert torch.equal(got, want)
    # the prefill tile with a split key range also takes its partials from the array
    q = torch.randn(2, 8, 40, 128, generator=g, device="cuda").to(dtype)
    got, want, family = both(c, q, 0.09, kvhip.MaskMode.causal())
    assert family == 3 and torch.equal(got, want)


def test_static_scratch_rejects_what_does_not_fit():
    # the plain kernel (here: a quantized cache whose scales are float32) materialises one float per (query row, key):
    # 4 * 32 * 64 * 40000 * 4 bytes > 16 MiB
    c, g = filled(kvhip.QuantizedKVCache, 4, 8, 40000, 32, torch.float32, 5, group_size=32, bits=8)
    q = torch.randn(4, 32, 64, 32, generator=g, device="cuda")
    out = torch.zeros(4, 32, 64, 32, device="cuda")
    with pytest.raises(L.KVHipError) as e:
        c.attend(q, 0.2, out=out, static_scratch=True)
    assert e.value.status == -3 and "scratch" in str(e.value)
    torch.cuda.synchronize()
    assert not out.any(), "a rejected call must enqueue nothing"
    # the allocating entry point still serves it
    assert torch.isfinite(c.attend(q[:, :, :2].contiguous(), 0.2)).all()


def test_static_scratch_alone_on_a_fresh_cache_allocates_nothing():
    # a cache that has never gone through the allocating entry point, so its own workspace does not exist: the
    # result must come from the fixed array.  Device memory is observed around the calls (hipMemGetInfo), and the
    # result is checked against the oracle rather than against another call of the library.
    from oracle import c_oracle as CO
    from oracle import kv_oracle as O
    rng = np.random.default_rng(11)
    B, Hq, Hkv, T, D = 2, 8, 2, 9000, 128
    k = O.round_to(rng.standard_normal((B, Hkv, T, D)).astype(np.float32), "float16")
    v = O.round_to(rng.standard_normal((B, Hkv, T, D)).astype(np.float32), "float16")
    qn = O.round_to(rng.standard_normal((B, Hq, 1, D)).astype(np.float32), "float16")
    cache = kvhip.QuantizedKVCache(64, 4)
    cache.update_quantized(torch.from_numpy(k).half().cuda(), torch.from_numpy(v).half().cuda(), fetch=False)
    q = torch.from_numpy(qn).half().cuda()
    out = torch.full((B, Hq, 1, D), float("nan"), dtype=torch.float16, device="cuda")
    q4 = torch.from_numpy(O.round_to(rng.standard_normal((B, Hq, 4, D)).astype(np.float32), "float16")).half().cuda()
    out4 = torch.full((B, Hq, 4, D), float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    cache.attend(q, D ** -0.5, out=out, static_scratch=True)                     # 4-row kernel, many spans
    cache.attend(q4, D ** -0.5, kvhip.MaskMode.causal(), out=out4, static_scratch=True)  # 16-row kernel
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the allocation-free entry point changed the device's free memory"
    o = O.QuantizedKVCache(64, 4, "float16")
    qk, qv = o.update_quantized(k, v)
    ref = CO.qsdpa(qn, qk, qv, D ** -0.5, None, 64, 4, "float16")
    d = np.abs(out.float().cpu().numpy() - ref)
    assert d.max() <= 1e-2 and d.mean() <= 1e-3
    ref4 = CO.qsdpa(q4.float().cpu().numpy(), qk, qv, D ** -0.5, "causal", 64, 4, "float16")
    d = np.abs(out4.float().cpu().numpy() - ref4)
    assert d.max() <= 1e-2 and d.mean() <= 1e-3


def test_static_scratch_takes_large_batches_and_plans_fewer_parts_when_the_array_is_small():
    # many (batch row, kv head) pairs: one span each, the kernel writes the output itself and needs no scratch,
    # whatever the number of pairs (1024 pairs x 16 rows x 258 floats would be 16.9 MB of partials)
    big, g = filled(kvhip.QuantizedKVCache, 128, 8, 200, 256, torch.float16, 6, group_size=64, bits=4)
    q = torch.randn(128, 32, 4, 256, generator=g, device="cuda").half()
    got, want, family = both(big, q, 256 ** -0.5, kvhip.MaskMode.causal())
    assert family == 1 and torch.equal(got, want)
    del big
    # a prompt chunk whose two key-range parts would need 25.5 MB of partials: the allocating entry point splits the
    # keys, the allocation-free one plans a single part (another summation order: compared within the tolerance)
    c, g = filled(kvhip.KVCacheSimple, 1, 8, 1024, 128, torch.float16, 7)
    q = torch.randn(1, 32, 768, 128, generator=g, device="cuda").half()
    got, want, family = both(c, q, 128 ** -0.5, kvhip.MaskMode.causal())
    assert family == 3
    d = (got.float() - want.float()).abs()
    assert float(d.max()) <= 2e-3 and float(d.mean()) <= 1e-4
