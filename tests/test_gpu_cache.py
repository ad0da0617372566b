"""GPU parity tests of the cache write/read path through the C ABI: packed
codes, scales/biases, ring indices, trim offsets and state layouts are compared
bit for bit with the CPU oracle on the same seeded inputs."""
import numpy as np
import pytest
import torch

import kvhip
from oracle import kv_oracle as O
from tests.util import NAME, TORCH, bits_equal, dev, np32, randn

import quantizer_kats as QK

pytestmark = pytest.mark.gpu

DTYPES = [torch.float16, torch.bfloat16, torch.float32]


def positioned(lo, hi, D=2, dtype=torch.float16):
    p = np.arange(lo, hi, dtype=np.float32)
    k = np.broadcast_to(p[None, None, :, None], (1, 1, hi - lo, D)).copy()
    return (k, -k), (dev(k, dtype), dev(-k, dtype))


# ------------------------------------------------------------------ quantizer
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bits", [2, 3, 4, 5, 6, 8])
@pytest.mark.parametrize("gs", [32, 64, 128])
def test_affine_quantize_bit_exact(dtype, bits, gs):
    rng = np.random.default_rng(bits * 100 + gs)
    w = rng.standard_normal((2, 3, 19, 128)).astype(np.float32)
    w *= (10.0 ** rng.uniform(-1, 1, size=(128,))).astype(np.float32)
    w[0, 0, 0] = 0.0
    w[0, 0, 1] = 3.25
    w[0, 0, 2, :64] = -w[0, 0, 2, 64:]
    w[0, 0, 3] = np.abs(w[0, 0, 3])
    w[0, 0, 4] = -np.abs(w[0, 0, 4])
    w = O.round_to(w, NAME[dtype])
    wq, s, b = kvhip.affine_quantize(dev(w, dtype), gs, bits)
    owq, os_, ob = O.affine_quantize(w, gs, bits, NAME[dtype])
    assert np.array_equal(np32(wq), owq)
    assert bits_equal(s, os_, dtype) and bits_equal(b, ob, dtype)
    deq = kvhip.affine_dequantize(wq, s, b, gs, bits)
    assert bits_equal(deq, O.affine_dequantize(owq, os_, ob, gs, bits, NAME[dtype]), dtype)


@pytest.mark.parametrize("path", ["standalone", "append one row", "append whole tiles"])
@pytest.mark.parametrize("gs", [32, 64])
@pytest.mark.parametrize("case", QK.CASES, ids=[c["name"] for c in QK.CASES])
def test_quantizers_on_hand_worked_known_answers(case, gs, path):
    """The device quantizers (the standalone one, the per-row append kernel and the whole-tile
    append kernel, whose quotient comes from the hardware reciprocal) against literals worked out by
    hand from MLX's published CPU loop (tests/quantizer_kats.py) -- not against the oracle."""
    dtype = TORCH[case["dtype"]]
    bits, reps = case["bits"], gs // 32
    row = np.asarray(QK.group_values(case) * reps + [0.0] * gs, np.float32)       # D = 2 * gs
    rows = 1 if path != "append whole tiles" else 128
    w = np.broadcast_to(row, (1, 1, rows, 2 * gs)).copy()
    if path == "standalone":
        wq, s, b = kvhip.affine_quantize(dev(w, dtype), gs, bits)
    else:
        cache = kvhip.QuantizedKVCache(gs, bits)
        cache.update_quantized(dev(w, dtype), dev(w, dtype), fetch=False)
        st = cache.state
        for i in range(3):   # K and V planes hold the same rows (V through its transposed tile layout)
            assert torch.equal(st[i], st[i + 3])
        wq, s, b = st[0], st[1], st[2]
    words = QK.packed_words(case) * reps
    got_w = np32(wq).reshape(rows, -1)
    sb = O.to_bits(np32(s), case["dtype"]).reshape(rows, 2)
    bb = O.to_bits(np32(b), case["dtype"]).reshape(rows, 2)
    for r in range(rows):
        assert [int(x) for x in got_w[r, :len(words)]] == words, case["wrong"]
        assert not got_w[r, len(words):].any()
        assert int(sb[r, 0]) == case["scale_bits"] and int(bb[r, 0]) == case["bias_bits"], case["wrong"]
        assert int(sb[r, 1]) == {"float16": 0x8002, "bfloat16": 0xB3D7}[case["dtype"]] and int(bb[r, 1]) == 0


def check_quantized_state(cache, ocache, dtype):
    st = cache.state
    ost = ocache.get_state()
    assert len(st) == len(ost) == 6
    for i, (a, o) in enumerate(zip(st, ost)):
        assert tuple(a.shape) == tuple(o.shape), (i, a.shape, o.shape)
        if i % 3 == 0:
            assert np.array_equal(np32(a), o), f"packed codes differ in state[{i}]"
        else:
            assert bits_equal(a, o, dtype), f"scales/biases differ in state[{i}]"
    assert cache.meta_state == ocache.get_meta_state()
    assert cache.capacity == ocache.capacity


@pytest.mark.parametrize("dtype,bits,gs,D", [
    (torch.float16, 4, 64, 128), (torch.float16, 8, 64, 64), (torch.bfloat16, 4, 32, 64),
    (torch.float32, 8, 64, 128), (torch.float16, 2, 64, 128), (torch.float16, 4, 128, 256),
    # code widths that do not divide 32: a code may straddle two words of a K row / of a V tile row
    (torch.float16, 3, 64, 128), (torch.bfloat16, 5, 32, 96), (torch.float16, 6, 64, 64), (torch.float32, 3, 32, 96),
    (torch.bfloat16, 6, 128, 256), (torch.float16, 5, 64, 128),
])
def test_quantized_cache_append_trim_state(dtype, bits, gs, D):
    rng = np.random.default_rng(11)
    B, H = 2, 3
    cache = kvhip.QuantizedKVCache(gs, bits)
    ocache = O.QuantizedKVCache(gs, bits, NAME[dtype])
    # ragged schedule: crosses octets, 32-token blocks, pages and step growth; trims between
    for L, trim in [(5, 0), (1, 0), (1, 0), (37, 2), (1, 1), (300, 0), (1, 0), (4, 3), (4, 4), (4, 0), (250, 7), (1, 0)]:
        k, kd = randn(rng, (B, H, L, D), dtype, 2.0)
        v, vd = randn(rng, (B, H, L, D), dtype, 0.5)
        cache.update_quantized(kd, vd, fetch=False)
        ocache.update_quantized(k, v)
        assert cache.offset == ocache.offset
        check_quantized_state(cache, ocache, dtype)
        assert cache.trim(trim) == ocache.trim(trim)
        assert cache.offset == ocache.offset
    check_quantized_state(cache, ocache, dtype)
    # copy is independent and equal
    cp = cache.copy()
    ocp = ocache.copy()
    k, kd = randn(rng, (B, H, 3, D), dtype)
    cache.update_quantized(kd, kd, fetch=False)
    check_quantized_state(cp, ocp, dtype)
    ocache.update_quantized(k, k)
    check_quantized_state(cache, ocache, dtype)
    # state round trip into a fresh cache (restore order: state, then metaState)
    fresh = kvhip.QuantizedKVCache(gs, bits)
    fresh.state = cache.state
    fresh.meta_state = cache.meta_state
    assert fresh.offset == cache.offset
    for a, b in zip(fresh.state, cache.state):
        assert torch.equal(a, b)
    # and it keeps working after the restore
    k, kd = randn(rng, (B, H, 2, D), dtype)
    fresh.update_quantized(kd, kd, fetch=False)
    ocache2 = ocache.copy()
    ocache2.update_quantized(k, k)
    check_quantized_state(fresh, ocache2, dtype)


@pytest.mark.parametrize("bits", [4, 8])
def test_quantized_prompt_append_on_rounding_ties(bits):
    """Whole-tile appends whose quotients (w - bias) / scale sit exactly on, and within a few ulps
    of, half-integers: the codes must still be the restatement's (round-half-to-even of the
    correctly rounded quotient)."""
    rng = np.random.default_rng(31)
    B, H, L, D, gs = 1, 2, 128, 128, 64
    nb = (1 << bits) - 1
    step = 0.125 if bits == 4 else 2.0 ** -7
    k = (rng.integers(0, nb, size=(B, H, L, D)).astype(np.float32) + 0.5) * np.float32(step)   # exact ties
    near = rng.random((B, H, L, D)) < 0.3
    k = np.where(near, k * np.float32(1.0 + 2.0 ** -10), k).astype(np.float32)                  # one fp16 ulp off
    k[..., 0::gs] = 0.0                       # pin every group's extrema: scale = step exactly
    k[..., 1::gs] = nb * step
    k = O.round_to(k, "float16")
    kd = dev(k, torch.float16)
    cache = kvhip.QuantizedKVCache(gs, bits)
    ocache = O.QuantizedKVCache(gs, bits, "float16")
    cache.update_quantized(kd, kd, fetch=False)
    ocache.update_quantized(k, k)
    check_quantized_state(cache, ocache, torch.float16)
    # scales that are not powers of two: about two in 10^4 quotients land within 10^-4 of a
    # half-integer by chance, so half a million elements hold about a hundred of them
    L2 = 1920
    k2 = rng.standard_normal((B, H, L2, D)).astype(np.float32) * (10.0 ** rng.uniform(-2, 2, size=(B, H, L2, 1))).astype(np.float32)
    k2 = O.round_to(k2, "float16")
    k2d = dev(k2, torch.float16)
    cache.update_quantized(k2d, k2d, fetch=False)
    ocache.update_quantized(k2, k2)
    check_quantized_state(cache, ocache, torch.float16)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bits", [2, 3, 4, 5, 6, 8])
@pytest.mark.parametrize("D,gs", [(64, 32), (64, 64), (96, 32), (128, 32), (128, 64), (128, 128), (256, 32), (256, 64), (256, 128)])
def test_quantized_prompt_append_every_tile_shape(dtype, bits, D, gs):
    """Whole 64-token tiles for every head size, group size and code width the tile quantizer is built for (how
    many lanes share a group, and how many groups a lane works parameters out for, differ between
    them; 2-, 3-, 5- and 6-bit codes leave as bit streams), with a ragged head and tail around the tiles."""
    rng = np.random.default_rng(D + gs + bits)
    B, H = 2, 2
    cache = kvhip.QuantizedKVCache(gs, bits)
    ocache = O.QuantizedKVCache(gs, bits, NAME[dtype])
    for L in (7, 210, 64):
        k, kd = randn(rng, (B, H, L, D), dtype, 3.0)
        v, vd = randn(rng, (B, H, L, D), dtype, 0.25)
        cache.update_quantized(kd, vd, fetch=False)
        ocache.update_quantized(k, v)
        check_quantized_state(cache, ocache, dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bits,gs", [(4, 64), (8, 64), (4, 32), (8, 32)])
def test_keys_of_192_values_of_128_fill_and_convert_by_whole_tiles(dtype, bits, gs):
    """Keys and values of different head sizes: whole tiles are quantized by a launch for the keys and one for
    the values, on append and in `toQuantized`; codes and pairs are the oracle's."""
    rng = np.random.default_rng(192 + bits + gs)
    B, H = 2, 3
    cache, ocache = kvhip.QuantizedKVCache(gs, bits), O.QuantizedKVCache(gs, bits, NAME[dtype])
    c, o = kvhip.KVCacheSimple(), O.KVCacheSimple(NAME[dtype])
    for L in (7, 210, 64, 1, 300):
        k, kd = randn(rng, (B, H, L, 192), dtype, 3.0)
        v, vd = randn(rng, (B, H, L, 128), dtype, 0.25)
        cache.update_quantized(kd, vd, fetch=False)
        ocache.update_quantized(k, v)
        check_quantized_state(cache, ocache, dtype)
        c.update(kd, vd, fetch=False)
        o.update(k, v)
    assert cache.group_size == gs
    check_quantized_state(c.to_quantized(gs, bits), o.to_quantized(gs, bits), dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bits", [3, 4, 6, 8])
def test_head_size_96_converts_by_whole_tiles(dtype, bits):
    """`toQuantized` of a full-precision cache of head size 96 (twelve 16-byte chunks per row: a row's
    threads do not divide the workgroup) gives the oracle's codes and pairs."""
    rng = np.random.default_rng(96 + bits)
    c, o = kvhip.KVCacheSimple(), O.KVCacheSimple(NAME[dtype])
    for L in (200, 1, 70):
        k, kd = randn(rng, (2, 3, L, 96), dtype, 2.0)
        v, vd = randn(rng, (2, 3, L, 96), dtype, 0.5)
        c.update(kd, vd, fetch=False)
        o.update(k, v)
    check_quantized_state(c.to_quantized(32, bits), o.to_quantized(32, bits), dtype)


@pytest.mark.parametrize("kind", ["simple", "quantized"])
def test_state_of_a_cache_trimmed_back_to_empty(kind):
    """Trimming every row leaves buffers with offset 0: `state` is then arrays of no rows (a slice `[..<0]`,
    KVCache.swift:449-460, 1113-1130), which round-trip into a fresh cache."""
    rng = np.random.default_rng(2)
    k, kd = randn(rng, (2, 2, 5, 64), torch.float16)
    if kind == "simple":
        c, o = kvhip.KVCacheSimple(), O.KVCacheSimple("float16")
        c.update(kd, kd, fetch=False)
        o.update(k, k)
    else:
        c, o = kvhip.QuantizedKVCache(64, 4), O.QuantizedKVCache(64, 4, "float16")
        c.update_quantized(kd, kd, fetch=False)
        o.update_quantized(k, k)
    assert c.trim(9) == o.trim(9) == 5 and c.offset == 0
    st, ost = c.state, o.get_state()
    assert [tuple(a.shape) for a in st] == [tuple(b.shape) for b in ost] and all(a.shape[2] == 0 for a in st)
    fresh = kvhip.KVCacheSimple() if kind == "simple" else kvhip.QuantizedKVCache(64, 4)
    fresh.state = st
    fresh.meta_state = c.meta_state
    assert fresh.offset == 0
    (fresh.update_quantized if kind == "quantized" else fresh.update)(kd, kd, fetch=False)
    assert fresh.offset == 5


def test_quantized_group_size_fallback_and_errors():
    # KVCacheTests.swift:477-501: QuantizedKVCache(64, 4) fed D=32 -> groupSize 32
    rng = np.random.default_rng(0)
    c = kvhip.QuantizedKVCache(64, 4)
    k, kd = randn(rng, (1, 2, 3, 32), torch.float16)
    c.update_quantized(kd, kd, fetch=False)
    assert c.group_size == 32
    c.update_quantized(kd, kd, fetch=False)
    assert c.group_size == 32 and c.offset == 6 and c.meta_state == ["256", "6", "32", "4"]
    with pytest.raises(RuntimeError):
        c.update(kd, kd)
    bad = kvhip.QuantizedKVCache(64, 4)
    _, k5 = randn(rng, (1, 1, 2, 5), torch.float16)
    with pytest.raises(kvhip.KVHipError) as e:
        bad.update_quantized(k5, k5, fetch=False)
    assert "group sizes" in str(e.value)


# ------------------------------------------------------------------ simple
@pytest.mark.parametrize("dtype", DTYPES)
def test_simple_cache_update_fetch_state(dtype):
    rng = np.random.default_rng(5)
    B, H, Dk, Dv = 2, 2, 64, 32
    c = kvhip.KVCacheSimple()
    o = O.KVCacheSimple(NAME[dtype])
    for L, trim in [(3, 0), (1, 0), (260, 1), (1, 0), (31, 30), (5, 0), (1, 0), (512, 0)]:
        k, kd = randn(rng, (B, H, L, Dk), dtype)
        v, vd = randn(rng, (B, H, L, Dv), dtype)
        gk, gv = c.update(kd, vd)
        ok, ov = o.update(k, v)
        assert np.array_equal(np32(gk), ok) and np.array_equal(np32(gv), ov)
        assert (c.offset, c.capacity) == (o.offset, o.capacity)
        assert c.trim(trim) == o.trim(trim)
    st, ost = c.state, o.get_state()
    assert all(np.array_equal(np32(a), b) for a, b in zip(st, ost))
    assert c.meta_state == [""] and c.is_trimmable and c.max_size is None
    cp = c.copy()
    assert cp.offset == c.offset and all(torch.equal(a, b) for a, b in zip(cp.state, c.state))
    _, kd = randn(rng, (B, H, 1, Dk), dtype)
    _, vd = randn(rng, (B, H, 1, Dv), dtype)
    c.update(kd, vd, fetch=False)
    assert cp.offset == c.offset - 1
    fresh = kvhip.KVCacheSimple()
    fresh.state = st
    assert fresh.offset == st[0].shape[2]
    assert all(torch.equal(a, b) for a, b in zip(fresh.state, st))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D", [64, 96, 128, 256, (192, 128)])
def test_simple_cache_prompt_sized_appends(dtype, D):
    """Appends that cover whole 64-token tiles take the tile kernel (head rows, tiles, tail rows)."""
    rng = np.random.default_rng(21)
    B, H = 2, 3
    Dk, Dv = D if isinstance(D, tuple) else (D, D)
    c = kvhip.KVCacheSimple()
    o = O.KVCacheSimple(NAME[dtype])
    for L, trim in [(37, 0), (200, 5), (64, 0), (1, 0), (459, 3), (128, 0)]:
        k, kd = randn(rng, (B, H, L, Dk), dtype)
        v, vd = randn(rng, (B, H, L, Dv), dtype)
        gk, gv = c.update(kd, vd)
        ok, ov = o.update(k, v)
        assert np.array_equal(np32(gk), ok) and np.array_equal(np32(gv), ov)
        assert c.trim(trim) == o.trim(trim)


def test_dynamic_conversion_at_compression_start():
    """`maybeAffineQuantizeKVCache` (KVCache.swift:2500-2520): simple caches past the threshold
    become quantized caches holding the same rows (bit-exact with the oracle's bulk quantize);
    rings, already quantized caches and heads no group size divides stay as they are."""
    rng = np.random.default_rng(4)
    dtype = torch.float16
    k, kd = randn(rng, (1, 2, 40, 64), dtype)
    v, vd = randn(rng, (1, 2, 40, 64), dtype)
    long_, short, ring, odd = kvhip.KVCacheSimple(), kvhip.KVCacheSimple(), kvhip.RotatingKVCache(64), kvhip.KVCacheSimple()
    long_.update(kd, vd, fetch=False)
    short.update(kd[:, :, :8].contiguous(), vd[:, :, :8].contiguous(), fetch=False)
    ring.update(kd, vd, fetch=False)
    _, k5 = randn(rng, (1, 1, 40, 5), dtype)
    odd.update(k5, k5, fetch=False)
    already = kvhip.QuantizedKVCache(64, 8)
    caches = [long_, short, ring, odd, already]
    assert kvhip.resolve_affine_scheme("affine4") == (4, 64) and kvhip.resolve_affine_scheme("turbo4") is None
    done = kvhip.maybe_affine_quantize_kv_cache(caches, 4, 64, 16)
    assert done is False                      # `short` still waits for the threshold
    assert isinstance(caches[0], kvhip.QuantizedKVCache) and caches[0].offset == 40
    assert caches[1] is short and caches[2] is ring and caches[3] is odd and caches[4] is already
    o = O.KVCacheSimple("float16")
    o.update(k, v)
    check_quantized_state(caches[0], o.to_quantized(64, 4), dtype)
    short.update(kd[:, :, 8:20].contiguous(), vd[:, :, 8:20].contiguous(), fetch=False)
    assert kvhip.maybe_affine_quantize_kv_cache(caches, 4, 64, 16) is True
    assert isinstance(caches[1], kvhip.QuantizedKVCache) and caches[1].offset == 20


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_simple_to_quantized_and_back(dtype):
    rng = np.random.default_rng(9)
    c = kvhip.KVCacheSimple()
    o = O.KVCacheSimple(NAME[dtype])
    for L in (70, 1, 1):
        k, kd = randn(rng, (2, 2, L, 64), dtype)
        v, vd = randn(rng, (2, 2, L, 64), dtype)
        c.update(kd, vd, fetch=False)
        o.update(k, v)
    c.trim(1)
    o.trim(1)
    q = c.to_quantized(64, 4)
    oq = o.to_quantized(64, 4)
    check_quantized_state(q, oq, dtype)
    for bits in (3, 5, 6):
        qb, ob = c.to_quantized(32, bits), o.to_quantized(32, bits)
        check_quantized_state(qb, ob, dtype)
        for a, b in zip(qb.to_unquantized().state, ob.to_unquantized().get_state()):
            assert bits_equal(a, b, dtype)
    # empty Simple, offset 7, toQuantized(128, 4) -> ["256","7","128","4"] (KVCacheTests.swift:526-536)
    e = kvhip.KVCacheSimple()
    e.offset = 7
    assert e.to_quantized(128, 4).meta_state == ["256", "7", "128", "4"]
    # D=5 cannot be quantized; RotatingKVCache never can (KVCacheTests.swift:538-551)
    s5 = kvhip.KVCacheSimple()
    _, k5 = randn(rng, (1, 1, 2, 5), dtype)
    s5.update(k5, k5, fetch=False)
    with pytest.raises(kvhip.KVHipError):
        s5.to_quantized()
    r = kvhip.RotatingKVCache(8)
    with pytest.raises(kvhip.KVHipError):
        r.to_quantized()
    # back to full precision
    u = q.to_unquantized()
    ou = oq.to_unquantized()
    assert u.offset == ou.offset
    for a, b in zip(u.state, ou.get_state()):
        assert bits_equal(a, b, dtype)


# ------------------------------------------------------------------ rotating
def drive_pair(c, o, ks, vs, dtype):
    gk, gv = c.update(dev(ks, dtype), dev(vs, dtype))
    ok, ov = o.update(ks, vs)
    assert np.array_equal(np32(gk), ok), "presented keys differ"
    assert np.array_equal(np32(gv), ov), "presented values differ"
    assert c.meta_state == o.get_meta_state()
    assert c.presented_length == ok.shape[2]


@pytest.mark.parametrize("keep", [0, 2])
def test_rotating_single_token_ring_and_logical_view(keep):
    # KVCacheTests.swift:1312-1404
    dtype = torch.float16
    c = kvhip.RotatingKVCache(8, keep=keep)
    o = O.RotatingKVCache(8, keep=keep)
    assert c.logical_view(8) is None
    for p in range(20):
        (k, v), _ = positioned(p, p + 1)
        drive_pair(c, o, k, v, dtype)
        assert c.idx == o.idx and c.offset == o.offset
    for tail in (8, 7, 5, 3, 2, 1, 0, -1, 99):
        gk, gv = c.logical_view(tail)
        ok, ov = o.logical_view(tail)
        assert np.array_equal(np32(gk), ok) and np.array_equal(np32(gv), ov), tail
    if keep == 0:
        assert [int(x) for x in np32(c.logical_view(8)[0])[0, 0, :, 0]] == list(range(12, 20))
        assert [int(x) for x in np32(c.logical_view(3)[0])[0, 0, :, 0]] == [17, 18, 19]
    else:
        assert [int(x) for x in np32(c.logical_view(5)[0])[0, 0, :, 0]] == [0, 1, 17, 18, 19]
        assert [int(x) for x in np32(c.logical_view(1)[0])[0, 0, :, 0]] == [0, 1]
    # reads leave the ring untouched
    before = (c.meta_state, [a.clone() for a in c.state])
    c.logical_view(7)
    assert before[0] == c.meta_state and all(torch.equal(a, b) for a, b in zip(before[1], c.state))
    assert not c.is_trimmable and c.max_size == 8


def test_rotating_view_plus_new_rows_equals_write_presentation():
    # KVCacheTests.swift:1409-1446
    dtype = torch.float16
    c = kvhip.RotatingKVCache(8)
    o = O.RotatingKVCache(8)
    for p in range(20):
        (k, v), _ = positioned(p, p + 1)
        drive_pair(c, o, k, v, dtype)
    vk, vv = c.logical_view(7)
    mask = c.make_mask(4, 8, False)
    omask = o.make_mask(4, 8, False)
    (k, v), (kd, vd) = positioned(20, 24)
    pk, pv = c.update(kd, vd)
    assert torch.equal(pk, torch.cat([vk, kd], 2)) and torch.equal(pv, torch.cat([vv, vd], 2))
    assert mask.array.shape == (4, 11) and np.array_equal(mask.array.cpu().numpy(), omask.array)


@pytest.mark.parametrize("M,keep,step,schedule", [
    (8, 0, 256, [1, 1, 1, 4, 1, 1, 6, 1, 1, 1, 1, 1, 1, 1, 1, 1, 3, 9, 1, 1, 12, 1, 1]),
    (8, 2, 4, [3, 1, 1, 1, 1, 1, 1, 1, 1, 5, 1, 1, 1, 1, 1, 1, 1, 1, 1, 2, 1]),
    (16, 4, 3, [1] * 5 + [7] + [1] * 30 + [20] + [1] * 20 + [2, 2, 2] + [1] * 20),
    (64, 4, 256, [32, 32, 32, 32, 1, 1, 1, 32, 1] + [1] * 70 + [40, 1, 1]),
    (300, 4, 256, [128, 128, 128, 128, 128] + [1] * 310 + [128, 1, 1]),
])
def test_rotating_mixed_updates_match_reference_buffers(M, keep, step, schedule):
    """Every update's presentation, metaState (offset, idx) and state equal the
    reference's buffers row for row, through growth, wrap, front-trim and re-linearisation."""
    dtype = torch.float16
    c = kvhip.RotatingKVCache(M, keep=keep, step=step)
    o = O.RotatingKVCache(M, keep=keep, step=step)
    pos = 0
    for L in schedule:
        (k, v), _ = positioned(pos, pos + L, D=4)
        drive_pair(c, o, k, v, dtype)
        pos += L
        assert c.is_trimmable == o.is_trimmable
    st, ost = c.state, o.get_state()
    assert all(np.array_equal(np32(a), b) for a, b in zip(st, ost))
    # copy + state/meta restore
    cp = c.copy()
    assert cp.meta_state == c.meta_state and all(torch.equal(a, b) for a, b in zip(cp.state, st))
    fresh = kvhip.RotatingKVCache(M)
    fresh.state = st
    fresh.meta_state = c.meta_state
    (k, v), _ = positioned(pos, pos + 1, D=4)
    o2 = o.copy()
    drive_pair(fresh, o, k, v, dtype)
    drive_pair(cp, o2, k, v, dtype)


def test_rotating_trim_then_write():
    # trim is pure bookkeeping: offset -= n, idx -= n (KVCache.swift:826-831)
    dtype = torch.float16
    c = kvhip.RotatingKVCache(32)
    o = O.RotatingKVCache(32)
    pos = 0
    for L, trim in [(5, 0), (4, 3), (4, 4), (4, 0), (1, 0), (4, 2), (1, 1), (1, 0)]:
        (k, v), _ = positioned(pos, pos + L, D=4)
        drive_pair(c, o, k, v, dtype)
        pos += L
        assert c.is_trimmable_after(L) == o.is_trimmable_after(L)
        assert c.trim(trim) == o.trim(trim)
        pos -= trim
        assert c.meta_state == o.get_meta_state()


def test_rotating_cfg4_trace_reduced():
    """BASELINE config 4 at reduced batch/heads: maxSize 4096, keep 4, 512-token chunks
    wrap the ring three times, then single-token decode (lengths from KVCache.swift:660-740)."""
    dtype = torch.bfloat16
    c = kvhip.RotatingKVCache(4096, keep=4)
    o = O.RotatingKVCache(4096, keep=4, dtype="bfloat16")
    rng = np.random.default_rng(4)
    lens = []
    for i in range(24):
        k, kd = randn(rng, (1, 1, 512, 8), dtype)
        c.update(kd, kd, fetch=False)
        o.update(k, k)
        lens.append(c.presented_length)
        assert c.meta_state == o.get_meta_state()
    assert lens[:8] == [512 * i for i in range(1, 9)] and all(n == 4607 for n in lens[8:])
    gk, _ = c.fetch()
    assert np.array_equal(np32(gk), o.keys)
    for i in range(5):
        k, kd = randn(rng, (1, 1, 1, 8), dtype)
        gk, _ = c.update(kd, kd)
        ok, _ = o.update(k, k)
        assert np.array_equal(np32(gk), ok) and c.meta_state == o.get_meta_state()
    assert c.presented_length == 4096 and (c.offset, c.idx) == (12293, 9)


def test_mask_materialize_matches_create_causal_mask():
    c = kvhip.KVCacheSimple()
    c.offset = 37
    for n, w, ra in [(5, None, True), (9, 4, False), (3, 8, True)]:
        m = c.make_mask(n, w, ra)
        om = O.base_make_mask(37, n, w, ra)
        assert np.array_equal(m.array.cpu().numpy(), om.array)
    r = kvhip.RotatingKVCache(16)
    o = O.RotatingKVCache(16)
    r.meta_state = ["0", "16", "256", "21", "5"]
    o.set_meta_state(["0", "16", "256", "21", "5"])
    m, om = r.make_mask(1, 8), o.make_mask(1, 8)
    assert np.array_equal(m.array.cpu().numpy(), om.array)
