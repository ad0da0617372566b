"""Pins the CPU oracle against the known answers held by the reference's own
tests (integers: offsets, ring order, trim counts, mask truth tables, group
size resolution, metaState strings) and against what the mathematics fixes for
the affine quantizer (closed forms, invariants, an independent scalar
implementation).  Citations are file:line in the reference's Tests/MLXLMTests.
"""
import numpy as np
import pytest

from oracle import kv_oracle as O
from oracle import c_oracle as CO

import quantizer_kats as QK


def positioned_kv(lo, hi, head_dim=2):
    """positionedKV (KVCacheTests.swift:1282-1293): keys hold +p, values -p."""
    p = np.arange(lo, hi, dtype=np.float32)
    k = np.broadcast_to(p[None, None, :, None], (1, 1, hi - lo, head_dim)).copy()
    return k, -k


def encoded(keys):
    return [int(x) for x in keys[0, 0, :, 0]]


def fill_one_at_a_time(cache, lo, hi):
    for p in range(lo, hi):
        cache.update(*positioned_kv(p, p + 1))


# ---------------------------------------------------------------- trimmability
def test_rotating_trimmable_prediction():
    # KVCacheTests.swift:136-154
    c = O.RotatingKVCache(8)
    c.offset = 3
    assert c.is_trimmable_after(4) and not c.is_trimmable_after(5)
    for off in (8, 9):
        c.offset = off
        assert not c.is_trimmable


# ---------------------------------------------------------------- group size
def test_group_size_resolution():
    # KVCacheTests.swift:477-501, Gemma4TextTests.swift:18-21
    assert O.resolved_group_size(64, 32, 32) == 32
    assert O.resolved_group_size(64, 128, 128) == 64
    assert O.resolved_group_size(64, 5, 5) is None
    assert O.resolved_group_size(48, 128, 128) == 32  # tie -> smaller
    c = O.QuantizedKVCache(64, 4)
    k = np.random.default_rng(0).standard_normal((1, 2, 3, 32)).astype(np.float16).astype(np.float32)
    c.update_quantized(k, k)
    assert c.group_size == 32
    c.update_quantized(k, k)
    assert c.group_size == 32 and c.offset == 6


def test_quantized_meta_state_roundtrip():
    # KVCacheTests.swift:503-512
    c = O.QuantizedKVCache(64, 8)
    c.set_meta_state(["256", "11", "32", "4"])
    assert (c.offset, c.group_size, c.bits) == (11, 32, 4)
    assert c.get_meta_state() == ["256", "11", "32", "4"]


def test_empty_simple_to_quantized_meta():
    # KVCacheTests.swift:526-536
    s = O.KVCacheSimple()
    s.offset = 7
    q = s.to_quantized(128, 4)
    assert q.get_meta_state() == ["256", "7", "128", "4"]


def test_to_quantized_errors():
    # KVCacheTests.swift:538-551
    s = O.KVCacheSimple()
    k = np.zeros((1, 1, 2, 5), np.float32)
    s.update(k, k)
    with pytest.raises(ValueError):
        s.to_quantized()
    with pytest.raises(ValueError):
        O.RotatingKVCache(8).to_quantized()


def test_rotating_meta_legacy_five_fields():
    # KVCacheTests.swift:553-603 (legacy 5-field rotating meta -> modelNative)
    c = O.RotatingKVCache(8)
    c.set_meta_state(["0", "16", "256", "3", "3"])
    assert c.get_meta_state() == ["0", "16", "256", "3", "3", "modelNative"]
    with pytest.raises(ValueError):
        c.set_meta_state(["0", "16", "256", "3", "3", "bogus"])
    with pytest.raises(ValueError):
        c.set_meta_state(["0", "x", "256", "3", "3"])


# ---------------------------------------------------------------- masks
def test_simple_mask_modes_and_truth_table():
    # KVCacheTests.swift:816-848
    c = O.KVCacheSimple()
    assert c.make_mask(3).mode == "causal"
    assert c.make_mask(1).mode == "none"
    c.offset = 2
    m = c.make_mask(3, return_array=True)
    assert m.mode == "array" and m.array.shape == (3, 5)
    T, F = True, False
    assert m.array.tolist() == [[T, T, T, F, F], [T, T, T, T, F], [T, T, T, T, T]]


# ---------------------------------------------------------------- ring
def test_logical_view_nil_before_write():
    assert O.RotatingKVCache(8).logical_view(8) is None  # :1308-1310


def test_logical_view_past_wrap():
    # KVCacheTests.swift:1312-1327
    c = O.RotatingKVCache(8, keep=0)
    fill_one_at_a_time(c, 0, 20)
    assert c.offset == 20
    k, v = c.logical_view(8)
    assert encoded(k) == list(range(12, 20))
    assert [-x for x in encoded(v)] == list(range(12, 20))
    assert encoded(c.logical_view(3)[0]) == [17, 18, 19]


def test_logical_view_clamps():
    # KVCacheTests.swift:1329-1337
    c = O.RotatingKVCache(8)
    fill_one_at_a_time(c, 0, 5)
    assert encoded(c.logical_view(99)[0]) == [0, 1, 2, 3, 4]
    assert encoded(c.logical_view(5)[0]) == [0, 1, 2, 3, 4]
    assert c.logical_view(0)[0].shape[2] == 0
    assert c.logical_view(-1)[0].shape[2] == 0


def test_logical_view_read_only():
    # KVCacheTests.swift:1339-1360
    c = O.RotatingKVCache(8)
    fill_one_at_a_time(c, 0, 20)
    before = (c.keys.copy(), c.values.copy(), c.offset, c.get_meta_state())
    c.logical_view(7)
    c.logical_view(3)
    assert np.array_equal(before[0], c.keys) and np.array_equal(before[1], c.values)
    assert before[2] == c.offset and before[3] == c.get_meta_state()


def test_logical_view_pinned_prefix():
    # KVCacheTests.swift:1362-1404
    c = O.RotatingKVCache(8, keep=2)
    fill_one_at_a_time(c, 0, 20)
    pos = encoded(c.logical_view(5)[0])
    assert len(pos) == 5 and pos[:2] == [0, 1] and sorted(pos[2:]) == pos[2:]
    assert pos[2:] == [17, 18, 19]
    for tail in range(3):
        k, v = c.logical_view(tail)
        assert encoded(k) == [0, 1] and [-x for x in encoded(v)] == [0, 1]
    p3 = encoded(c.logical_view(3)[0])
    assert len(p3) == 3 and p3[:2] == [0, 1]
    c = O.RotatingKVCache(8, keep=4)
    fill_one_at_a_time(c, 0, 2)
    assert encoded(c.logical_view(0)[0]) == [0, 1]
    assert encoded(c.logical_view(9)[0]) == [0, 1]


def test_logical_view_plus_new_rows_equals_write_presentation():
    # KVCacheTests.swift:1409-1446
    window, staged = 8, 4
    c = O.RotatingKVCache(window)
    fill_one_at_a_time(c, 0, 20)
    vk, vv = (a.copy() for a in c.logical_view(window - 1))
    mask = c.make_mask(staged, window, False)
    nk, nv = positioned_kv(20, 24)
    pk, pv = c.update(nk, nv)
    assert np.array_equal(pk, np.concatenate([vk, nk], 2))
    assert np.array_equal(pv, np.concatenate([vv, nv], 2))
    assert mask.mode == "array" and mask.array.shape[-1] == pk.shape[2] and mask.array.shape[-2] == staged


def test_attention_past_wrap_matches_never_rotated_reference():
    # KVCacheTests.swift:1451-1491
    rng = np.random.default_rng(0)
    window, history, nq, heads, hd = 8, 20, 4, 2, 4
    scale = 1.0 / np.sqrt(hd)
    ak = rng.standard_normal((1, heads, history + nq, hd)).astype(np.float32)
    av = rng.standard_normal((1, heads, history + nq, hd)).astype(np.float32)
    q = rng.standard_normal((1, heads, nq, hd)).astype(np.float32)
    c = O.RotatingKVCache(window, dtype="float32")
    for p in range(history):
        c.update(ak[:, :, p:p + 1], av[:, :, p:p + 1])
    mask = c.make_mask(nq, window, False)
    ck, cv = c.update(ak[:, :, history:], av[:, :, history:])
    out = O.sdpa(q, ck, cv, scale, mask, "float32")
    qp = np.arange(history, history + nq)[:, None]
    kp = np.arange(history + nq)[None, :]
    ref_mask = (qp >= kp) & (qp < kp + window)
    ref = O.sdpa(q, ak, av, scale, O.Mask("array", ref_mask), "float32")
    assert np.allclose(out, ref, rtol=1e-5, atol=1e-5)


def test_cfg4_trace():
    """Chunked prefill through a ring of 4096/keep 4 with 512-token chunks, then
    single-token decode: buffer lengths, offset and idx follow from
    KVCache.swift:660-740."""
    c = O.RotatingKVCache(4096, keep=4)
    z = np.zeros((1, 1, 512, 2), np.float32)
    lens = []
    for _ in range(24):
        k, _ = c.update(z, z)
        lens.append(k.shape[2])
    assert lens[:8] == [512 * i for i in range(1, 9)]
    assert all(n == 4607 for n in lens[8:])
    assert (c.offset, c.idx) == (12288, 4607)
    z1 = np.zeros((1, 1, 1, 2), np.float32)
    k, _ = c.update(z1, z1)
    assert k.shape[2] == 4096 and (c.offset, c.idx) == (12289, 5)
    for _ in range(4096 - 5):
        c.update(z1, z1)
    assert c.idx == 4096
    c.update(z1, z1)
    assert c.idx == 5


def test_single_token_slot_formula():
    # slot(t) = t for t < M, else keep + (t - M) mod (M - keep)
    M, keep = 8, 2
    c = O.RotatingKVCache(M, keep=keep)
    for t in range(40):
        c.update(*positioned_kv(t, t + 1))
        slot = t if t < M else keep + (t - M) % (M - keep)
        assert int(c.keys[0, 0, slot, 0]) == t and c.idx == slot + 1


# ---------------------------------------------------------------- staged rounds
@pytest.mark.parametrize("window,keep,prefill,schedule", [
    (8, 0, 7, [(4, 1), (4, 4), (4, 0), (4, 2), (4, 3), (4, 1), (4, 4), (4, 2), (4, 0), (4, 3)]),
    (8, 2, 7, [(4, 1), (4, 4), (4, 0), (4, 2), (4, 3)]),
    (4, 0, 3, [(6, 2), (8, 8), (6, 0), (8, 5)]),
])
def test_staged_commit_equals_accepted_only_replay(window, keep, prefill, schedule):
    # KVCacheRoundTests.swift:286-327: staging then commit(retaining: a) leaves the
    # ring exactly as writing only the accepted rows would.
    live = O.RotatingKVCache(window, keep=keep)
    replay = O.RotatingKVCache(window, keep=keep)
    k, v = positioned_kv(0, prefill)
    live.update(k, v)
    replay.update(k, v)
    pos = prefill
    for written, accepted in schedule:
        st = O.RotatingStagedKVCache(live)
        nk, nv = positioned_kv(pos, pos + written)
        st.update(nk, nv)
        st.commit(accepted)
        if accepted > 0:
            replay.update(nk[:, :, :accepted], nv[:, :, :accepted])
        pos += accepted
        assert live.get_meta_state() == replay.get_meta_state()
        assert np.array_equal(live.keys, replay.keys)


def test_trim_prompt_cache_counts():
    # KVCache.swift:2302-2306 with SpeculativeDecodingTests.swift:219-261 style offsets
    caches = [O.KVCacheSimple(), O.QuantizedKVCache(64, 4)]
    caches[0].offset = 4
    caches[1].offset = 4
    assert O.trim_prompt_cache(caches, 3) == 3 and [c.offset for c in caches] == [1, 1]
    assert O.trim_prompt_cache(caches, 5) == 1 and [c.offset for c in caches] == [0, 0]


# ---------------------------------------------------------------- quantizer
@pytest.mark.parametrize("bits", [2, 4, 8])
@pytest.mark.parametrize("gs", [32, 64, 128])
@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "float32"])
def test_quantize_numpy_vs_scalar_c(bits, gs, dtype):
    """Two independent restatements (vectorised numpy, scalar C) agree bit for bit."""
    rng = np.random.default_rng(bits * 1000 + gs)
    w = rng.standard_normal((3, 2, 17, 128)).astype(np.float32)
    w *= 10.0 ** rng.uniform(-1, 1, size=(128,)).astype(np.float32)
    w[0, 0, 0] = 0.0           # all-zero groups
    w[0, 0, 1] = 3.25          # constant groups
    w[0, 0, 2, :64] = -w[0, 0, 2, 64:]
    w = O.round_to(w, dtype)
    a = O.affine_quantize(w, gs, bits, dtype)
    b = CO.affine_quantize(w, gs, bits, dtype)
    assert np.array_equal(a[0], b[0])
    assert np.array_equal(O.to_bits(a[1], dtype), O.to_bits(b[1], dtype))
    assert np.array_equal(O.to_bits(a[2], dtype), O.to_bits(b[2], dtype))
    da = O.affine_dequantize(*a, gs, bits, dtype)
    db = CO.affine_dequantize(*b, gs, bits, dtype)
    assert np.array_equal(da, db)


@pytest.mark.parametrize("bits", [3, 4, 5, 6, 8])
def test_quantize_closed_forms(bits):
    gs, D = 64, 128
    nb = (1 << bits) - 1
    # all-zero group: code 0, scale T(-1e-7), bias 0
    wq, s, b = O.affine_quantize(np.zeros((1, D), np.float32), gs, bits, "float16")
    assert not wq.any() and not b.any()
    assert np.all(s == np.float32(np.float16(-1e-7)))
    # constant group c: scale eps-signed, q0 = rint(c/-1e-7) != 0 -> scale = c/q0, bias = c, codes 0
    wq, s, b = O.affine_quantize(np.full((1, D), 2.5, np.float32), gs, bits, "float32")
    assert not wq.any() and np.all(b == 2.5)
    # integers in [0, nb] with both ends present in every group: edge is w_max = nb,
    # scale = -1, q0 = -nb, scale = nb / -nb = -1, bias = nb, code(x) = nb - x (all exact)
    ramp = np.rint((np.arange(D) % gs) * (nb / (gs - 1.0))).astype(np.float32)[None]
    wq, s, b = O.affine_quantize(ramp, gs, bits, "float32")
    codes = O.unpack_codes(wq, bits)
    assert np.all(s == -1.0) and np.all(b == nb)
    assert np.array_equal(codes[0], (nb - ramp[0]).astype(np.uint32))
    assert np.array_equal(O.affine_dequantize(wq, s, b, gs, bits, "float32"), ramp)
    # mirrored ramp: |w_min| > |w_max| -> edge = w_min, scale positive
    wq, s, b = O.affine_quantize(-ramp - 1, gs, bits, "float32")
    assert np.all(s > 0) and np.all(b == -(nb + 1))
    assert np.array_equal(O.affine_dequantize(wq, s, b, gs, bits, "float32"), -ramp - 1)


@pytest.mark.parametrize("impl", ["numpy", "c"])
@pytest.mark.parametrize("gs", [32, 64])
@pytest.mark.parametrize("case", QK.CASES, ids=[c["name"] for c in QK.CASES])
def test_quantize_hand_worked_known_answers(case, gs, impl):
    """Known answers worked out by hand from MLX's published CPU loop (`quantize<T, U>`,
    mlx/backend/cpu/quantized.cpp, reached from KVCache.swift:1069-1070); the expected
    codes, words and parameter bits are literals of tests/quantizer_kats.py, not outputs of
    a restatement.  Each case separates the algorithm from one plausible misreading
    (T-rounded scale for the codes, round-half-away, no 1e-7 floor, a non-strict
    magnitude comparison).  With group size 64 the 32 values are repeated, which leaves
    the extrema and so every expected value unchanged."""
    q = O if impl == "numpy" else CO
    reps = gs // 32
    row = np.asarray(QK.group_values(case) * reps, np.float32)
    assert np.array_equal(O.round_to(row, case["dtype"]), row), "case values must be exact in the dtype"
    # two groups per row, the second one all zeros, so that group boundaries are exercised
    w = np.concatenate([row, np.zeros(gs, np.float32)])[None]
    wq, s, b = q.affine_quantize(w, gs, case["bits"], case["dtype"])
    words = QK.packed_words(case) * reps
    assert [int(x) for x in wq[0, :len(words)]] == words, case["wrong"]
    assert [int(x) for x in O.unpack_codes(wq, case["bits"])[0, :32]] == QK.group_codes(case)
    assert int(O.to_bits(s, case["dtype"])[0, 0]) == case["scale_bits"], case["wrong"]
    assert int(O.to_bits(b, case["dtype"])[0, 0]) == case["bias_bits"], case["wrong"]
    # the all-zero neighbour: codes 0, scale T(-1e-7), bias 0.  float32(1e-7) = 0x33D6BF95:
    # float16 -> 1.68 * 2^-24 -> 2 * 2^-24; bfloat16 -> the low half 0xBF95 rounds 0x33D6 up
    assert not wq[0, len(words):].any()
    assert int(O.to_bits(s, case["dtype"])[0, 1]) == {"float16": 0x8002, "bfloat16": 0xB3D7}[case["dtype"]]
    assert int(O.to_bits(b, case["dtype"])[0, 1]) == 0


@pytest.mark.parametrize("bits,bytes_per_group", [(8, 68), (4, 36)])
def test_compression_matches_reference_documentation(bits, bytes_per_group):
    # kv-cache-quantization.md:109-110: 64 fp16 values (128 B) -> 68 B / 36 B
    wq, s, b = O.affine_quantize(np.ones((1, 64), np.float32), 64, bits, "float16")
    assert wq.size * 4 + s.size * 2 + b.size * 2 == bytes_per_group


@pytest.mark.parametrize("bits", [2, 3, 4, 5, 6, 8])
def test_quantize_invariants(bits):
    rng = np.random.default_rng(7)
    w = O.round_to(rng.standard_normal((64, 128)).astype(np.float32) * 3, "float16")
    wq, s, b = O.affine_quantize(w, 64, bits, "float32")
    codes = O.unpack_codes(wq, bits)
    assert codes.max() <= (1 << bits) - 1
    deq = O.affine_dequantize(wq, s, b, 64, bits, "float32")
    g = w.reshape(64, 2, 64)
    err = np.abs(deq - w).reshape(64, 2, 64).max(-1)
    # half a step, plus whatever the re-anchored grid (scale = edge / q0) no longer
    # covers at the far end of the group's range
    nb = (1 << bits) - 1
    uncovered = np.maximum(0, (g.max(-1) - g.min(-1)) - nb * np.abs(s))
    assert np.all(err <= (np.abs(s) * 0.5 + uncovered) * (1 + 1e-5) + 1e-6)
    # little-endian nibble order: element k of a word sits at bits [k*bits, (k+1)*bits)
    if 32 % bits == 0:
        per = 32 // bits
        assert codes[3, per + 1] == (wq[3, 1] >> bits) & ((1 << bits) - 1)
    # the extreme element |edge| reproduces exactly (bias == edge, code 0)
    edge = np.where(np.abs(g.min(-1)) > np.abs(g.max(-1)), g.min(-1), g.max(-1))
    assert np.array_equal(b, edge)


@pytest.mark.parametrize("bits,codes,packed", [
    # 3 bits, 8 codes in 3 bytes: 1 + 2*8 + 3*64 + 4*512 + 5*4096 + 6*32768 + 7*262144 + 0 = 0x1F58D1
    (3, [1, 2, 3, 4, 5, 6, 7, 0], [0xD1, 0x58, 0x1F]),
    # 6 bits, 4 codes in 3 bytes: 1 + 2*64 + 3*4096 + 63*262144 = 0xFC3081
    (6, [1, 2, 3, 63], [0x81, 0x30, 0xFC]),
    # 5 bits, 8 codes in 5 bytes: 1 + 2*2^5 + 3*2^10 + 4*2^15 + 5*2^20 + 6*2^25 + 7*2^30 + 31*2^35 = 0xF9CC520C41
    (5, [1, 2, 3, 4, 5, 6, 7, 31], [0x41, 0x0C, 0x52, 0xCC, 0xF9]),
])
def test_odd_width_packing_known_bytes(bits, codes, packed):
    """MLX packs 3-, 5- and 6-bit codes 8 / 8 / 4 at a time, low code first, into 3 / 5 / 3 bytes
    (`quantize<T, U>`, mlx/backend/cpu/quantized.cpp, reached from KVCache.swift:1069-1070); the
    expected bytes are worked out by hand above, not taken from a restatement."""
    n = 32 * len(codes)  # whole uint32 words
    row = np.asarray(codes * 32, np.uint32)
    wq = O.pack_codes(row[None], bits)
    assert wq.dtype == np.uint32 and wq.shape == (1, n * bits // 32)
    stream = wq.astype("<u4").view(np.uint8)[0]
    assert [int(x) for x in stream[:len(packed)]] == packed
    assert [int(x) for x in stream] == packed * 32
    assert np.array_equal(O.unpack_codes(wq, bits)[0], row)
    # through the quantizer: integers 0 .. nb with both ends present -> code(x) = nb - x exactly
    nb = (1 << bits) - 1
    group = [nb - c for c in codes] * (32 // len(codes))
    group[0], group[1] = nb, 0  # both extremes in every group whatever the codes above are
    w = np.asarray(group * len(codes), np.float32)[None]
    q, s, b = O.affine_quantize(w, 32, bits, "float32")
    assert np.array_equal(O.unpack_codes(q, bits)[0], (nb - w[0]).astype(np.uint32))


# ---------------------------------------------------------------- attention
@pytest.mark.parametrize("r", [1, 2])
def test_quantized_attention_close_to_full_precision(r):
    # KVCacheTests.swift:1185-1217: 8-bit g64 causal, rtol .05 / atol .1
    rng = np.random.default_rng(0)
    B, Hkv, L, D = 1, 2, 4, 64
    scale = 1.0 / np.sqrt(D)
    q = rng.standard_normal((B, Hkv * r, L, D)).astype(np.float32)
    k = rng.standard_normal((B, Hkv, L, D)).astype(np.float32)
    v = rng.standard_normal((B, Hkv, L, D)).astype(np.float32)
    ref = O.sdpa(q, k, v, scale, O.Mask.CAUSAL, "float32")
    c = O.QuantizedKVCache(64, 8, "float32")
    qk, qv = c.update_quantized(k, v)
    out = O.quantized_sdpa(q, qk, qv, scale, O.Mask.CAUSAL, c.group_size, c.bits, "float32")
    assert out.shape == ref.shape
    assert np.allclose(out, ref, rtol=0.05, atol=0.1)
    # scalar C restatement agrees with the numpy one
    out_c = CO.qsdpa(q, qk, qv, scale, "causal", 64, 8, "float32")
    assert np.allclose(out_c, out, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "float32"])
def test_quantized_attention_finite_with_causal_fill(dtype):
    # KVCacheTests.swift:1219-1242 (finfo.min fill must not produce NaN)
    rng = np.random.default_rng(0)
    q, k, v = (O.round_to(rng.standard_normal((1, 2, 4, 64)).astype(np.float32), dtype) for _ in range(3))
    c = O.QuantizedKVCache(64, 8, dtype)
    qk, qv = c.update_quantized(k, v)
    out = O.quantized_sdpa(q, qk, qv, 0.125, O.Mask.CAUSAL, 64, 8, dtype)
    assert np.isfinite(out).all()
    assert np.array_equal(out, O.round_to(out, dtype))
    # first query row attends to key 0 only -> equals dequantised V row 0
    v0 = O.affine_dequantize(qv[0], qv[1], qv[2], 64, 8, "float32")[:, :, 0]
    assert np.allclose(out[:, :, 0], v0, atol=2e-2)


def test_sdpa_numpy_vs_c_with_masks():
    rng = np.random.default_rng(3)
    B, Hq, Hkv, L, T, D = 2, 4, 2, 3, 37, 32
    q = rng.standard_normal((B, Hq, L, D)).astype(np.float32)
    k = rng.standard_normal((B, Hkv, T, D)).astype(np.float32)
    v = rng.standard_normal((B, Hkv, T, D)).astype(np.float32)
    for mask_np, mask_c in [
        (O.Mask.NONE, None), (O.Mask.CAUSAL, "causal"),
        (O.Mask("array", O.create_causal_mask(L, T - L, 8)), O.create_causal_mask(L, T - L, 8)),
        (O.Mask("array", O.create_causal_mask(L, T - L, None, [30, 37])),
         O.create_causal_mask(L, T - L, None, [30, 37])),
    ]:
        a = O.sdpa(q, k, v, 0.2, mask_np, "float32")
        b = CO.sdpa(q, k, v, 0.2, mask_c, "float32")
        assert np.allclose(a, b, rtol=1e-5, atol=1e-5)
    # textbook check: uniform keys -> output is the mean of V
    out = O.sdpa(q, np.zeros_like(k), v, 1.0, O.Mask.NONE, "float32")
    assert np.allclose(out[:, 0, 0], v[:, 0].mean(1), atol=1e-5)


def test_round_helpers_agree_with_c():
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(2000).astype(np.float32) * 10.0 ** rng.uniform(-9, 5, 2000).astype(np.float32),
                        np.array([0, -0.0, 65504, 65519.9, 65520, 1e-7, -1e-7, 5.9e-8, 2.9e-8, 3e-8, 6.1e-5], np.float32)])
    lib = CO.lib()
    for dt in ("float16", "bfloat16"):
        a = O.round_to(x, dt)
        b = np.array([lib.kvo_round(float(v), CO.DT[dt]) for v in x], np.float32)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), dt


# ---------------------------------------------------------------- attention against an independent implementation
# torch's CPU scaled_dot_product_attention shares no code with the oracle.  These cases fix what the
# closed forms above leave open: which query heads share a kv head (blocked: head h reads kv head
# h // r, KVCache.swift:2372-2384), the lower-right alignment of `.causal` when fewer queries than
# keys are given (:2396-2400), how a [B, 1, L, T] or [B, Hq, L, T] mask broadcasts over the
# (kv head, repeat) split (:2438-2440), and exclusion (bool) versus addition (other dtypes) (:2441-2445).
def _torch_sdpa(q, k, v, scale, bool_mask=None, add_mask=None):
    import torch
    import torch.nn.functional as F
    r = q.shape[1] // k.shape[1]
    tq, tk, tv = (torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)) for a in (q, k, v))
    tk, tv = tk.repeat_interleave(r, dim=1), tv.repeat_interleave(r, dim=1)
    m = None
    if bool_mask is not None:
        m = torch.from_numpy(np.ascontiguousarray(bool_mask))
    if add_mask is not None:
        m = torch.from_numpy(np.ascontiguousarray(add_mask, dtype=np.float32))
    return F.scaled_dot_product_attention(tq, tk, tv, attn_mask=m, scale=float(scale)).numpy()


def _attention_mask_cases(rng, B, Hq, L, T):
    lower_right = np.tril(np.ones((L, T), bool), k=T - L)
    ragged = rng.random((B, 1, L, T)) < 0.7
    ragged[..., 0] = True  # no empty row
    per_head = rng.random((B, Hq, L, T)) < 0.7
    per_head[..., T - 1] = True
    return [
        ("none", O.Mask.NONE, None, None),
        ("causal", O.Mask.CAUSAL, lower_right, None),
        ("causal as array", O.Mask("array", O.create_causal_mask(L, T - L)), lower_right, None),
        ("window array", O.Mask("array", O.create_causal_mask(L, T - L, 7)),
         lower_right & ~np.tril(np.ones((L, T), bool), k=T - L - 7), None),
        ("bool [B,1,L,T]", O.Mask("array", ragged), ragged, None),
        ("bool [B,Hq,L,T]", O.Mask("array", per_head), per_head, None),
        ("additive [B,1,L,T]", O.Mask("array", (rng.standard_normal((B, 1, L, T)) * 2).astype(np.float32)), None, "same"),
        ("additive [B,Hq,L,T]", O.Mask("array", (rng.standard_normal((B, Hq, L, T)) * 2).astype(np.float32)), None, "same"),
        ("additive [L,T]", O.Mask("array", (rng.standard_normal((L, T)) * 2).astype(np.float32)), None, "same"),
    ]


@pytest.mark.parametrize("r", [1, 4, 8])
def test_sdpa_matches_torch(r):
    rng = np.random.default_rng(10 + r)
    B, Hkv, L, T, D = 2, 2, 5, 37, 32
    Hq = Hkv * r
    q = rng.standard_normal((B, Hq, L, D)).astype(np.float32)
    k = rng.standard_normal((B, Hkv, T, D)).astype(np.float32)
    v = rng.standard_normal((B, Hkv, T, D)).astype(np.float32)
    for name, mask, bm, am in _attention_mask_cases(rng, B, Hq, L, T):
        want = _torch_sdpa(q, k, v, 0.2, bm, mask.array if am else None)
        got = O.sdpa(q, k, v, 0.2, mask, "float32")
        assert np.abs(got - want).max() < 5e-6, (name, np.abs(got - want).max())
        if name in ("none", "causal") or (mask.array is not None and mask.array.dtype == np.bool_):
            got_c = CO.sdpa(q, k, v, 0.2, None if name == "none" else ("causal" if name == "causal" else mask.array), "float32")
            assert np.abs(got_c - want).max() < 5e-6, ("C", name)
    # single query over many keys (decode): row T-1 of the lower-right mask sees everything
    want = _torch_sdpa(q[:, :, -1:], k, v, 0.2)
    assert np.abs(O.sdpa(q[:, :, -1:], k, v, 0.2, O.Mask.CAUSAL, "float32") - want).max() < 5e-6


@pytest.mark.parametrize("bits,gs", [(4, 32), (8, 64)])
@pytest.mark.parametrize("r", [1, 4, 8])
def test_quantized_sdpa_matches_torch_on_dequantized_cache(r, bits, gs):
    rng = np.random.default_rng(100 * bits + r)
    B, Hkv, L, T, D = 2, 2, 5, 37, 64
    Hq = Hkv * r
    q = rng.standard_normal((B, Hq, L, D)).astype(np.float32)
    k = rng.standard_normal((B, Hkv, T, D)).astype(np.float32)
    v = rng.standard_normal((B, Hkv, T, D)).astype(np.float32)
    qk = O.affine_quantize(k, gs, bits, "float32")
    qv = O.affine_quantize(v, gs, bits, "float32")
    kd = O.affine_dequantize(*qk, gs, bits, "float32")
    vd = O.affine_dequantize(*qv, gs, bits, "float32")
    assert np.abs(kd - k).max() <= np.abs(qk[1]).max() * 2  # the dequantised cache is the cache, to about a code step
    for name, mask, bm, am in _attention_mask_cases(rng, B, Hq, L, T):
        want = _torch_sdpa(q, kd, vd, 0.125, bm, mask.array if am else None)
        if r > 1 and "[B,Hq,L,T]" in name:
            # the reference inserts one axis at -3 into a 4-D mask (KVCache.swift:2438-2440): [B, Hq, 1, L, T] does not
            # broadcast against scores [B, Hkv, r, L, T], so a mask per query head is an error there, and here
            with pytest.raises(ValueError):
                O.quantized_sdpa(q, qk, qv, 0.125, mask, gs, bits, "float32")
            continue
        got = O.quantized_sdpa(q, qk, qv, 0.125, mask, gs, bits, "float32")
        assert np.abs(got - want).max() < 1e-5, (name, np.abs(got - want).max())
        if am is None:
            got_c = CO.qsdpa(q, qk, qv, 0.125, None if name == "none" else ("causal" if name == "causal" else mask.array),
                             gs, bits, "float32")
            assert np.abs(got_c - want).max() < 1e-5, ("C", name)


@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_16_bit_attention_within_the_stated_tolerance_of_torch_float32(dtype):
    # the rounding points the oracle adds for a 16-bit T keep it inside max-abs 1e-2 / mean-abs 1e-3 of the
    # unrounded float32 result (bfloat16: inside two steps of the type at the largest output)
    rng = np.random.default_rng(5)
    B, Hkv, r, L, T, D = 2, 2, 4, 3, 200, 64
    q, k, v = (O.round_to(rng.standard_normal(s).astype(np.float32), dtype)
               for s in ((B, Hkv * r, L, D), (B, Hkv, T, D), (B, Hkv, T, D)))
    lower_right = np.tril(np.ones((L, T), bool), k=T - L)
    want = _torch_sdpa(q, k, v, 0.125, lower_right)
    got = O.sdpa(q, k, v, 0.125, O.Mask.CAUSAL, dtype)
    step = 2.0 ** -10 if dtype == "float16" else 2.0 ** -7
    assert np.abs(got - want).max() <= max(1e-2, 2 * step * np.abs(want).max()) and np.abs(got - want).mean() <= 1e-3
    qk, qv = O.affine_quantize(k, 64, 8, dtype), O.affine_quantize(v, 64, 8, dtype)
    want = _torch_sdpa(q, O.affine_dequantize(*qk, 64, 8, "float32"), O.affine_dequantize(*qv, 64, 8, "float32"), 0.125, lower_right)
    got = O.quantized_sdpa(q, qk, qv, 0.125, O.Mask.CAUSAL, 64, 8, dtype)
    assert np.abs(got - want).max() <= max(1e-2, 2 * step * np.abs(want).max()) and np.abs(got - want).mean() <= 1e-3


def test_softmax_matches_torch():
    import torch
    rng = np.random.default_rng(6)
    x = (rng.standard_normal((3, 5, 129)) * 6).astype(np.float32)
    x[0, 0, :40] = O.finfo_min("float16")   # masked scores as `maskFill` leaves them
    want = torch.softmax(torch.from_numpy(x), -1).numpy()
    assert np.abs(O.softmax_last(x, "float32") - want).max() < 1e-6
    assert np.allclose(O.softmax_last(x, "float32").sum(-1), 1.0, atol=1e-5)
    got16 = O.softmax_last(x, "float16")
    assert np.abs(got16 - want).max() <= 2.0 ** -11   # half a float16 step below 1


def test_round_to_matches_torch_casts():
    import torch
    rng = np.random.default_rng(7)
    x = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * 10.0 ** rng.uniform(-9, 5, 20000).astype(np.float32),
        np.array([0, -0.0, 65504, 65519.9, 65520, 1e-7, -1e-7, 5.9e-8, 2.9e-8, 3e-8, 6.1e-5, 1 + 2.0 ** -8, 1 + 3 * 2.0 ** -8,
                  1 + 2.0 ** -11, 1 + 3 * 2.0 ** -11, 3.3895e38, 3.4e38, 1e-40, -1e-40], np.float32)])
    t = torch.from_numpy(x)
    for name, td in (("float16", torch.float16), ("bfloat16", torch.bfloat16)):
        want = t.to(td).to(torch.float32).numpy()
        got = O.round_to(x, name)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), name
        bits_want = t.to(td).view(torch.int16).numpy().view(np.uint16)
        assert np.array_equal(O.to_bits(got, name), bits_want), name
        assert np.array_equal(O.from_bits(bits_want, name).view(np.uint32), want.view(np.uint32)), name
