"""Head sizes the tuned kernels are not built for (the reference accepts any: AttentionUtils.swift:86-93,
KVCache.swift:2387-2419).  A 16-bit cache stores such rows zero-padded to the next head size the kernels take --
zero key columns add nothing to a score, zero value columns give output columns that are dropped -- and the arrays
that cross the C ABI keep the caller's sizes: queries, outputs, fetched rows and exported state are compared with the
oracle at the caller's head sizes, state bit for bit, and every attention call is checked to have run on a tuned
kernel (family 1, 2 or 3), not on the plain one."""
import numpy as np
import pytest
import torch

import kvhip
from kvhip import _lib as L
from oracle import kv_oracle as O
from tests.util import NAME, bits_equal, check_attention, exact_attention, np32, presented_f64, randn

pytestmark = pytest.mark.gpu


def family():
    return kvhip.load().kvhip_last_attend_kernel()


def state_equal(c, o, dtype):
    for i, (a, b) in enumerate(zip(c.state, o.get_state())):
        assert tuple(a.shape) == tuple(b.shape), (i, tuple(a.shape), tuple(b.shape))
        if a.dtype == torch.int32 or a.dtype == torch.uint32:
            assert np.array_equal(np32(a), b), i
        else:
            assert bits_equal(a, b, dtype), i


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("Dk,Dv,r", [(72, 72, 4), (112, 112, 2), (160, 160, 1), (192, 192, 2), (96, 64, 4), (64, 32, 1), (40, 40, 8),
                                      (100, 120, 2)])
def test_simple_cache_of_other_head_sizes(dtype, Dk, Dv, r):
    rng = np.random.default_rng(Dk + Dv + r)
    name = NAME[dtype]
    B, Hkv = 2, 2
    scale = Dk ** -0.5
    c, o = kvhip.KVCacheSimple(), O.KVCacheSimple(name)
    for Lq, mode in [(70, "causal"), (1, "none"), (3, "causal"), (1, "none"), (200, "array"), (1, "none")]:
        k, kd = randn(rng, (B, Hkv, Lq, Dk), dtype)
        v, vd = randn(rng, (B, Hkv, Lq, Dv), dtype)
        q, qd = randn(rng, (B, Hkv * r, Lq, Dk), dtype)
        if mode == "array":
            mask, om = c.make_mask(Lq, 64, True), o.make_mask(Lq, 64, True)
        else:
            mask = kvhip.MaskMode.causal() if mode == "causal" else kvhip.MaskMode.none()
            om = O.Mask.CAUSAL if mode == "causal" else O.Mask.NONE
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
        assert tuple(out.shape) == (B, Hkv * r, Lq, Dv) and family() in (2, 3)
        ref = O.attention_with_cache_update(q, k, v, o, scale, om, name)
        check_attention(out, ref, dtype, f"L={Lq} {mode}", lambda: exact_attention(q, *presented_f64(o), scale, om))
    assert c.offset == o.offset
    state_equal(c, o, dtype)
    # the state setter of a fresh cache, then trim and copy
    fresh = kvhip.KVCacheSimple()
    fresh.state = c.state
    assert fresh.offset == c.offset
    q, qd = randn(rng, (B, Hkv * r, 1, Dk), dtype)
    assert torch.equal(fresh.attend(qd, scale, kvhip.MaskMode.none()), c.attend(qd, scale, kvhip.MaskMode.none()))
    assert c.trim(5) == o.trim(5)
    state_equal(c, o, dtype)
    state_equal(c.copy(), o.copy(), dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_rotating_cache_of_head_size_112_wraps_and_stages(dtype):
    rng = np.random.default_rng(112)
    name = NAME[dtype]
    B, Hkv, r, D, M = 2, 2, 2, 112, 96
    scale = D ** -0.5
    c, o = kvhip.RotatingKVCache(M, keep=4), O.RotatingKVCache(M, keep=4, dtype=name)
    for i, Lq in enumerate([40, 1, 1, 70, 1, 1, 1, 30, 1]):
        k, kd = randn(rng, (B, Hkv, Lq, D), dtype)
        v, vd = randn(rng, (B, Hkv, Lq, D), dtype)
        q, qd = randn(rng, (B, Hkv * r, Lq, D), dtype)
        mask, om = c.make_mask(Lq, M, False), o.make_mask(Lq, M, False)
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
        assert family() in (2, 3)
        ref = O.attention_with_cache_update(q, k, v, o, scale, om, name)
        check_attention(out, ref, dtype, f"step {i}", lambda: exact_attention(q, *presented_f64(o), scale, om))
        assert c.meta_state == o.get_meta_state()
    state_equal(c, o, dtype)
    # the rows `update` hands back, in presented order
    k, kd = randn(rng, (B, Hkv, 1, D), dtype)
    ks, vs = c.update(kd, kd)
    ko, vo = o.update(k, k)
    assert tuple(ks.shape) == ko.shape and bits_equal(ks, ko, dtype) and bits_equal(vs, vo, dtype)


@pytest.mark.parametrize("dtype,bits,gs,D", [(torch.float16, 4, 32, 160), (torch.bfloat16, 8, 64, 192), (torch.float16, 4, 32, 32),
                                             (torch.float16, 3, 32, 224), (torch.bfloat16, 6, 64, 192)])
def test_quantized_cache_of_other_head_sizes(dtype, bits, gs, D):
    rng = np.random.default_rng(bits + gs + D)
    name = NAME[dtype]
    B, Hkv, r = 2, 2, 4
    scale = D ** -0.5
    c, o = kvhip.QuantizedKVCache(gs, bits), O.QuantizedKVCache(gs, bits, name)
    for Lq, mode in [(150, "causal"), (1, "none"), (70, "causal"), (1, "none"), (4, "causal"), (1, "none")]:
        k, kd = randn(rng, (B, Hkv, Lq, D), dtype)
        v, vd = randn(rng, (B, Hkv, Lq, D), dtype)
        q, qd = randn(rng, (B, Hkv * r, Lq, D), dtype)
        mask, om = (kvhip.MaskMode.causal(), O.Mask.CAUSAL) if mode == "causal" else (kvhip.MaskMode.none(), O.Mask.NONE)
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
        assert tuple(out.shape) == (B, Hkv * r, Lq, D) and family() in (1, 3)
        ref = O.attention_with_cache_update(q, k, v, o, scale, om, name)
        check_attention(out, ref, dtype, f"L={Lq}", lambda: exact_attention(q, *presented_f64(o), scale, om))
    assert c.group_size == gs and c.offset == o.offset
    state_equal(c, o, dtype)
    # the six arrays into a fresh cache; then trim, back to full precision, copy
    fresh = kvhip.QuantizedKVCache(gs, bits)
    fresh.state = c.state
    fresh.meta_state = c.meta_state
    state_equal(fresh, o, dtype)
    q, qd = randn(rng, (B, Hkv * r, 1, D), dtype)
    assert torch.equal(fresh.attend(qd, scale, kvhip.MaskMode.none()), c.attend(qd, scale, kvhip.MaskMode.none()))
    assert c.trim(3) == o.trim(3)
    state_equal(c, o, dtype)
    state_equal(c.to_unquantized(), o.to_unquantized(), dtype)
    state_equal(c.copy(), o.copy(), dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_simple_cache_of_head_size_160_converts_to_quantized(dtype):
    rng = np.random.default_rng(160)
    name = NAME[dtype]
    c, o = kvhip.KVCacheSimple(), O.KVCacheSimple(name)
    for Lq in (130, 1, 70):
        k, kd = randn(rng, (2, 3, Lq, 160), dtype, 2.0)
        v, vd = randn(rng, (2, 3, Lq, 160), dtype, 0.5)
        c.update(kd, vd, fetch=False)
        o.update(k, v)
    for bits in (4, 8, 5):
        qc, qo = c.to_quantized(32, bits), o.to_quantized(32, bits)
        assert qc.meta_state == qo.get_meta_state()
        state_equal(qc, qo, dtype)
    # group size 64 does not divide 160: the reference's resolution falls back to 32 (KVCache.swift:1020-1037)
    assert c.to_quantized(64, 4).group_size == o.to_quantized(64, 4).group_size == 32


def test_allocation_free_entry_on_a_padded_cache():
    rng = np.random.default_rng(7)
    dtype, D = torch.float16, 112
    c = kvhip.KVCacheSimple()
    k, kd = randn(rng, (2, 2, 700, D), dtype)
    c.update(kd, kd.flip(-1).contiguous(), fetch=False)
    for Lq in (1, 40):
        q, qd = randn(rng, (2, 8, Lq, D), dtype)
        mask = kvhip.MaskMode.causal() if Lq > 1 else kvhip.MaskMode.none()
        want = c.attend(qd, D ** -0.5, mask)
        fam = family()
        got = torch.full_like(want, float("nan"))
        c.attend(qd, D ** -0.5, mask, out=got, static_scratch=True)
        assert family() == fam and fam in (2, 3) and torch.equal(got, want)


def test_float32_and_head_sizes_above_256_run_on_the_vector_alu_kernel():
    rng = np.random.default_rng(9)
    for dtype, D in ((torch.float32, 72), (torch.float16, 320)):
        c, o = kvhip.KVCacheSimple(), O.KVCacheSimple(NAME[dtype])
        k, kd = randn(rng, (1, 2, 50, D), dtype)
        q, qd = randn(rng, (1, 4, 50, D), dtype)
        out = kvhip.attention_with_cache_update(qd, kd, kd, c, D ** -0.5, kvhip.MaskMode.causal())
        assert family() == 5
        ref = O.attention_with_cache_update(q, k, k, o, D ** -0.5, O.Mask.CAUSAL, NAME[dtype])
        check_attention(out, ref, dtype, f"D={D}", lambda: exact_attention(q, *presented_f64(o), D ** -0.5, O.Mask.CAUSAL))
