"""float32 caches (AttentionUtils.swift:86-93 with float32 arrays, as most of KVCacheTests.swift builds them): the
vector-ALU kernel against the oracle and against a float64 evaluation at the reference test's own tolerance
(KVCacheTests.swift:1489, rtol = atol = 1e-5), and against the plain kernel over drawn shapes and masks.  Every
call is checked to have run on the float32 kernel (family 5), through the allocation-free entry point too."""
import numpy as np
import pytest
import torch

import kvhip
from oracle import kv_oracle as O
from tests.util import exact_attention, np32, presented_f64, randn

pytestmark = pytest.mark.gpu
F32 = torch.float32


def family():
    return kvhip.load().kvhip_last_attend_kernel()


def close(out, ref64, what):
    got = np32(out).astype(np.float64)
    assert np.isfinite(got).all(), what
    assert np.allclose(got, ref64, rtol=1e-5, atol=1e-5), f"{what}: max-abs {np.abs(got - ref64).max():.3e}"


@pytest.mark.parametrize("Dk,Dv,r", [(64, 64, 4), (128, 128, 1), (128, 128, 8), (72, 72, 4), (100, 120, 2), (256, 256, 2), (320, 192, 2),
                                      (6, 6, 1), (512, 256, 1), (30, 70, 3), (192, 128, 16)])
def test_simple_cache_against_the_oracle(Dk, Dv, r):
    rng = np.random.default_rng(Dk + Dv + r)
    B, Hkv = 2, 2
    scale = Dk ** -0.5
    c, o = kvhip.KVCacheSimple(), O.KVCacheSimple("float32")
    for Lq, mode in [(70, "causal"), (1, "none"), (3, "causal"), (1, "none"), (200, "array"), (1, "none"), (5, "additive"), (300, "causal")]:
        k, kd = randn(rng, (B, Hkv, Lq, Dk), F32)
        v, vd = randn(rng, (B, Hkv, Lq, Dv), F32)
        q, qd = randn(rng, (B, Hkv * r, Lq, Dk), F32)
        if mode == "array":
            mask, om = c.make_mask(Lq, 64, True), o.make_mask(Lq, 64, True)
        elif mode == "additive":
            T = o.offset + Lq
            add = np.where(rng.random((B, 1, Lq, T)) < 0.6, rng.standard_normal((B, 1, Lq, T)), -np.inf).astype(np.float32)
            add[..., 0] = 0.25  # no row without a key
            mask, om = kvhip.MaskMode.from_array(torch.from_numpy(add).cuda()), O.Mask("array", add)
        else:
            mask = kvhip.MaskMode.causal() if mode == "causal" else kvhip.MaskMode.none()
            om = O.Mask.CAUSAL if mode == "causal" else O.Mask.NONE
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
        assert tuple(out.shape) == (B, Hkv * r, Lq, Dv) and out.dtype == F32 and family() == 5
        ref = O.attention_with_cache_update(q, k, v, o, scale, om, "float32")
        close(out, ref.astype(np.float64), f"L={Lq} {mode} vs oracle")
        close(out, exact_attention(q, *presented_f64(o), scale, om), f"L={Lq} {mode} vs float64")
    # the allocation-free entry point takes the same kernel and gives the same bits
    q, qd = randn(rng, (B, Hkv * r, 2, Dk), F32)
    want = c.attend(qd, scale, kvhip.MaskMode.causal())
    got = torch.full_like(want, float("nan"))
    c.attend(qd, scale, kvhip.MaskMode.causal(), out=got, static_scratch=True)
    assert family() == 5 and torch.equal(got, want)


def test_long_sequence_is_divided_into_key_ranges_and_merged():
    rng = np.random.default_rng(5)
    B, Hkv, r, D, T = 1, 2, 4, 128, 5000
    c, o = kvhip.KVCacheSimple(), O.KVCacheSimple("float32")
    k, kd = randn(rng, (B, Hkv, T, D), F32)
    v, vd = randn(rng, (B, Hkv, T, D), F32)
    c.update(kd, vd, fetch=False)
    o.update(k, v)
    for Lq, mask, om in [(1, kvhip.MaskMode.none(), O.Mask.NONE), (4, kvhip.MaskMode.causal(), O.Mask.CAUSAL),
                         (9, kvhip.MaskMode.causal(), O.Mask.CAUSAL)]:
        q, qd = randn(rng, (B, Hkv * r, Lq, D), F32, 2.0)
        out = c.attend(qd, D ** -0.5, mask)
        assert family() == 5
        close(out, exact_attention(q, *presented_f64(o), D ** -0.5, om), f"L={Lq}")
    # a row that sees no key at all gives zeros, as the fused op's excluded keys contribute nothing
    q, qd = randn(rng, (B, Hkv * r, 3, D), F32)
    lens = torch.tensor([0], dtype=torch.int32)
    out = c.attend(qd, D ** -0.5, kvhip.MaskMode.window_mask(T - 3, 0, lengths=lens))
    lib = kvhip.load()
    try:
        lib.kvhip_set_kernel_policy(1)
        plain = c.attend(qd, D ** -0.5, kvhip.MaskMode.window_mask(T - 3, 0, lengths=lens))
    finally:
        lib.kvhip_set_kernel_policy(0)
    assert torch.equal(out, plain) and float(out.abs().max()) == 0.0


def test_rotating_cache_wraps():
    # KVCacheTests.swift:1451-1491: after the ring wraps, attention equals that over the last `window` keys
    rng = np.random.default_rng(11)
    B, Hkv, r, D, M = 2, 2, 2, 64, 96
    scale = D ** -0.5
    c, o = kvhip.RotatingKVCache(M, keep=4), O.RotatingKVCache(M, keep=4, dtype="float32")
    for i, Lq in enumerate([40, 1, 1, 70, 1, 1, 1, 30, 1, 1]):
        k, kd = randn(rng, (B, Hkv, Lq, D), F32)
        v, vd = randn(rng, (B, Hkv, Lq, D), F32)
        q, qd = randn(rng, (B, Hkv * r, Lq, D), F32)
        mask, om = c.make_mask(Lq, M), o.make_mask(Lq, M)
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
        assert family() == 5
        ref = O.attention_with_cache_update(q, k, v, o, scale, om, "float32")
        close(out, ref.astype(np.float64), f"step {i} L={Lq}")
    assert c.offset == o.offset and c.idx == o.idx


@pytest.mark.parametrize("seed", range(60))
def test_against_the_plain_kernel(seed):
    rng = np.random.default_rng(7000 + seed)
    kind = rng.choice(["simple", "rotating"])
    Dk = int(rng.choice([8, 64, 80, 128, 200, 256, 384]))
    Dv = Dk if rng.random() < 0.6 else int(rng.choice([16, 64, 100, 128, 256]))
    Dv = min(Dv, 256)
    if kind == "rotating":
        Dv = Dk = min(Dk, 256)
    B, Hkv, r = int(rng.integers(1, 5)), int(rng.choice([1, 2, 4])), int(rng.choice([1, 2, 4, 8]))
    Lq = int(rng.choice([1, 1, 2, 4, 7, 9, 33, 70]))
    T0 = int(rng.choice([1, 63, 64, 65, 200, 257, 700, 1500, 2600]))
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)

    def rand(*shape):
        return torch.randn(*shape, generator=g, device="cuda")

    c = kvhip.KVCacheSimple() if kind == "simple" else kvhip.RotatingKVCache(int(rng.choice([96, 300, 1024])), keep=int(rng.choice([0, 4])))
    c.update(rand(B, Hkv, T0, Dk), rand(B, Hkv, T0, Dv), fetch=False)
    for _ in range(int(rng.integers(0, 40)) if kind == "rotating" else 0):  # walk (and wrap) the ring
        c.update(rand(B, Hkv, 1, Dk), rand(B, Hkv, 1, Dv), fetch=False)
    c.update(rand(B, Hkv, Lq, Dk), rand(B, Hkv, Lq, Dv), fetch=False)
    T = c.presented_length
    Lq = min(Lq, T)
    q = rand(B, Hkv * r, Lq, Dk)
    which = rng.choice(["none", "causal", "window", "lengths", "left_pad", "bool", "additive"])
    if which == "none":
        mask = kvhip.MaskMode.none()
    elif which == "causal":
        mask = kvhip.MaskMode.causal()
    elif which == "window":
        mask = kvhip.MaskMode.window_mask(T - Lq, int(rng.integers(1, T + 2)))
    elif which == "lengths":
        mask = kvhip.MaskMode.window_mask(T - Lq, 0, lengths=torch.from_numpy(rng.integers(0, T + 1, size=B).astype(np.int32)))
    elif which == "left_pad":
        pad = torch.from_numpy(rng.integers(0, max(T - Lq, 1), size=B).astype(np.int32))
        mask = kvhip.MaskMode.window_mask(T - Lq, int(rng.choice([0, 50])), left_pad=pad)
    else:
        shape = [(B, 1, Lq, T), (1, 1, Lq, T), (B, Hkv * r, Lq, T)][rng.integers(3)]
        keep = rng.random(shape) < 0.7
        if which == "bool":
            mask = kvhip.MaskMode.from_array(torch.from_numpy(keep).cuda())
        else:
            add = np.where(keep, rng.standard_normal(shape).astype(np.float32), -np.inf)
            mask = kvhip.MaskMode.from_array(torch.from_numpy(add).cuda())
    scale = float(rng.choice([Dk ** -0.5, 0.05, -0.1]))
    print(f"seed {seed}: {kind} Dk{Dk} Dv{Dv} B{B} Hkv{Hkv} r{r} L{Lq} T{T} mask {which} scale {scale:.3f}", flush=True)
    lib = kvhip.load()
    try:
        lib.kvhip_set_kernel_policy(1)
        ref = np32(c.attend(q, scale, mask)).astype(np.float64)
        assert lib.kvhip_last_attend_kernel() == 0
        lib.kvhip_set_kernel_policy(0)
        out = c.attend(q, scale, mask)
        assert lib.kvhip_last_attend_kernel() == 5
    finally:
        lib.kvhip_set_kernel_policy(0)
    close(out, ref, "against the plain kernel")


@pytest.mark.parametrize("bits,gs,Dk,Dv", [(8, 64, 64, 64), (4, 64, 128, 128), (4, 32, 96, 96), (3, 64, 128, 128), (6, 64, 64, 128), (2, 128, 256, 256), (5, 32, 32, 32)])
def test_quantized_cache_with_float32_scales(bits, gs, Dk, Dv):
    """A quantized cache built from float32 arrays (as KVCacheTests.swift builds them) keeps float32 scales and biases;
    the matrix-core kernels take 16-bit ones.  Every call dequantizes it into scratch pages of float32 and runs the
    vector-ALU kernel over them (family 6); against the oracle's quantized sequence, with a batch row that is all
    padding and boolean rows of zeros, and the state untouched."""
    from tests.util import check_attention
    rng = np.random.default_rng(bits + Dk + gs)
    B, Hkv, r = 2, 2, 4
    scale = Dk ** -0.5
    c, o = kvhip.QuantizedKVCache(gs, bits), O.QuantizedKVCache(gs, bits, "float32")
    for Lq, mode in [(70, "causal"), (1, "none"), (3, "causal"), (1, "none"), (130, "lengths"), (1, "none"), (40, "bool"), (200, "causal")]:
        k, kd = randn(rng, (B, Hkv, Lq, Dk), F32)
        v, vd = randn(rng, (B, Hkv, Lq, Dv), F32)
        q, qd = randn(rng, (B, Hkv * r, Lq, Dk), F32)
        T = o.offset + Lq
        j = np.arange(T)[None, None, None, :]
        causal = np.broadcast_to(O.create_causal_mask(Lq, T - Lq)[None, None], (B, 1, Lq, T))
        if mode == "lengths":
            lengths = np.array([0, T - 20], np.int32)
            m = causal & (j < lengths[:, None, None, None])
            mask, om = kvhip.MaskMode.window_mask(T - Lq, 0, lengths=torch.from_numpy(lengths)), O.Mask("array", m)
        elif mode == "bool":
            m = causal & (rng.random((B, 1, Lq, T)) < 0.8)
            m[..., 0] = True
            m[0, 0, 3:9] = False
            mask, om = kvhip.MaskMode.from_array(torch.from_numpy(m).cuda()), O.Mask("array", m)
        else:
            mask = kvhip.MaskMode.causal() if mode == "causal" else kvhip.MaskMode.none()
            om = O.Mask.CAUSAL if mode == "causal" else O.Mask.NONE
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
        assert tuple(out.shape) == (B, Hkv * r, Lq, Dv) and out.dtype == F32 and family() == 6, (Lq, mode)
        ref = O.attention_with_cache_update(q, k, v, o, scale, om, "float32")
        close(out, ref.astype(np.float64), f"L={Lq} {mode}")
    for i, (a, b) in enumerate(zip(c.state, o.get_state())):
        assert np.array_equal(np32(a), b.astype(np.float32) if i % 3 else b), i
