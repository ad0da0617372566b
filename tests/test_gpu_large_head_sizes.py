"""16-bit caches of head sizes above 256 (Gemma 4's full-attention layers use 512: Gemma4Text.swift:53, :243-245), which
the matrix-core kernels are not built for: the vector-ALU kernel (family 5) against the oracle, through the
allocation-free entry point, and against the plain kernel over drawn shapes and masks."""
import numpy as np
import pytest
import torch

import kvhip
from oracle import kv_oracle as O
from tests.util import NAME, check_attention, exact_attention, np32, presented_f64, randn

pytestmark = pytest.mark.gpu


def family():
    return kvhip.load().kvhip_last_attend_kernel()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("Dk,Dv,r", [(512, 512, 4), (512, 512, 1), (320, 320, 2), (576, 512, 8), (320, 64, 4), (264, 300, 3), (1024, 128, 2)])
def test_simple_cache_against_the_oracle(dtype, Dk, Dv, r):
    rng = np.random.default_rng(Dk + Dv + r)
    name = NAME[dtype]
    B, Hkv = 2, 2
    scale = Dk ** -0.5
    c, o = kvhip.KVCacheSimple(), O.KVCacheSimple(name)
    for Lq, mode in [(70, "causal"), (1, "none"), (3, "causal"), (1, "none"), (200, "array"), (1, "none"), (300, "causal")]:
        k, kd = randn(rng, (B, Hkv, Lq, Dk), dtype)
        v, vd = randn(rng, (B, Hkv, Lq, Dv), dtype)
        q, qd = randn(rng, (B, Hkv * r, Lq, Dk), dtype)
        if mode == "array":
            mask, om = c.make_mask(Lq, 64, True), o.make_mask(Lq, 64, True)
        else:
            mask = kvhip.MaskMode.causal() if mode == "causal" else kvhip.MaskMode.none()
            om = O.Mask.CAUSAL if mode == "causal" else O.Mask.NONE
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
        assert tuple(out.shape) == (B, Hkv * r, Lq, Dv) and out.dtype == dtype and family() == 5
        ref = O.attention_with_cache_update(q, k, v, o, scale, om, name)
        check_attention(out, ref, dtype, f"L={Lq} {mode}", lambda: exact_attention(q, *presented_f64(o), scale, om))
    q, qd = randn(rng, (B, Hkv * r, 2, Dk), dtype)
    want = c.attend(qd, scale, kvhip.MaskMode.causal())
    got = torch.full_like(want, float("nan"))
    c.attend(qd, scale, kvhip.MaskMode.causal(), out=got, static_scratch=True)
    assert family() == 5 and torch.equal(got, want)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_long_sequence_and_ring_at_head_size_512(dtype):
    rng = np.random.default_rng(512)
    name = NAME[dtype]
    B, Hkv, r, D, T = 1, 2, 4, 512, 5000
    scale = D ** -0.5
    c, o = kvhip.KVCacheSimple(), O.KVCacheSimple(name)
    k, kd = randn(rng, (B, Hkv, T, D), dtype)
    v, vd = randn(rng, (B, Hkv, T, D), dtype)
    c.update(kd, vd, fetch=False)
    o.update(k, v)
    for Lq, mask, om in [(1, kvhip.MaskMode.none(), O.Mask.NONE), (2, kvhip.MaskMode.causal(), O.Mask.CAUSAL), (9, kvhip.MaskMode.causal(), O.Mask.CAUSAL)]:
        q, qd = randn(rng, (B, Hkv * r, Lq, D), dtype, 2.0)
        out = c.attend(qd, scale, mask)
        assert family() == 5
        ref = O.sdpa(q, *(x.astype(np.float32) for x in presented_f64(o)), scale, om, name)
        check_attention(out, ref, dtype, f"L={Lq}", lambda: exact_attention(q, *presented_f64(o), scale, om))
    M = 96
    c, o = kvhip.RotatingKVCache(M, keep=4), O.RotatingKVCache(M, keep=4, dtype=name)
    for i, Lq in enumerate([40, 1, 1, 70, 1, 1, 1, 30, 1, 1]):
        k, kd = randn(rng, (2, Hkv, Lq, D), dtype)
        v, vd = randn(rng, (2, Hkv, Lq, D), dtype)
        q, qd = randn(rng, (2, Hkv * r, Lq, D), dtype)
        mask, om = c.make_mask(Lq, M), o.make_mask(Lq, M)
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
        assert family() == 5
        ref = O.attention_with_cache_update(q, k, v, o, scale, om, name)
        check_attention(out, ref, dtype, f"ring step {i} L={Lq}", lambda: exact_attention(q, *presented_f64(o), scale, om))
    assert c.offset == o.offset and c.idx == o.idx


@pytest.mark.parametrize("seed", range(40))
def test_against_the_plain_kernel(seed):
    rng = np.random.default_rng(9000 + seed)
    dtype = [torch.float16, torch.bfloat16][seed % 2]
    kind = rng.choice(["simple", "rotating"])
    Dk = int(rng.choice([264, 320, 512, 576, 768]))
    Dv = Dk if rng.random() < 0.6 else int(rng.choice([64, 128, 300, 512]))
    Dv = min(Dv, 512)
    B, Hkv, r = int(rng.integers(1, 4)), int(rng.choice([1, 2])), int(rng.choice([1, 2, 4, 8]))
    Lq = int(rng.choice([1, 1, 2, 4, 7, 9, 33, 70]))
    T0 = int(rng.choice([1, 63, 64, 65, 200, 257, 700, 1500]))
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)

    def rand(*shape):
        return torch.randn(*shape, generator=g, device="cuda").to(dtype)

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
            mask = kvhip.MaskMode.from_array(torch.from_numpy(add).to(dtype).cuda())
    scale = float(rng.choice([Dk ** -0.5, 0.02, -0.03]))
    print(f"seed {seed}: {kind} {dtype} Dk{Dk} Dv{Dv} B{B} Hkv{Hkv} r{r} L{Lq} T{T} mask {which} scale {scale:.3f}", flush=True)
    lib = kvhip.load()
    try:
        lib.kvhip_set_kernel_policy(1)
        ref = np32(c.attend(q, scale, mask))
        assert lib.kvhip_last_attend_kernel() == 0
        lib.kvhip_set_kernel_policy(0)
        out = np32(c.attend(q, scale, mask))
        assert lib.kvhip_last_attend_kernel() == 5
    finally:
        lib.kvhip_set_kernel_policy(0)
    # both kernels compute in float32 and round once: they differ by the summation order, at most a unit of the
    # output type at the largest output
    assert np.isfinite(out).all()
    d = np.abs(out.astype(np.float64) - ref.astype(np.float64))
    ulp = max(float(np.abs(ref).max()), 1e-3) * (2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10)
    assert d.max() <= ulp and d.mean() <= ulp / 8, f"max-abs {d.max():.3e} mean-abs {d.mean():.3e} (unit {ulp:.3e})"


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bits,gs,Dk,Dv", [(4, 64, 512, 512), (8, 64, 512, 512), (4, 32, 320, 320), (3, 64, 512, 512), (6, 128, 384, 256)])
def test_quantized_cache_is_dequantized_for_the_vector_alu_kernel(dtype, bits, gs, Dk, Dv):
    """A quantized cache of such head sizes (Gemma 4 with kvBits): no quantized kernel takes it, so every call
    dequantizes it into scratch pages and runs the vector-ALU kernel over them (family 6); against the oracle's
    quantized sequence, a batch row that is all padding included, and the state untouched."""
    rng = np.random.default_rng(bits + Dk + gs)
    name = NAME[dtype]
    B, Hkv, r = 2, 2, 4
    scale = Dk ** -0.5
    c, o = kvhip.QuantizedKVCache(gs, bits), O.QuantizedKVCache(gs, bits, name)
    for Lq, mode in [(70, "causal"), (1, "none"), (3, "causal"), (1, "none"), (130, "lengths"), (1, "none"), (40, "bool")]:
        k, kd = randn(rng, (B, Hkv, Lq, Dk), dtype)
        v, vd = randn(rng, (B, Hkv, Lq, Dv), dtype)
        q, qd = randn(rng, (B, Hkv * r, Lq, Dk), dtype)
        T = o.offset + Lq
        j = np.arange(T)[None, None, None, :]
        causal = np.broadcast_to(O.create_causal_mask(Lq, T - Lq)[None, None], (B, 1, Lq, T))
        m = None
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
        assert tuple(out.shape) == (B, Hkv * r, Lq, Dv) and family() == 6, (Lq, mode)
        ref = O.attention_with_cache_update(q, k, v, o, scale, om, name)

        def exact():
            kk, vv = presented_f64(o)
            with np.errstate(invalid="ignore"):
                ex = exact_attention(q, kk, vv, scale, om)
            if m is not None:
                empty = ~np.broadcast_to(m, (B, Hkv * r, Lq, T)).any(axis=-1)
                ex[empty] = np.broadcast_to(np.repeat(vv, r, axis=1).mean(axis=2)[:, :, None, :], ex.shape)[empty]
            return ex
        check_attention(out, ref, dtype, f"L={Lq} {mode}", exact)
    for i, (a, b) in enumerate(zip(c.state, o.get_state())):
        assert np.array_equal(np32(a), b) if i % 3 == 0 else np.array_equal(np32(a), b.astype(np.float32)), i
