"""GPU parity of the rotary embedding in front of the cache write.

`kvhip_rope_apply` is held to one unit in the last place of a 16-bit array dtype against the
CPU restatement (angles are the same float32 values on both sides; the device rounds its
float32 products, the restatement works in float64: which intermediate roundings MLX's own
CPU path makes is parity unpinned).  The fused rotate-and-append must equal rotate-then-append
on the device bit for bit, for every cache kind, since both run the same element function.
"""
import numpy as np
import pytest
import torch

import kvhip
from oracle import kv_oracle as O
from oracle import rope as OR
from tests.util import NAME, dev, err_stats, np32, randn

pytestmark = pytest.mark.gpu

# float32 arrays: the device's three float32 roundings and its sincosf against float64, a few ulp
ULP = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7, torch.float32: 2.0 ** -19}


def within_one_ulp(got, want, dtype, pair_norm):
    """|got - want| <= one ulp of dtype at the magnitude of the rotated pair (an element of a
    pair may be tiny while its error scales with the pair)."""
    d = np.abs(got.astype(np.float64) - want.astype(np.float64))
    return bool((d <= ULP[dtype] * np.maximum(pair_norm, 1e-30) * 1.001 + 1e-30).all()), float(d.max())


def pair_norms(x, dims, traditional):
    n = np.abs(x).astype(np.float64).copy()
    half = dims // 2
    if traditional:
        m = np.maximum(np.abs(x[..., 0:dims:2]), np.abs(x[..., 1:dims:2]))
        n[..., 0:dims:2] = m
        n[..., 1:dims:2] = m
    else:
        m = np.maximum(np.abs(x[..., :half]), np.abs(x[..., half:dims]))
        n[..., :half] = m
        n[..., half:dims] = m
    return n * np.sqrt(2.0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("traditional", [False, True])
@pytest.mark.parametrize("D,dims,offset", [(128, 128, 0), (128, 128, 4097), (64, 32, 100000), (256, 256, 17)])
def test_rope_apply_matches_the_restatement(dtype, traditional, D, dims, offset):
    rng = np.random.default_rng(0)
    x32, xd = randn(rng, (2, 3, 5, D), dtype)
    rope = kvhip.RoPE(dims, traditional=traditional, base=500000.0, scale=1.0)
    got = np32(kvhip.apply_rotary_position(rope, xd, offset))
    want = OR.rope(x32, dims, traditional, 500000.0, 1.0, offset, dtype=NAME[dtype])
    ok, mx = within_one_ulp(got, want, dtype, pair_norms(x32, dims, traditional))
    assert ok, f"max diff {mx:.3e}"
    if offset == 0:
        assert np.array_equal(got[:, :, 0], x32[:, :, 0])   # position 0 is the identity
    assert np.array_equal(got[..., dims:], x32[..., dims:])


def test_rope_scale_freqs_and_batch_offsets():
    rng = np.random.default_rng(1)
    dtype = torch.float16
    x32, xd = randn(rng, (3, 2, 4, 64), dtype)
    freqs = (1.0 / OR.inv_freqs(64, 10000.0) * np.linspace(1.0, 8.0, 32)).astype(np.float32)
    rope = kvhip.RoPE(64, traditional=False, scale=0.5, freqs=freqs)
    offs = torch.tensor([0, 9, 1234], dtype=torch.int32)
    got = np32(kvhip.apply_rotary_position(rope, xd, offs))
    want = OR.rope(x32, 64, False, 10000.0, 0.5, offs.numpy(), freqs=freqs, dtype="float16")
    ok, mx = within_one_ulp(got, want, dtype, pair_norms(x32, 64, False))
    assert ok, f"max diff {mx:.3e}"
    # in place
    y = xd.clone()
    r, keep = rope.to_c()
    import ctypes as C
    from kvhip import _lib as L
    L.check(kvhip.load().kvhip_rope_apply(C.byref(r), C.c_void_p(y.data_ptr()), C.c_void_p(y.data_ptr()), 3, 2, 4, 64,
                                          L.F16, 0, C.c_void_p(offs.cuda().data_ptr()), None))
    torch.cuda.synchronize()
    assert np.array_equal(np32(y), got)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fused_append_equals_rotate_then_append_simple_and_ring(dtype):
    rng = np.random.default_rng(2)
    rope = kvhip.RoPE(64, traditional=False, base=10000.0)
    for make in (lambda: kvhip.KVCacheSimple(), lambda: kvhip.RotatingKVCache(24, keep=2)):
        fused, plain = make(), make()
        for Lq in (7, 1, 1, 9, 1, 12, 1):          # ring: multi-token writes, single-token writes, wraps
            _, k = randn(rng, (2, 2, Lq, 64), dtype)
            _, v = randn(rng, (2, 2, Lq, 64), dtype)
            off = plain.offset
            assert fused.rope_offset == off
            fused.update_rope(rope, k, v)
            plain.update(kvhip.apply_rotary_position(rope, k, off), v, fetch=False)
            assert fused.offset == plain.offset
            fk, fv = fused.fetch()
            pk, pv = plain.fetch()
            assert torch.equal(fk, pk) and torch.equal(fv, pv)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("traditional", [False, True])
@pytest.mark.parametrize("Dk,Dv,dims", [(128, 128, 128), (192, 128, 64)])
def test_fused_prompt_sized_append_equals_rotate_then_append(dtype, traditional, Dk, Dv, dims):
    """Whole-tile appends rotate inside the tile kernel."""
    rng = np.random.default_rng(7)
    rope = kvhip.RoPE(dims, traditional=traditional, base=500000.0)
    fused, plain = kvhip.KVCacheSimple(), kvhip.KVCacheSimple()
    for Lq in (5, 200, 130):
        _, k = randn(rng, (2, 2, Lq, Dk), dtype)
        _, v = randn(rng, (2, 2, Lq, Dv), dtype)
        off = plain.offset
        fused.update_rope(rope, k, v)
        plain.update(kvhip.apply_rotary_position(rope, k, off), v, fetch=False)
    fk, fv = fused.fetch()
    pk, pv = plain.fetch()
    assert torch.equal(fk, pk) and torch.equal(fv, pv)


@pytest.mark.parametrize("bits,gs,D,dims", [(4, 64, 128, 96), (8, 32, 128, 96), (4, 32, 96, 96), (8, 32, 96, 48),
                                            (4, 64, (192, 128), 64), (8, 32, (192, 128), 192)])
def test_fused_quantize_on_append_equals_rotate_then_append(bits, gs, D, dims):
    rng = np.random.default_rng(3)
    dtype = torch.float16
    Dk, Dv = D if isinstance(D, tuple) else (D, D)
    rope = kvhip.RoPE(dims, traditional=True, base=1e6)          # (partial rotation of a 128-wide head)
    fused, plain = kvhip.QuantizedKVCache(gs, bits), kvhip.QuantizedKVCache(gs, bits)
    for Lq in (70, 1, 1, 3, 190):
        _, k = randn(rng, (2, 2, Lq, Dk), dtype)
        _, v = randn(rng, (2, 2, Lq, Dv), dtype)
        off = plain.offset
        fused.update_rope(rope, k, v)
        plain.update_quantized(kvhip.apply_rotary_position(rope, k, off), v, fetch=False)
    for a, b in zip(fused.state, plain.state):
        assert torch.equal(a, b)
    # and the codes are what the restatement gives for the rotated keys (bit-exact quantizer)
    assert fused.offset == 265


def test_layer_sequence_against_the_restatement():
    """rope(q), rope(k) at the cache offset, append, attend -- the sequence of an attention
    layer -- against rope + sdpa of the restatement, prefill chunk then decode steps."""
    rng = np.random.default_rng(4)
    dtype = torch.float16
    B, Hq, Hkv, D = 2, 8, 2, 64
    rope = kvhip.RoPE(D, traditional=False, base=10000.0)
    cache = kvhip.KVCacheSimple()
    ks, vs = [], []
    for step, Lq in enumerate((33, 1, 1, 1)):
        q32, q = randn(rng, (B, Hq, Lq, D), dtype)
        k32, k = randn(rng, (B, Hkv, Lq, D), dtype)
        v32, v = randn(rng, (B, Hkv, Lq, D), dtype)
        off = cache.offset
        mask = kvhip.MaskMode.causal() if Lq > 1 else kvhip.MaskMode.none()
        out = kvhip.attention_with_rope_and_cache_update(rope, q, k, v, cache, D ** -0.5, mask)
        ks.append(OR.rope(k32, D, offset=off, dtype="float16"))
        vs.append(v32)
        ref = O.sdpa(OR.rope(q32, D, offset=off, dtype="float16"), np.concatenate(ks, 2), np.concatenate(vs, 2),
                     D ** -0.5, O.Mask.CAUSAL if Lq > 1 else O.Mask.NONE, "float16")
        mx, mean = err_stats(np32(out), ref)
        assert mx <= 1e-2 and mean <= 1e-3, f"step {step}: {mx:.3e} {mean:.3e}"
    assert cache.offset == 36


def test_staged_round_positions_count_the_staged_rows():
    rng = np.random.default_rng(5)
    dtype = torch.float16
    rope = kvhip.RoPE(64)
    live = kvhip.RotatingKVCache(16, keep=0)
    _, k0 = randn(rng, (1, 2, 10, 64), dtype)
    live.update_rope(rope, k0, k0)
    staged = kvhip.RotatingStagedKVCache(live)
    _, k1 = randn(rng, (1, 2, 2, 64), dtype)
    _, k2 = randn(rng, (1, 2, 1, 64), dtype)
    assert staged.rope_offset == 10
    staged.update_rope(rope, k1, k1)
    assert staged.rope_offset == 12
    staged.update_rope(rope, k2, k2)
    sk, _ = staged.staged_arrays
    want = torch.cat([kvhip.apply_rotary_position(rope, k1, 10), kvhip.apply_rotary_position(rope, k2, 12)], 2)
    assert torch.equal(sk, want)
    staged.commit(3)
    assert live.offset == 13


def test_rope_argument_errors():
    _, x = randn(np.random.default_rng(6), (1, 1, 1, 64), torch.float16)
    for bad in (kvhip.RoPE(63), kvhip.RoPE(66), kvhip.RoPE(0), kvhip.RoPE(64, base=0.0)):
        with pytest.raises(kvhip.KVHipError):
            kvhip.apply_rotary_position(bad, x, 0)
    c = kvhip.KVCacheSimple()
    with pytest.raises(kvhip.KVHipError):
        c.update_rope(kvhip.RoPE(130), x, x)
    assert c.offset == 0
