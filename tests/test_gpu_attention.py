"""GPU parity tests of attention over the device caches against the CPU oracle.

Tolerance (BASELINE north star): max-abs <= 1e-2 and mean-abs <= 1e-3 against
the oracle's restatement of the reference path.  Every case runs twice: with the
library's default kernel choice and with the generic kernel forced, so the
matrix-core kernels are checked against both the oracle and the generic kernel.
"""
import numpy as np
import pytest
import torch

import kvhip
from kvhip import _lib as L
from oracle import c_oracle as CO
from oracle import kv_oracle as O
from tests.util import NAME, bits_equal, check_attention, dev, err_stats, exact_attention, np32, presented_f64, randn

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS = 1e-2, 1e-3


@pytest.fixture(params=[0, 1], ids=["auto", "generic"])
def policy(request):
    kvhip.load().kvhip_set_kernel_policy(request.param)
    yield request.param
    kvhip.load().kvhip_set_kernel_policy(0)


def check(out, ref, what="", exact=None):
    """max-abs <= 1e-2 and mean-abs <= 1e-3 against the oracle; outside that only with a float64 evaluation of
    the same attention that shows the device as close to the exact result as the oracle (tests/util.py)."""
    check_attention(out, ref, out.dtype, what, exact)


def omask(mask, dtype):
    """kvhip MaskMode -> oracle Mask"""
    if mask is None or mask.mode == L.MASK_NONE:
        return O.Mask.NONE
    if mask.mode == L.MASK_CAUSAL:
        return O.Mask.CAUSAL
    a = mask.array
    return O.Mask("array", a.cpu().numpy() if a.dtype == torch.bool else np32(a))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("bits,gs,D", [(8, 64, 64), (4, 64, 128), (4, 32, 64), (2, 64, 128), (4, 64, 256), (8, 128, 256),
                                        (8, 32, 128), (4, 32, 96), (8, 32, 96), (3, 64, 128), (5, 32, 96), (6, 64, 64)])
@pytest.mark.parametrize("r", [1, 4])
def test_quantized_attention_modes(policy, dtype, bits, gs, D, r):
    rng = np.random.default_rng(bits + D + r)
    B, Hkv, T0, Lq = 2, 2, 83, 4
    name = NAME[dtype]
    c = kvhip.QuantizedKVCache(gs, bits)
    o = O.QuantizedKVCache(gs, bits, name)
    k, kd = randn(rng, (B, Hkv, T0, D), dtype)
    v, vd = randn(rng, (B, Hkv, T0, D), dtype)
    c.update_quantized(kd, vd, fetch=False)
    o.update_quantized(k, v)
    scale = 1.0 / np.sqrt(D)
    # multi-token step with .causal, then an array mask, then single-token .none
    k, kd = randn(rng, (B, Hkv, Lq, D), dtype)
    v, vd = randn(rng, (B, Hkv, Lq, D), dtype)
    q, qd = randn(rng, (B, Hkv * r, Lq, D), dtype)
    out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, kvhip.MaskMode.causal())
    ref = O.attention_with_cache_update(q, k, v, o, scale, O.Mask.CAUSAL, name)
    check(out, ref, "causal")
    T = c.offset
    m = torch.from_numpy(O.create_causal_mask(Lq, T - Lq, 16)).cuda()
    out = c.attend(qd, scale, kvhip.MaskMode.from_array(m))
    ref = O.quantized_sdpa(q, *o.get_quantized_state(), scale, O.Mask("array", m.cpu().numpy()), gs if D % gs == 0 else 32, bits, name)
    check(out, ref, "bool array")
    lens = torch.tensor([T - 7, T], dtype=torch.int32)
    mb = torch.from_numpy(O.create_causal_mask(Lq, T - Lq, None, lens.numpy())).cuda()  # [B,1,L,T]
    out = c.attend(qd, scale, kvhip.MaskMode.from_array(mb))
    ref = O.quantized_sdpa(q, *o.get_quantized_state(), scale, O.Mask("array", mb.cpu().numpy()), o.group_size, bits, name)
    check(out, ref, "batched bool array")
    # per-head masks only line up in the reference without GQA (KVCache.swift:2436-2440)
    add = O.round_to(rng.standard_normal((B, Hkv if r == 1 else 1, Lq, T)).astype(np.float32), name)
    out = c.attend(qd, scale, kvhip.MaskMode.from_array(dev(add, dtype)))
    ref = O.quantized_sdpa(q, *o.get_quantized_state(), scale, O.Mask("array", add), o.group_size, bits, name)
    check(out, ref, "additive array")
    # the symbolic window mask equals the materialised createCausalMask
    outw = c.attend(qd, scale, kvhip.MaskMode.window_mask(T - Lq, 16))
    refw = O.quantized_sdpa(q, *o.get_quantized_state(), scale, O.Mask("array", O.create_causal_mask(Lq, T - Lq, 16)), o.group_size, bits, name)
    check(outw, refw, "window")
    k, kd = randn(rng, (B, Hkv, 1, D), dtype)
    v, vd = randn(rng, (B, Hkv, 1, D), dtype)
    q, qd = randn(rng, (B, Hkv * r, 1, D), dtype)
    out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale)
    ref = O.attention_with_cache_update(q, k, v, o, scale, O.Mask.NONE, name)
    assert out.dtype == dtype  # KVCacheTests.swift:1219-1242
    check(out, ref, "decode")


@pytest.mark.parametrize("bits,D,gs", [(4, 128, 64), (8, 64, 64), (4, 128, 32), (8, 128, 32), (4, 64, 32), (4, 96, 32), (8, 96, 32)])
@pytest.mark.parametrize("B,Hkv,T0", [(32, 8, 777), (64, 8, 300), (32, 8, 70)])
def test_quantized_decode_many_pairs(bits, D, gs, B, Hkv, T0):
    """Many (batch, kv-head) pairs, the shape of the headline workload scaled down in length:
    with 256 pairs two spans per pair fold into one workgroup of 8 wavefronts that writes the
    output itself, with 512 pairs a single span of 4 does; both skip the partial-merge
    kernel.  One token (no mask), two and four tokens (causal: 8 and 16 query rows per kv head, the 16-row
    kernel, which also takes every row count of head size 96) per step, against the oracle."""
    rng = np.random.default_rng(B + T0 + bits)
    dtype, name = torch.float16, "float16"
    r = 4
    c = kvhip.QuantizedKVCache(gs, bits)
    o = O.QuantizedKVCache(gs, bits, name)
    k, kd = randn(rng, (B, Hkv, T0, D), dtype)
    v, vd = randn(rng, (B, Hkv, T0, D), dtype)
    c.update_quantized(kd, vd, fetch=False)
    o.update_quantized(k, v)
    scale = 1.0 / np.sqrt(D)
    for Lq, mask, om in ((1, None, O.Mask.NONE), (2, kvhip.MaskMode.causal(), O.Mask.CAUSAL), (4, kvhip.MaskMode.causal(), O.Mask.CAUSAL)):
        k, kd = randn(rng, (B, Hkv, Lq, D), dtype)
        v, vd = randn(rng, (B, Hkv, Lq, D), dtype)
        q, qd = randn(rng, (B, Hkv * r, Lq, D), dtype)
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
        assert kvhip.load().kvhip_last_attend_kernel() == 1
        ref = O.attention_with_cache_update(q, k, v, o, scale, om, name)
        check(out, ref, f"L={Lq}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bits,gs", [(4, 64), (8, 64), (4, 128), (8, 128)])
@pytest.mark.parametrize("B,Hkv,r,T0", [(16, 8, 2, 777), (32, 8, 4, 300), (3, 2, 1, 2100)])
def test_quantized_decode_head_size_256(dtype, bits, gs, B, Hkv, r, T0):
    """Head size 256 (four or two groups per row) on the matrix-core decode kernels: one token
    without a mask, as many tokens as still make four query rows per kv head under .causal (the 4-row
    kernel), then four tokens (up to 16 rows: the 16-row kernel)."""
    rng = np.random.default_rng(B + T0 + bits + gs)
    name, D = NAME[dtype], 256
    c = kvhip.QuantizedKVCache(gs, bits)
    o = O.QuantizedKVCache(gs, bits, name)
    k, kd = randn(rng, (B, Hkv, T0, D), dtype)
    v, vd = randn(rng, (B, Hkv, T0, D), dtype)
    c.update_quantized(kd, vd, fetch=False)
    o.update_quantized(k, v)
    scale = 1.0 / np.sqrt(D)
    for Lq, mask, om in ((1, None, O.Mask.NONE), (4 // r, kvhip.MaskMode.causal(), O.Mask.CAUSAL),
                         (4, kvhip.MaskMode.causal(), O.Mask.CAUSAL), (3, kvhip.MaskMode.causal(), O.Mask.CAUSAL)):
        k, kd = randn(rng, (B, Hkv, Lq, D), dtype)
        v, vd = randn(rng, (B, Hkv, Lq, D), dtype)
        q, qd = randn(rng, (B, Hkv * r, Lq, D), dtype)
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
        assert kvhip.load().kvhip_last_attend_kernel() == 1
        ref = O.attention_with_cache_update(q, k, v, o, scale, om, name)
        check(out, ref, f"L={Lq}")


@pytest.mark.parametrize("r", [1, 2])
def test_quantized_causal_close_to_full_precision(policy, r):
    # KVCacheTests.swift:1185-1217: 8-bit g64 causal vs fp SDPA, rtol .05 / atol .1
    rng = np.random.default_rng(0)
    B, Hkv, Lq, D = 1, 2, 4, 64
    scale = 1.0 / np.sqrt(D)
    q, qd = randn(rng, (B, Hkv * r, Lq, D), torch.float32)
    k, kd = randn(rng, (B, Hkv, Lq, D), torch.float32)
    v, vd = randn(rng, (B, Hkv, Lq, D), torch.float32)
    c = kvhip.QuantizedKVCache(64, 8)
    out = np32(kvhip.attention_with_cache_update(qd, kd, vd, c, scale, kvhip.MaskMode.causal()))
    ref = O.sdpa(q, k, v, scale, O.Mask.CAUSAL, "float32")
    assert np.allclose(out, ref, rtol=0.05, atol=0.1)
    s = kvhip.KVCacheSimple()
    out_fp = np32(kvhip.attention_with_cache_update(qd, kd, vd, s, scale, kvhip.MaskMode.causal()))
    assert np.allclose(out_fp, ref, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("Dk,Dv,r", [(128, 128, 4), (64, 32, 1), (256, 256, 2), (80, 80, 2), (96, 96, 4), (96, 96, 1), (192, 128, 1), (192, 128, 4)])
def test_simple_cache_attention(policy, dtype, Dk, Dv, r):
    rng = np.random.default_rng(Dk + r)
    B, Hkv = 2, 2
    name = NAME[dtype]
    c = kvhip.KVCacheSimple()
    o = O.KVCacheSimple(name)
    scale = 1.0 / np.sqrt(Dk)
    for Lq, mode in [(70, "causal"), (1, "none"), (3, "causal"), (1, "none"), (260, "array"), (1, "none")]:
        k, kd = randn(rng, (B, Hkv, Lq, Dk), dtype)
        v, vd = randn(rng, (B, Hkv, Lq, Dv), dtype)
        q, qd = randn(rng, (B, Hkv * r, Lq, Dk), dtype)
        if mode == "array":
            mask = c.make_mask(Lq, 64, True)
            om = o.make_mask(Lq, 64, True)
            assert np.array_equal(mask.array.cpu().numpy(), om.array)
        else:
            mask = kvhip.MaskMode.causal() if mode == "causal" else kvhip.MaskMode.none()
            om = O.Mask.CAUSAL if mode == "causal" else O.Mask.NONE
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
        ref = O.attention_with_cache_update(q, k, v, o, scale, om, name)
        exact = lambda: exact_attention(q, *presented_f64(o), scale, om)
        check(out, ref, f"L={Lq} {mode}", exact)
        if mode == "array":
            # the same mask handed over as data (boolean, then additive), as unmodified model code does
            out = c.attend(qd, scale, kvhip.MaskMode.from_array(mask.array))
            check(out, ref, f"L={Lq} boolean array", exact)
            addm = torch.where(mask.array, 0.0, -30000.0).to(dtype if dtype != torch.float32 else torch.float32)
            out = c.attend(qd, scale, kvhip.MaskMode.from_array(addm))
            check(out, ref, f"L={Lq} additive array", exact)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_keys_of_192_values_of_128_on_the_prefill_tile(dtype):
    """The multi-head latent attention models cache keys of 192 (qk_nope 128 + qk_rope 64) and values of
    128 per head (DeepseekV3.swift:128-156, also DeepseekV2 / GLM4MOELite / MiMoV2Flash): prompt chunks,
    single-token steps over a key range long enough to be split into parts and merged, and a ring."""
    rng = np.random.default_rng(192)
    name, Dk, Dv = NAME[dtype], 192, 128
    scale = Dk ** -0.5
    lib = kvhip.load()
    B, H = 1, 2
    c, o = kvhip.KVCacheSimple(), O.KVCacheSimple(name)
    for Lq, mode in [(1100, "causal"), (1, "none"), (400, "causal"), (1, "none"), (5, "causal")]:
        k, kd = randn(rng, (B, H, Lq, Dk), dtype)
        v, vd = randn(rng, (B, H, Lq, Dv), dtype)
        q, qd = randn(rng, (B, H, Lq, Dk), dtype)
        mask, om = (kvhip.MaskMode.causal(), O.Mask.CAUSAL) if mode == "causal" else (kvhip.MaskMode.none(), O.Mask.NONE)
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
        assert lib.kvhip_last_attend_kernel() == 3 and tuple(out.shape) == (B, H, Lq, Dv)
        ref = O.attention_with_cache_update(q, k, v, o, scale, om, name)
        check(out, ref, f"simple L={Lq}", lambda: exact_attention(q, *presented_f64(o), scale, om))
    M = 256
    c, o = kvhip.RotatingKVCache(M, keep=4), O.RotatingKVCache(M, keep=4, dtype=name)
    for i, Lq in enumerate([64] * 7 + [1] * 6):
        k, kd = randn(rng, (2, H, Lq, Dk), dtype)
        v, vd = randn(rng, (2, H, Lq, Dv), dtype)
        q, qd = randn(rng, (2, 2 * H, Lq, Dk), dtype)
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, c.make_mask(Lq, M, False))
        assert lib.kvhip_last_attend_kernel() == 3
        om = o.make_mask(Lq, M, False)
        ref = O.attention_with_cache_update(q, k, v, o, scale, om, name)
        check(out, ref, f"ring step {i}", lambda: exact_attention(q, *presented_f64(o), scale, om))


@pytest.mark.parametrize("dtype,bits,gs", [(torch.float16, 4, 64), (torch.bfloat16, 8, 64), (torch.float16, 8, 32), (torch.bfloat16, 4, 32),
                                           (torch.float16, 3, 64), (torch.bfloat16, 5, 32), (torch.float16, 6, 32), (torch.bfloat16, 2, 64)])
def test_quantized_keys_of_192_values_of_128_on_the_prefill_tile(dtype, bits, gs):
    """The same head sizes in a QuantizedKVCache (group sizes 32 and 64 divide both): decode steps run on the 16-row
    decode kernel, everything else on the quantized prefill tile; codes and pairs equal the oracle's, outputs are the
    oracle's within the bound."""
    rng = np.random.default_rng(bits + gs)
    name, Dk, Dv = NAME[dtype], 192, 128
    scale = Dk ** -0.5
    lib = kvhip.load()
    B, H, r = 2, 2, 2
    c, o = kvhip.QuantizedKVCache(gs, bits), O.QuantizedKVCache(gs, bits, name)
    for Lq, mode in [(330, "causal"), (1, "none"), (70, "causal"), (1, "none"), (4, "causal")]:
        k, kd = randn(rng, (B, H, Lq, Dk), dtype)
        v, vd = randn(rng, (B, H, Lq, Dv), dtype)
        q, qd = randn(rng, (B, H * r, Lq, Dk), dtype)
        mask, om = (kvhip.MaskMode.causal(), O.Mask.CAUSAL) if mode == "causal" else (kvhip.MaskMode.none(), O.Mask.NONE)
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
        # up to 16 query rows per kv head: the 16-row decode kernel (other code widths than 4 / 8 bits: its instances
        # are built for group size 64); otherwise the prefill tile
        want = 1 if ((bits in (4, 8) or gs == 64) and r * Lq <= 16) else 3
        assert lib.kvhip_last_attend_kernel() == want and tuple(out.shape) == (B, H * r, Lq, Dv)
        ref = O.attention_with_cache_update(q, k, v, o, scale, om, name)
        check(out, ref, f"L={Lq}", lambda: exact_attention(q, *presented_f64(o), scale, om))
    assert c.group_size == gs and c.offset == o.offset
    for i, (a, b) in enumerate(zip(c.state, o.get_state())):
        assert np.array_equal(np32(a), b) if i % 3 == 0 else bits_equal(a, b, dtype), i


def test_rotating_attention_past_wrap_matches_never_rotated_reference(policy):
    # KVCacheTests.swift:1451-1491 (rtol = atol = 1e-5, float32)
    rng = np.random.default_rng(0)
    window, history, nq, heads, hd = 8, 20, 4, 2, 4
    scale = 1.0 / np.sqrt(hd)
    ak, akd = randn(rng, (1, heads, history + nq, hd), torch.float32)
    av, avd = randn(rng, (1, heads, history + nq, hd), torch.float32)
    q, qd = randn(rng, (1, heads, nq, hd), torch.float32)
    c = kvhip.RotatingKVCache(window)
    for p in range(history):
        c.update(akd[:, :, p:p + 1], avd[:, :, p:p + 1], fetch=False)
    mask = c.make_mask(nq, window, False)
    out = kvhip.attention_with_cache_update(qd, akd[:, :, history:], avd[:, :, history:], c, scale, mask)
    qp = np.arange(history, history + nq)[:, None]
    kp = np.arange(history + nq)[None, :]
    ref = O.sdpa(q, ak, av, scale, O.Mask("array", (qp >= kp) & (qp < kp + window)), "float32")
    assert np.allclose(np32(out), ref, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_rotating_cfg4_reduced(policy, dtype):
    """BASELINE config 4 scaled down (maxSize 512, keep 4, D 256, 64-token chunks):
    chunked prefill wraps the ring, windowed array masks, then single-token decode."""
    rng = np.random.default_rng(4)
    B, Hq, Hkv, D, M, chunk = 2, 4, 2, 256, 512, 64
    name = NAME[dtype]
    scale = 1.0 / np.sqrt(D)
    c = kvhip.RotatingKVCache(M, keep=4)
    o = O.RotatingKVCache(M, keep=4, dtype=name)
    for i in range(20):
        k, kd = randn(rng, (B, Hkv, chunk, D), dtype)
        v, vd = randn(rng, (B, Hkv, chunk, D), dtype)
        q, qd = randn(rng, (B, Hq, chunk, D), dtype)
        mask = c.make_mask(chunk, M, False)
        om = o.make_mask(chunk, M, False)
        # an array mask that is a function of the indices is handed to the kernels as such
        assert mask.mode in {"none": (L.MASK_NONE,), "causal": (L.MASK_CAUSAL,), "array": (L.MASK_ARRAY, L.MASK_WINDOW)}[om.mode]
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
        ref = O.attention_with_cache_update(q, k, v, o, scale, om, name)
        exact = lambda: exact_attention(q, *presented_f64(o), scale, om)
        if i in (0, 7, 8, 9, 19):
            check(out, ref, f"chunk {i}", exact)
        if i in (8, 19) and om.mode == "array":
            # ring rows in run order, the mask handed over as data
            out = c.attend(qd, scale, kvhip.MaskMode.from_array(mask.array))
            check(out, ref, f"chunk {i} boolean array", exact)
    for i in range(40):
        k, kd = randn(rng, (B, Hkv, 1, D), dtype)
        v, vd = randn(rng, (B, Hkv, 1, D), dtype)
        q, qd = randn(rng, (B, Hq, 1, D), dtype)
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, c.make_mask(1, M, False))
        om = o.make_mask(1, M, False)
        ref = O.attention_with_cache_update(q, k, v, o, scale, om, name)
        check(out, ref, f"decode {i}", lambda: exact_attention(q, *presented_f64(o), scale, om))
        assert kvhip.load().kvhip_last_attend_kernel() == (2 if policy == 0 else 0)  # MFMA fp decode
        assert c.meta_state == o.get_meta_state()


def test_cfg1_quantized_prefill_then_decode(policy):
    """BASELINE config 1 at full size: B1, 16q/4kv heads, D64, fp16, 8-bit g64; prefill
    512 with .causal, then 128 single-token appends each followed by quantized SDPA."""
    rng = np.random.default_rng(0)
    B, Hq, Hkv, D = 1, 16, 4, 64
    scale = 0.125
    dtype = torch.float16
    c = kvhip.QuantizedKVCache(64, 8)
    o = O.QuantizedKVCache(64, 8, "float16")
    q, qd = randn(rng, (B, Hq, 512, D), dtype)
    k, kd = randn(rng, (B, Hkv, 512, D), dtype)
    v, vd = randn(rng, (B, Hkv, 512, D), dtype)
    out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, c.make_mask(512))
    qk, qv = o.update_quantized(k, v)
    ref = CO.qsdpa(q, qk, qv, scale, "causal", 64, 8, "float16")
    check(out, ref, "prefill")
    # (the quantized MFMA prefill tile: a chunk this small is not worth a conversion pass of its own)
    assert kvhip.load().kvhip_last_attend_kernel() == (3 if policy == 0 else 0)
    # the same causal mask handed over as a boolean array
    tri = torch.ones(512, 512, dtype=torch.bool, device="cuda").tril()
    out = c.attend(qd, scale, kvhip.MaskMode.from_array(tri))
    check(out, ref, "prefill, boolean array")
    for step in range(128):
        q, qd = randn(rng, (B, Hq, 1, D), dtype)
        k, kd = randn(rng, (B, Hkv, 1, D), dtype)
        v, vd = randn(rng, (B, Hkv, 1, D), dtype)
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, c.make_mask(1))
        qk, qv = o.update_quantized(k, v)
        ref = CO.qsdpa(q, qk, qv, scale, None, 64, 8, "float16")
        check(out, ref, f"decode {step}")
    assert kvhip.load().kvhip_last_attend_kernel() == (1 if policy == 0 else 0)  # MFMA quantized decode
    assert c.offset == 640 and c.meta_state == ["256", "640", "64", "8"]
    for a, b in zip(c.state, o.get_state()):
        if a.dtype == torch.int32:
            assert np.array_equal(np32(a), b)
        else:
            assert np.array_equal(O.to_bits(np32(a), "float16"), O.to_bits(b, "float16"))


def test_cfg5_ragged_speculative_rollback_reduced(policy):
    """BASELINE config 5 scaled down: ragged left-padded batch, rounds of 4 draft tokens
    scored under causal AND left-padding masks, then trim(n)."""
    rng = np.random.default_rng(0)
    B, Hq, Hkv, D, Lq = 4, 8, 2, 128, 4
    dtype = torch.float16
    lens = rng.integers(40, 300, size=B)
    Tmax = int(lens.max())
    pad = (Tmax - lens).astype(np.int32)
    c = kvhip.QuantizedKVCache(64, 4)
    o = O.QuantizedKVCache(64, 4, "float16")
    k, kd = randn(rng, (B, Hkv, Tmax, D), dtype)
    v, vd = randn(rng, (B, Hkv, Tmax, D), dtype)
    c.update_quantized(kd, vd, fetch=False)
    o.update_quantized(k, v)
    scale = 1.0 / np.sqrt(D)
    trims = np.random.default_rng(1).integers(0, 5, size=12)
    for rnd in range(12):
        k, kd = randn(rng, (B, Hkv, Lq, D), dtype)
        v, vd = randn(rng, (B, Hkv, Lq, D), dtype)
        q, qd = randn(rng, (B, Hq, Lq, D), dtype)
        T = c.offset + Lq
        m = O.create_causal_mask(Lq, T - Lq)[None, None] & (np.arange(T)[None, None, None, :] >= pad[:, None, None, None])
        if rnd % 2 == 0:
            mask = kvhip.MaskMode.from_array(torch.from_numpy(m).cuda())
        else:
            mask = kvhip.MaskMode.window_mask(T - Lq, 0, left_pad=torch.from_numpy(pad))
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
        ref = O.attention_with_cache_update(q, k, v, o, scale, O.Mask("array", m), "float16")
        check(out, ref, f"round {rnd}")
        assert kvhip.load().kvhip_last_attend_kernel() == (1 if policy == 0 else 0)  # 16 query rows per kv head
        n = int(trims[rnd])
        assert c.trim(n) == o.trim(n) and c.offset == o.offset
    for a, b in zip(c.state, o.get_state()):
        if a.dtype == torch.int32:
            assert np.array_equal(np32(a), b)


@pytest.mark.parametrize("kind,Lq", [("q4", 1), ("q4", 4), ("q8", 2), ("fp16", 1), ("bf16", 2), ("q3", 1), ("q5", 4), ("q2", 2), ("q6", 1)])
def test_ragged_batch_spans(policy, kind, Lq):
    """Per-batch lengths and left padding far apart (1 .. 3000 rows visible): the decode kernels
    divide each row's own visible range over the spans; every row must come out as under the
    equivalent array mask (the oracle's)."""
    rng = np.random.default_rng(11 + Lq)
    B, Hq, Hkv, D = 7, 8, 2, 128
    dtype = torch.bfloat16 if kind == "bf16" else torch.float16
    name = NAME[dtype]
    T0 = 3000 - Lq
    if kind[0] == "q":
        bits = int(kind[1])
        c, o = kvhip.QuantizedKVCache(64, bits), O.QuantizedKVCache(64, bits, name)
    else:
        c, o = kvhip.KVCacheSimple(), O.KVCacheSimple(name)
    k, kd = randn(rng, (B, Hkv, T0, D), dtype)
    v, vd = randn(rng, (B, Hkv, T0, D), dtype)
    if kind[0] == "q":
        c.update_quantized(kd, vd, fetch=False)
        o.update_quantized(k, v)
    else:
        c.update(kd, vd, fetch=False)
        o.update(k, v)
    scale = 1.0 / np.sqrt(D)
    T = T0 + Lq
    j = np.arange(T)[None, None, None, :]
    causal = O.create_causal_mask(Lq, T - Lq)[None, None]
    cases = {
        "lengths": dict(lengths=np.array([T, 1, 1500, 64, T - 1, 65, 700], np.int32)),
        "left_pad": dict(left_pad=np.array([0, T - Lq - 1, 1500, T - 64 - Lq, 1, 2047, 2300], np.int32)),
        "both": dict(lengths=np.array([T, 900, 1500, T, 2100, 2500, T], np.int32),
                     left_pad=np.array([0, 800, 0, 2900, 100, 2400, 2990], np.int32)),
    }
    kn, knd = randn(rng, (B, Hkv, Lq, D), dtype)
    vn, vnd = randn(rng, (B, Hkv, Lq, D), dtype)
    q, qd = randn(rng, (B, Hq, Lq, D), dtype)
    first = True
    for what, kw in cases.items():
        m = np.broadcast_to(causal, (B, 1, Lq, T)).copy()
        if "lengths" in kw:
            m &= j < kw["lengths"][:, None, None, None]
        if "left_pad" in kw:
            m &= j >= kw["left_pad"][:, None, None, None]
        mask = kvhip.MaskMode.window_mask(T - Lq, 0, **{a: torch.from_numpy(b) for a, b in kw.items()})
        if first:
            out = kvhip.attention_with_cache_update(qd, knd, vnd, c, scale, mask)
            ref = O.attention_with_cache_update(q, kn, vn, o, scale, O.Mask("array", m), name)
            first = False
        else:
            out = c.attend(qd, scale, mask)
            if kind[0] == "q" and int(kind[1]) in (3, 5, 6):  # (the C oracle unpacks whole-word code widths only)
                ref = O.quantized_sdpa(q, *o.get_quantized_state(), scale, O.Mask("array", m), 64, int(kind[1]), name)
            elif kind[0] == "q":
                ref = CO.qsdpa(q, *o.get_quantized_state(), scale, m, 64, int(kind[1]), name)
            else:
                ref = CO.sdpa(q, o.keys[:, :, :T], o.values[:, :, :T], scale, m, name)
        check(out, ref, f"{kind} L={Lq} {what}")
        assert kvhip.load().kvhip_last_attend_kernel() == (0 if policy else (1 if kind[0] == "q" else 2))


def test_ring_in_temporal_order_with_lengths(policy):
    """A wrapped ring after a multi-token write is presented through a row map (temporal order);
    per-batch lengths over the presented rows must bound each row's keys there too."""
    rng = np.random.default_rng(5)
    B, Hq, Hkv, D, M, Lq = 4, 8, 4, 128, 1024, 2
    dtype, name = torch.float16, "float16"
    c, o = kvhip.RotatingKVCache(M, keep=4), O.RotatingKVCache(M, keep=4)
    k, kd = randn(rng, (B, Hkv, 700, D), dtype)
    c.update(kd, kd.flip(-1), fetch=False)
    o.update(k, k[..., ::-1].copy())
    for _ in range(400):  # single-token writes wrap the ring
        k, kd = randn(rng, (B, Hkv, 1, D), dtype)
        c.update(kd, kd.flip(-1), fetch=False)
        o.update(k, k[..., ::-1].copy())
    k, kd = randn(rng, (B, Hkv, Lq, D), dtype)
    c.update(kd, kd.flip(-1), fetch=False)
    ok, ov = o.update(k, k[..., ::-1].copy())
    T = ok.shape[2]
    assert c.presented_length == T and c.idx == o.idx
    q, qd = randn(rng, (B, Hq, Lq, D), dtype)
    lengths = np.array([T, T - 100, 300, 77], np.int32)
    m = O.create_causal_mask(Lq, T - Lq)[None, None] & (np.arange(T)[None, None, None, :] < lengths[:, None, None, None])
    out = c.attend(qd, 1.0 / np.sqrt(D), kvhip.MaskMode.window_mask(T - Lq, 0, lengths=torch.from_numpy(lengths)))
    ref = CO.sdpa(q, ok, ov, 1.0 / np.sqrt(D), m, name)
    check(out, ref, "ring, temporal order, lengths")


@pytest.mark.parametrize("dtype,bits,gs,D,B,Hq,Hkv", [
    (torch.float16, 4, 64, 128, 3, 8, 2), (torch.bfloat16, 4, 64, 128, 2, 4, 4), (torch.float16, 8, 64, 64, 1, 16, 4),
    (torch.float16, 4, 32, 128, 2, 8, 2), (torch.float16, 8, 128, 256, 1, 4, 2), (torch.bfloat16, 8, 32, 64, 2, 6, 2),
    (torch.float16, 4, 64, 256, 2, 8, 4),
    # the 16-row kernel: more than 4 query heads per kv head, head size 96, keys of 192 with values of 128, bit streams
    (torch.float16, 4, 64, 128, 2, 16, 2), (torch.bfloat16, 8, 64, 64, 1, 16, 1), (torch.bfloat16, 8, 32, 96, 2, 4, 2),
    (torch.float16, 4, 32, 96, 1, 8, 1), (torch.float16, 4, 64, (192, 128), 2, 4, 4), (torch.bfloat16, 8, 32, (192, 128), 1, 16, 2),
    (torch.float16, 3, 64, 128, 2, 8, 2), (torch.bfloat16, 5, 32, 128, 1, 4, 4), (torch.float16, 6, 64, 64, 2, 4, 2),
    (torch.float16, 2, 128, 128, 2, 16, 2), (torch.bfloat16, 3, 64, 256, 1, 4, 2), (torch.float16, 5, 32, 96, 2, 6, 2),
    (torch.bfloat16, 6, 64, (192, 128), 1, 8, 2), (torch.float16, 3, 32, 64, 2, 2, 2),
])
def test_single_token_steps_write_their_row_inside_the_decode_kernel(dtype, bits, gs, D, B, Hq, Hkv):
    """`attentionWithCacheUpdate` with one new token and no mask on a quantized cache is one launch: the decode
    kernel quantizes the new row into the cache itself.  Codes, scale / bias pairs and offsets must be the
    append kernel's (the oracle's) bit for bit after every step -- across octets, 64-token tiles, pages and
    trims -- and the outputs the oracle's within the bound."""
    D, Dv = D if isinstance(D, tuple) else (D, D)
    rng = np.random.default_rng(bits * 7 + D + gs)
    cache = kvhip.QuantizedKVCache(gs, bits)
    ocache = O.QuantizedKVCache(gs, bits, NAME[dtype])
    scale = D ** -0.5
    tol = 1e-2 if dtype == torch.float16 else 1.6e-2
    for start, steps, trim in [(1, 9, 0), (52, 14, 3), (250, 9, 0), (1500, 5, 2)]:
        n = start - ocache.offset
        if n > 0:
            k, kd = randn(rng, (B, Hkv, n, D), dtype, 1.5)
            v, vd = randn(rng, (B, Hkv, n, Dv), dtype, 0.7)
            cache.update_quantized(kd, vd, fetch=False)
            ocache.update_quantized(k, v)
        for _ in range(steps):
            q, qd = randn(rng, (B, Hq, 1, D), dtype)
            k, kd = randn(rng, (B, Hkv, 1, D), dtype, 1.5)
            v, vd = randn(rng, (B, Hkv, 1, Dv), dtype, 0.7)
            got = np32(cache.update_attend(qd, kd, vd, scale))
            assert kvhip.load().kvhip_last_attend_kernel() == 1
            ref = O.attention_with_cache_update(q, k, v, ocache, scale, O.Mask.NONE, NAME[dtype])
            mx, mean = err_stats(got, ref)
            assert mx <= tol and mean <= 1e-3, (ocache.offset, mx, mean)
            assert cache.offset == ocache.offset
        for i, (a, b) in enumerate(zip(cache.state, ocache.get_state())):
            assert np.array_equal(np32(a), b) if i % 3 == 0 else bits_equal(a, b, dtype), (start, i)
        assert cache.trim(trim) == ocache.trim(trim)


def stream_decode_shape(D, gs):
    """Head and group sizes the 16-row decode kernel has 2- / 3- / 5- / 6-bit instances for."""
    return (D == 64 and gs in (32, 64)) or (D == 96 and gs == 32) or D == 128 or (D == 256 and gs == 64)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bits,D,gs", [(2, 128, 64), (3, 128, 64), (5, 128, 32), (6, 128, 64), (3, 64, 32), (6, 64, 64), (2, 256, 64),
                                        (5, 256, 128), (3, 256, 32), (3, 96, 32), (6, 96, 32), (2, 96, 32), (5, 96, 32)])
def test_other_code_widths_on_the_pipelined_tile(dtype, bits, D, gs):
    """2-, 3-, 5- and 6-bit codes (KVCacheConfiguration.swift:124 lists them beside 4 and 8): prompt chunks run on the
    pipelined prefill tile, which cuts the codes out of the rows' bit streams; up to 16 query rows per kv head run on
    the 16-row decode kernel where it has an instance for the shape (`stream_decode_shape`), on the tile otherwise.
    Prompt chunks, single-token steps and a multi-token step against the oracle; codes and pairs bit for bit."""
    rng = np.random.default_rng(100 * bits + D + gs)
    name = NAME[dtype]
    B, Hkv, r = 2, 2, 4
    scale = D ** -0.5
    lib = kvhip.load()
    c, o = kvhip.QuantizedKVCache(gs, bits), O.QuantizedKVCache(gs, bits, name)
    for Lq, mode in [(200, "causal"), (1, "none"), (70, "causal"), (1, "none"), (4, "causal"), (1, "none")]:
        k, kd = randn(rng, (B, Hkv, Lq, D), dtype)
        v, vd = randn(rng, (B, Hkv, Lq, D), dtype)
        q, qd = randn(rng, (B, Hkv * r, Lq, D), dtype)
        mask, om = (kvhip.MaskMode.causal(), O.Mask.CAUSAL) if mode == "causal" else (kvhip.MaskMode.none(), O.Mask.NONE)
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
        assert lib.kvhip_last_attend_kernel() == (1 if r * Lq <= 16 and stream_decode_shape(D, gs) else 3)
        ref = O.attention_with_cache_update(q, k, v, o, scale, om, name)
        check(out, ref, f"L={Lq}", lambda: exact_attention(q, *presented_f64(o), scale, om))
    # a boolean array mask and a window evaluated from indices
    T = c.offset
    q, qd = randn(rng, (B, Hkv * r, 40, D), dtype)
    m = O.create_causal_mask(40, T - 40, 33)
    ref = O.quantized_sdpa(q, *o.get_quantized_state(), scale, O.Mask("array", m), o.group_size, bits, name)
    exact = lambda: exact_attention(q, *presented_f64(o), scale, O.Mask("array", m))
    check(c.attend(qd, scale, kvhip.MaskMode.from_array(torch.from_numpy(m).cuda())), ref, "bool array", exact)
    check(c.attend(qd, scale, kvhip.MaskMode.window_mask(T - 40, 33)), ref, "window", exact)
    assert lib.kvhip_last_attend_kernel() == 3
    for i, (a, b) in enumerate(zip(c.state, o.get_state())):
        assert np.array_equal(np32(a), b) if i % 3 == 0 else bits_equal(a, b, dtype), i


STREAM_DECODE_CASES = [(torch.float16, b, 128, g) for b in (2, 3, 5, 6) for g in (32, 64, 128)] + [
    (torch.bfloat16, 3, 128, 64), (torch.bfloat16, 6, 128, 32), (torch.bfloat16, 2, 128, 128), (torch.bfloat16, 5, 128, 64),
    (torch.float16, 3, 64, 32), (torch.bfloat16, 5, 64, 32), (torch.float16, 2, 64, 64), (torch.bfloat16, 6, 64, 64),
    (torch.float16, 2, 256, 64), (torch.bfloat16, 3, 256, 64), (torch.float16, 5, 256, 64), (torch.float16, 6, 256, 64),
    (torch.float16, 2, 96, 32), (torch.bfloat16, 3, 96, 32), (torch.float16, 5, 96, 32), (torch.bfloat16, 6, 96, 32),
    (torch.float16, 2, (192, 128), 64), (torch.float16, 3, (192, 128), 64), (torch.bfloat16, 5, (192, 128), 64), (torch.float16, 6, (192, 128), 64)]


@pytest.mark.parametrize("dtype,bits,D,gs", STREAM_DECODE_CASES)
def test_other_code_widths_on_the_16_row_decode_kernel(dtype, bits, D, gs):
    """Decode steps of 2-, 3-, 5- and 6-bit caches: a lane of the 16-row kernel cuts its segment of every group out
    of the row's bit stream (every segment width and alignment the head and group sizes give is a case here).  A
    cache long enough for several spans and the merge launch; 1, 3, 8, 13 and 16 query rows per kv head; no mask,
    causal, boolean and additive arrays, per-batch lengths and left padding -- against the oracle, and the kernel
    family asserted."""
    D, Dv = D if isinstance(D, tuple) else (D, D)  # (keys of 192 with values of 128)
    rng = np.random.default_rng(1000 * bits + D + gs)
    name = NAME[dtype]
    B, Hkv = 3, 2
    scale = D ** -0.5
    lib = kvhip.load()
    c, o = kvhip.QuantizedKVCache(gs, bits), O.QuantizedKVCache(gs, bits, name)
    T0 = 2900 + bits
    k, kd = randn(rng, (B, Hkv, T0, D), dtype)
    v, vd = randn(rng, (B, Hkv, T0, Dv), dtype)
    c.update_quantized(kd, vd, fetch=False)
    o.update_quantized(k, v)
    for r, Lq, mode in [(4, 1, "none"), (1, 1, "none"), (1, 3, "causal"), (4, 4, "causal"), (8, 1, "none"), (13, 1, "none"),
                        (2, 4, "bool"), (4, 2, "additive"), (4, 3, "lengths"), (2, 8, "left_pad"), (1, 16, "causal")]:
        k, kd = randn(rng, (B, Hkv, Lq, D), dtype)
        v, vd = randn(rng, (B, Hkv, Lq, Dv), dtype)
        q, qd = randn(rng, (B, Hkv * r, Lq, D), dtype)
        T = c.offset + Lq
        j = np.arange(T)[None, None, None, :]
        causal = np.broadcast_to(O.create_causal_mask(Lq, T - Lq)[None, None], (B, 1, Lq, T))
        if mode == "none":
            mask, om = kvhip.MaskMode.none(), O.Mask.NONE
        elif mode == "causal":
            mask, om = kvhip.MaskMode.causal(), O.Mask.CAUSAL
        elif mode == "bool":
            m = causal & (rng.random((B, 1, Lq, T)) < 0.8)
            m[..., 0] = True
            mask, om = kvhip.MaskMode.from_array(torch.from_numpy(m).cuda()), O.Mask("array", m)
        elif mode == "additive":
            add = np.where(causal, rng.standard_normal((B, 1, Lq, T)) * 0.5, -30000.0).astype(np.float32)
            add = O.round_to(add, name)
            mask = kvhip.MaskMode.from_array(torch.from_numpy(add).to(dtype).cuda())
            om = O.Mask("array", add)
        elif mode == "lengths":
            lengths = np.array([T, 70, 1500], np.int32)
            m = causal & (j < lengths[:, None, None, None])
            mask, om = kvhip.MaskMode.window_mask(T - Lq, 0, lengths=torch.from_numpy(lengths)), O.Mask("array", m)
        else:
            pad = np.array([0, T - Lq - 3, 1000], np.int32)
            m = causal & (j >= pad[:, None, None, None])
            mask, om = kvhip.MaskMode.window_mask(T - Lq, 0, left_pad=torch.from_numpy(pad)), O.Mask("array", m)
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
        assert lib.kvhip_last_attend_kernel() == 1 and tuple(out.shape) == (B, Hkv * r, Lq, Dv)
        ref = O.attention_with_cache_update(q, k, v, o, scale, om, name)
        check(out, ref, f"r={r} L={Lq} {mode}", lambda: exact_attention(q, *presented_f64(o), scale, om))
    for i, (a, b) in enumerate(zip(c.state, o.get_state())):
        assert np.array_equal(np32(a), b) if i % 3 == 0 else bits_equal(a, b, dtype), i


@pytest.mark.parametrize("dtype,bits,gs,D", [
    (torch.float16, 4, 64, 128), (torch.bfloat16, 4, 64, 128), (torch.float16, 8, 32, 64), (torch.bfloat16, 8, 64, 256),
    (torch.float16, 4, 32, 96), (torch.float16, 4, 64, (192, 128)), (torch.bfloat16, 8, 32, (192, 128)),
    (torch.float16, 2, 64, 128), (torch.bfloat16, 3, 32, 96), (torch.float16, 5, 128, 256), (torch.bfloat16, 6, 64, 64),
])
def test_quantized_prompt_chunks_dequantize_first(dtype, bits, gs, D):
    """A prompt chunk with many query rows per kv head over a quantized cache is not converted tile by tile: the
    cached rows are dequantized once into scratch pages (`MLX.dequantized`'s values) and the full-precision tile runs
    over them (kernel family 4).  Forced here on small chunks (policy 3) under every mask kind; against the oracle,
    and the cache's state untouched."""
    D, Dv = D if isinstance(D, tuple) else (D, D)
    rng = np.random.default_rng(31 * bits + D + gs)
    name = NAME[dtype]
    B, Hkv, r = 2, 2, 4
    scale = D ** -0.5
    lib = kvhip.load()
    c, o = kvhip.QuantizedKVCache(gs, bits), O.QuantizedKVCache(gs, bits, name)
    try:
        for Lq, mode, policy in [(150, "causal", 3), (70, "bool", 3), (40, "additive", 3), (33, "window", 3), (64, "lengths", 3),
                                 (300, "causal", 3), (20, "causal", 3)]:
            lib.kvhip_set_kernel_policy(policy)
            k, kd = randn(rng, (B, Hkv, Lq, D), dtype)
            v, vd = randn(rng, (B, Hkv, Lq, Dv), dtype)
            q, qd = randn(rng, (B, Hkv * r, Lq, D), dtype)
            T = c.offset + Lq
            j = np.arange(T)[None, None, None, :]
            causal = np.broadcast_to(O.create_causal_mask(Lq, T - Lq)[None, None], (B, 1, Lq, T))
            if mode == "causal":
                mask, om = kvhip.MaskMode.causal(), O.Mask.CAUSAL
            elif mode == "bool":
                m = causal & (rng.random((B, 1, Lq, T)) < 0.8)
                m[..., 0] = True
                mask, om = kvhip.MaskMode.from_array(torch.from_numpy(m).cuda()), O.Mask("array", m)
            elif mode == "additive":
                add = O.round_to(np.where(causal, rng.standard_normal((B, 1, Lq, T)) * 0.5, -30000.0).astype(np.float32), name)
                mask, om = kvhip.MaskMode.from_array(dev(add, dtype)), O.Mask("array", add)
            elif mode == "window":
                m = np.broadcast_to(O.create_causal_mask(Lq, T - Lq, 48)[None, None], (B, 1, Lq, T))
                mask, om = kvhip.MaskMode.window_mask(T - Lq, 48), O.Mask("array", m)
            else:
                lengths = np.array([T, T - 90], np.int32)
                m = causal & (j < lengths[:, None, None, None])
                mask, om = kvhip.MaskMode.window_mask(T - Lq, 0, lengths=torch.from_numpy(lengths)), O.Mask("array", m)
            out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
            assert lib.kvhip_last_attend_kernel() == 4 and tuple(out.shape) == (B, Hkv * r, Lq, Dv), (Lq, mode)
            ref = O.attention_with_cache_update(q, k, v, o, scale, om, name)
            check(out, ref, f"L={Lq} {mode}", lambda: exact_attention(q, *presented_f64(o), scale, om))
    finally:
        lib.kvhip_set_kernel_policy(0)
    for i, (a, b) in enumerate(zip(c.state, o.get_state())):
        assert np.array_equal(np32(a), b) if i % 3 == 0 else bits_equal(a, b, dtype), i


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("mode", ["lengths", "left_pad", "bool"])
def test_dequantize_first_gives_rows_without_keys_the_quantized_answer(dtype, mode):
    """A query row whose mask excludes every key (a batch row that is all padding): the reference's quantized sequence
    fills the scores with finfo.min, so the row weighs every key alike (KVCache.swift:2441-2445); the full-precision
    tile that dequantize-first runs would leave it at zero.  Both policies against the oracle."""
    rng = np.random.default_rng(77)
    name = NAME[dtype]
    B, Hkv, r, D, T0, Lq = 2, 2, 4, 128, 300, 70
    scale = D ** -0.5
    lib = kvhip.load()
    try:
        for policy, family in ((3, 4), (2, 3)):
            lib.kvhip_set_kernel_policy(policy)
            c, o = kvhip.QuantizedKVCache(64, 4), O.QuantizedKVCache(64, 4, name)
            k, kd = randn(rng, (B, Hkv, T0, D), dtype)
            v, vd = randn(rng, (B, Hkv, T0, D), dtype)
            c.update_quantized(kd, vd, fetch=False)
            o.update_quantized(k, v)
            k, kd = randn(rng, (B, Hkv, Lq, D), dtype)
            v, vd = randn(rng, (B, Hkv, Lq, D), dtype)
            q, qd = randn(rng, (B, Hkv * r, Lq, D), dtype)
            T = T0 + Lq
            j = np.arange(T)[None, None, None, :]
            causal = np.broadcast_to(O.create_causal_mask(Lq, T - Lq)[None, None], (B, 1, Lq, T))
            if mode == "lengths":
                lengths = np.array([0, T - 20], np.int32)
                m = causal & (j < lengths[:, None, None, None])
                mask = kvhip.MaskMode.window_mask(T - Lq, 0, lengths=torch.from_numpy(lengths))
            elif mode == "left_pad":
                pad = np.array([T0 + 30, 5], np.int32)  # batch row 0: its first 30 query positions are padding
                m = causal & (j >= pad[:, None, None, None])
                mask = kvhip.MaskMode.window_mask(T - Lq, 0, left_pad=torch.from_numpy(pad))
            else:
                m = causal & (rng.random((B, 1, Lq, T)) < 0.8)
                m[..., 0] = True
                m[0, 0, 3:9] = False   # rows without keys, in the middle of a block and ...
                m[1, -1, -1] = False   # ... the last row of the last head
                mask = kvhip.MaskMode.from_array(torch.from_numpy(np.ascontiguousarray(m)).cuda())
            om = O.Mask("array", np.ascontiguousarray(m))
            assert not m.any(axis=-1).all(), "the case needs a row without keys"
            out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
            assert lib.kvhip_last_attend_kernel() == family
            ref = O.attention_with_cache_update(q, k, v, o, scale, om, name)
            empty = ~np.broadcast_to(m, (B, Hkv * r, Lq, T)).any(axis=-1)

            def exact():  # float64, the rows without keys at the mean of V over all keys
                kk, vv = presented_f64(o)
                with np.errstate(invalid="ignore"):
                    ex = exact_attention(q, kk, vv, scale, om)
                ex[empty] = np.broadcast_to(np.repeat(vv, r, axis=1).mean(axis=2)[:, :, None, :], ex.shape)[empty]
                return ex
            check(out, ref, f"policy {policy} {mode}", exact)
            got = np32(out)
            assert np.abs(got[empty]).max() > 0 and np.abs(got[empty] - ref[empty]).max() <= 2e-3
    finally:
        lib.kvhip_set_kernel_policy(0)


@pytest.mark.parametrize("dtype,bits,D", [(torch.float16, 4, 128), (torch.bfloat16, 8, 128), (torch.float16, 3, 96), (torch.bfloat16, 4, (192, 128))])
def test_large_quantized_chunks_run_dequantize_first_by_the_librarys_choice(dtype, bits, D):
    """From 512 query rows per kv head, 2048 keys and rows x keys x (Dk + Dv) = 2^30 (1024 rows over 4096 keys at head
    size 128) a chunk over a quantized cache runs dequantize-first without being told to; a smaller one stays on the
    quantized tile.  The two paths agree to within the rounding of their
    intermediates (both are checked against the oracle at sizes it covers)."""
    D, Dv = D if isinstance(D, tuple) else (D, D)
    g = torch.Generator(device="cuda")
    g.manual_seed(bits + D)
    B, Hkv, r, L, T = 1, 8, 4, 1024, 4096
    c = kvhip.QuantizedKVCache(32 if D == 96 else 64, bits)
    c.update_quantized(torch.randn(B, Hkv, T, D, generator=g, device="cuda").to(dtype), torch.randn(B, Hkv, T, Dv, generator=g, device="cuda").to(dtype), fetch=False)
    lib = kvhip.load()
    scale = D ** -0.5
    try:
        for Lq in (L, 256, 128):
            want = 4 if r * Lq >= 512 and T >= 2048 and r * Lq * T * (D + Dv) >= 2 ** 30 else 3
            q = torch.randn(B, Hkv * r, Lq, D, generator=g, device="cuda").to(dtype)
            for mask in (kvhip.MaskMode.causal(), kvhip.MaskMode.window_mask(T - Lq, 1000)):
                lib.kvhip_set_kernel_policy(0)
                out = np32(c.attend(q, scale, mask))
                assert lib.kvhip_last_attend_kernel() == want
                lib.kvhip_set_kernel_policy(2)
                tile = np32(c.attend(q, scale, mask))
                assert lib.kvhip_last_attend_kernel() == 3
                d = np.abs(out.astype(np.float64) - tile.astype(np.float64))
                assert np.isfinite(out).all() and d.max() <= (4e-3 if dtype == torch.float16 else 2e-2) and d.mean() <= 2e-4, (Lq, d.max(), d.mean())
    finally:
        lib.kvhip_set_kernel_policy(0)
