"""BASELINE.json configs[1], [3] and [4] at their stated sizes, against the oracle.

The reduced versions of these workloads (tests/test_gpu_attention.py, tests/test_gpu_growth.py) cover the
arithmetic; the cases here meet the code that exists only for the full shapes at its own operating point:
the visiting order of a 4096-row ring's slot tiles under 512-row chunks, the one-off gather when the full
ring settles into single-token steps, the pairing of long and short batch rows over 512 workgroups, page
growth over 8192 single-token steps.  Inputs are drawn on the device from a seeded generator and copied to
the host for the oracle; the C restatement (oracle/kv_oracle.c) computes the reference attention at the
rows that are checked.
"""
import numpy as np
import pytest
import torch

import kvhip
from kvhip import _lib as L
from oracle import c_oracle as CO
from oracle import kv_oracle as O
from tests.util import NAME, err_stats, np32

pytestmark = pytest.mark.gpu


def draw(g, shape, dtype, scale=None):
    """N(0,1) (times a per-channel scale) rounded to dtype: (float32 numpy, device tensor)."""
    t = torch.randn(shape, generator=g, device="cuda")
    if scale is not None:
        t = t * scale
    t = t.to(dtype)
    return t.float().cpu().numpy(), t


def check(out, ref, dtype, what):
    """max-abs <= 1e-2 and mean-abs <= 1e-3 against the oracle."""
    got = np32(out)
    assert np.isfinite(got).all(), what
    mx, mean = err_stats(got, ref)
    assert mx <= 1e-2 and mean <= 1e-3, f"{what}: max-abs {mx:.3e} mean-abs {mean:.3e}"


def test_cfg4_ring_4096_at_full_size():
    """configs[3]: RotatingKVCache 4096 keep 4, B4, 8q/4kv, D256, bfloat16; 24 chunks of 512, then 512
    single-token steps.  Chunks 8, 9, 10 and 24 (first full window, first front-trim, steady state, last) and
    decode steps 1, 2 and 512 are compared with the oracle; ring bookkeeping at every chunk and checked step."""
    g = torch.Generator(device="cuda")
    g.manual_seed(4)
    B, Hq, Hkv, D, M, chunk = 4, 8, 4, 256, 4096, 512
    dtype, name = torch.bfloat16, "bfloat16"
    scale = D ** -0.5
    c = kvhip.RotatingKVCache(M, keep=4)
    o = O.RotatingKVCache(M, keep=4, dtype=name)
    lens = []
    for i in range(24):
        q, qd = draw(g, (B, Hq, chunk, D), dtype)
        k, kd = draw(g, (B, Hkv, chunk, D), dtype)
        v, vd = draw(g, (B, Hkv, chunk, D), dtype)
        mask, om = c.make_mask(chunk, M, False), o.make_mask(chunk, M, False)
        assert mask.mode in {"causal": (L.MASK_CAUSAL,), "array": (L.MASK_ARRAY, L.MASK_WINDOW)}[om.mode]
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
        assert kvhip.load().kvhip_last_attend_kernel() == 3
        ko, vo = o.update(k, v)
        lens.append(ko.shape[2])
        assert c.meta_state == o.get_meta_state() and c.presented_length == ko.shape[2]
        if i + 1 in (8, 9, 10, 24):
            ref = CO.sdpa(q, ko, vo, scale, om.array if om.mode == "array" else "causal", name)
            check(out, ref, dtype, f"chunk {i + 1}")
    assert lens[:8] == [512 * (i + 1) for i in range(8)] and lens[8:] == [4607] * 16   # the reference's length trace
    assert c.offset == 12288 and c.idx == 4607
    assert c.slot_span > 4607    # the chunks left unused slots between the ring's rows
    for step in range(1, 513):
        q, qd = draw(g, (B, Hq, 1, D), dtype)
        k, kd = draw(g, (B, Hkv, 1, D), dtype)
        v, vd = draw(g, (B, Hkv, 1, D), dtype)
        mask, om = c.make_mask(1, M, False), o.make_mask(1, M, False)
        assert mask.mode == L.MASK_NONE and om.mode == "none"
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
        ko, vo = o.update(k, v)
        if step in (1, 2, 512):
            assert kvhip.load().kvhip_last_attend_kernel() == 2
            assert c.meta_state == o.get_meta_state() and c.presented_length == 4096 == ko.shape[2]
            # the full ring that takes single tokens was gathered once: the kernels walk its 4096 rows and no more
            assert c.slot_span == 4096
            check(out, CO.sdpa(q, ko, vo, scale, None, name), dtype, f"decode step {step}")
    assert c.offset == 12800 and c.idx == o.idx
    # the ring itself, in the reference's buffer order, bit for bit
    for a, b in zip(c.state, o.get_state()):
        assert np.array_equal(O.to_bits(np32(a), name), O.to_bits(b, name))


def test_cfg5_ragged_rollback_at_full_size():
    """configs[4]: 4-bit QuantizedKVCache, B16, lengths U[1024, 16384] (seed 0) left-padded, 32q/8kv, D128;
    three rounds of 4 draft tokens under causal-and-padding masks, each followed by trim(n)."""
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    B, Hq, Hkv, D, Lq = 16, 32, 8, 128, 4
    dtype, name = torch.float16, "float16"
    lens = np.random.default_rng(0).integers(1024, 16385, size=B)
    Tmax = int(lens.max())
    pad = (Tmax - lens).astype(np.int32)
    pad_d = torch.from_numpy(pad).cuda()
    scale = D ** -0.5
    c = kvhip.QuantizedKVCache(64, 4)
    kq, vq = None, None   # the oracle's six arrays, grown by concatenation as the reference grows them
    for t0 in range(0, Tmax, 4096):
        n = min(4096, Tmax - t0)
        k, kd = draw(g, (B, Hkv, n, D), dtype)
        v, vd = draw(g, (B, Hkv, n, D), dtype)
        c.update_quantized(kd, vd, fetch=False)
        nk, nv = CO.affine_quantize(k, 64, 4, name), CO.affine_quantize(v, 64, 4, name)
        kq = nk if kq is None else tuple(np.concatenate([a, b], axis=2) for a, b in zip(kq, nk))
        vq = nv if vq is None else tuple(np.concatenate([a, b], axis=2) for a, b in zip(vq, nv))
    offset = Tmax
    trims = [3, 0, 2]
    order = np.argsort(lens)
    for rnd in range(3):
        q, qd = draw(g, (B, Hq, Lq, D), dtype)
        k, kd = draw(g, (B, Hkv, Lq, D), dtype)
        v, vd = draw(g, (B, Hkv, Lq, D), dtype)
        mask = kvhip.MaskMode.window_mask(offset, 0, left_pad=pad_d)
        out = kvhip.attention_with_cache_update(qd, kd, vd, c, scale, mask)
        assert kvhip.load().kvhip_last_attend_kernel() == 1
        nk, nv = CO.affine_quantize(k, 64, 4, name), CO.affine_quantize(v, 64, 4, name)
        kq = tuple(np.concatenate([a[:, :, :offset], b], axis=2) for a, b in zip(kq, nk))
        vq = tuple(np.concatenate([a[:, :, :offset], b], axis=2) for a, b in zip(vq, nv))
        T = offset + Lq
        assert c.offset == T
        # every batch row in the first round; afterwards the shortest, the longest and two from the middle
        rows = list(range(B)) if rnd == 0 else [int(order[0]), int(order[-1]), int(order[5]), int(order[10])]
        m = O.create_causal_mask(Lq, T - Lq)[None, None] & (np.arange(T)[None, None, None, :] >= pad[rows, None, None, None])
        ref = CO.qsdpa(q[rows], tuple(a[rows] for a in kq), tuple(a[rows] for a in vq), scale, m, 64, 4, name)
        check(out[rows], ref, dtype, f"round {rnd + 1}")
        assert c.trim(trims[rnd]) == trims[rnd]
        offset = T - trims[rnd]
        assert c.offset == offset and c.meta_state == ["256", str(offset), "64", "4"]
    # codes and scale / bias pairs of everything kept, bit for bit
    for a, b in zip(c.state, [x[:, :, :offset] for x in kq + vq]):
        if a.dtype == torch.int32:
            assert np.array_equal(np32(a), b)
        else:
            assert np.array_equal(O.to_bits(np32(a), name), O.to_bits(b, name))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_cfg2_simple_cache_one_token_per_step_to_8192(dtype):
    """configs[1]: KVCacheSimple, B8, 32q/8kv, D128, K/V ~ 0.5 N(0,1) with 1 % of the channels x8, grown from
    empty to 8192 rows one token per step; attention checked at 256, 4096 and 8192 rows."""
    g = torch.Generator(device="cuda")
    g.manual_seed(2)
    B, Hq, Hkv, D, N = 8, 32, 8, 128, 8192
    name = NAME[dtype]
    ch = torch.full((D,), 0.5, device="cuda")
    ch[torch.randperm(D, generator=g, device="cuda")[:max(1, D // 100)]] = 4.0
    k_all, kd_all = draw(g, (B, Hkv, N, D), dtype, ch)
    v_all, vd_all = draw(g, (B, Hkv, N, D), dtype, ch)
    qd_all = torch.randn((N, B, Hq, 1, D), generator=g, device="cuda").to(dtype)
    scale = D ** -0.5
    c = kvhip.KVCacheSimple()
    for t in range(N):
        out = c.update_attend(qd_all[t], kd_all[:, :, t:t + 1], vd_all[:, :, t:t + 1], scale)
        if t + 1 in (256, 4096, N):
            assert kvhip.load().kvhip_last_attend_kernel() == 2
            assert c.offset == t + 1 and c.capacity == 256 * ((t + 256) // 256)   # step growth of the reference
            ref = CO.sdpa(qd_all[t].float().cpu().numpy(), k_all[:, :, :t + 1], v_all[:, :, :t + 1], scale, None, name)
            check(out, ref, dtype, f"{t + 1} rows")
    ks, vs = c.state
    assert np.array_equal(O.to_bits(np32(ks), name), O.to_bits(k_all, name))
    assert np.array_equal(O.to_bits(np32(vs), name), O.to_bits(v_all, name))
