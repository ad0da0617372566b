"""Seeded random sweep over cache kind x dtype x head size x query rows x presentation x mask:
the library's own kernel choice against the generic kernel (which the other GPU tests pin to the
oracle), on the same device cache.  Every case prints what it is before it runs."""
import numpy as np
import pytest
import torch

import kvhip
from tests.util import np32

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS = 1e-2, 1e-3


def _case(seed):
    rng = np.random.default_rng(seed)
    kind = rng.choice(["simple", "rotating", "quantized"])
    dtype = [torch.float16, torch.bfloat16][rng.integers(2)]
    D = int(rng.choice([64, 128, 256] if kind != "quantized" else [64, 128]))
    if kind != "quantized" and seed % 5 == 4:
        D = 96 if seed % 10 == 4 else 80  # these head sizes run on the prefill tile at every row count
    B, Hkv, r = int(rng.integers(1, 6)), int(rng.choice([1, 2, 4])), int(rng.choice([1, 2, 4, 8]))
    Lq = int(rng.choice([1, 1, 2, 4, 7, 33, 70]))
    T0 = int(rng.choice([1, 63, 64, 65, 200, 257, 700, 1500, 2600]))
    return rng, kind, dtype, D, B, Hkv, r, Lq, T0


@pytest.mark.parametrize("seed", range(160))
def test_auto_kernel_against_generic(seed):
    rng, kind, dtype, D, B, Hkv, r, Lq, T0 = _case(seed)
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)

    def rand(*shape):
        return torch.randn(*shape, generator=g, device="cuda").to(dtype)

    if kind == "simple":
        c = kvhip.KVCacheSimple()
    elif kind == "rotating":
        c = kvhip.RotatingKVCache(int(rng.choice([96, 300, 1024])), keep=int(rng.choice([0, 4])))
    else:
        c = kvhip.QuantizedKVCache(64, int(rng.choice([4, 8])))
    upd = c.update_quantized if kind == "quantized" else c.update
    upd(rand(B, Hkv, T0, D), rand(B, Hkv, T0, D), fetch=False)
    for _ in range(int(rng.integers(0, 40)) if kind == "rotating" else 0):  # walk (and wrap) the ring
        upd(rand(B, Hkv, 1, D), rand(B, Hkv, 1, D), fetch=False)
    upd(rand(B, Hkv, Lq, D), rand(B, Hkv, Lq, D), fetch=False)
    T = c.presented_length
    Lq = min(Lq, T)
    q = rand(B, Hkv * r, Lq, D)
    which = rng.choice(["none", "causal", "window", "lengths", "left_pad", "bool", "additive"])
    if which == "none":
        mask = kvhip.MaskMode.none()
    elif which == "causal":
        mask = kvhip.MaskMode.causal()
    elif which == "window":
        mask = kvhip.MaskMode.window_mask(T - Lq, int(rng.integers(1, T + 2)))
    elif which == "lengths":
        lens = torch.from_numpy(rng.integers(1, T + 1, size=B).astype(np.int32))
        mask = kvhip.MaskMode.window_mask(T - Lq, 0, lengths=lens)
    elif which == "left_pad":
        pad = torch.from_numpy(rng.integers(0, max(T - Lq, 1), size=B).astype(np.int32))
        mask = kvhip.MaskMode.window_mask(T - Lq, int(rng.choice([0, 50])), left_pad=pad)
    else:
        shape = [(B, 1, Lq, T), (1, 1, Lq, T), (B, Hkv * r, Lq, T)][rng.integers(3)]
        keep = rng.random(shape) < 0.7
        keep[..., int(rng.integers(T))] = True  # no row without a key
        if which == "bool":
            mask = kvhip.MaskMode.from_array(torch.from_numpy(keep).cuda())
        else:
            add = np.where(keep, rng.standard_normal(shape).astype(np.float32), -np.inf)
            mask = kvhip.MaskMode.from_array(torch.from_numpy(add).to(dtype).cuda())
    scale = float(rng.choice([D ** -0.5, 0.05, -0.1]))
    print(f"seed {seed}: {kind} {dtype} D{D} B{B} Hkv{Hkv} r{r} L{Lq} T{T} mask {which} scale {scale:.3f}", flush=True)
    lib = kvhip.load()
    try:
        lib.kvhip_set_kernel_policy(1)
        ref = np32(c.attend(q, scale, mask))
        lib.kvhip_set_kernel_policy(0)
        out = np32(c.attend(q, scale, mask))
        chosen = lib.kvhip_last_attend_kernel()
    finally:
        lib.kvhip_set_kernel_policy(0)
    assert np.isfinite(ref).all() and np.isfinite(out).all(), f"kernel {chosen}"
    d = np.abs(out.astype(np.float64) - ref.astype(np.float64))
    # One ulp of a 16-bit output at the largest magnitude may separate two correctly rounded results;
    # with a handful of keys the outputs are as large as single V rows and, the probabilities being
    # rounded to the cache's dtype before the second product (as the reference does), a good part
    # of them round the other way: hence the quarter ulp on the mean.
    ulp = float(np.abs(ref).max()) * (2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10)
    assert d.max() <= max(MAX_ABS, ulp) and d.mean() <= max(MEAN_ABS, ulp / 4), \
        f"kernel {chosen}: max-abs {d.max():.3e} mean-abs {d.mean():.3e}"


@pytest.mark.parametrize("seed", range(72))
def test_quantized_shapes_against_generic(seed):
    """Quantized caches over head size x group size x bits x query rows (decode rows included: the
    shapes the decode kernels do not take go to the prefill tile, not to the generic kernel)."""
    rng = np.random.default_rng(1000 + seed)
    D = [64, 128, 256][seed % 3]
    gs = [32, 64, 128][(seed // 3) % 3]
    if gs > D:
        gs = 64
    if seed % 7 == 6:
        D, gs = 96, 32  # the only group size that divides 96 (16 rows or fewer: the 16-row kernel)
    bits = [4, 8][(seed // 9) % 2]
    dtype = [torch.float16, torch.bfloat16][(seed // 18) % 2]
    B, Hkv, r = int(rng.integers(1, 4)), int(rng.choice([1, 2])), int(rng.choice([1, 4, 8]))
    Lq = int(rng.choice([1, 1, 2, 4, 5, 40, 70]))
    T0 = int(rng.choice([1, 31, 64, 200, 257, 700, 1300]))
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)

    def rand(*shape):
        return torch.randn(*shape, generator=g, device="cuda").to(dtype)

    c = kvhip.QuantizedKVCache(gs, bits)
    c.update_quantized(rand(B, Hkv, T0, D), rand(B, Hkv, T0, D), fetch=False)
    c.update_quantized(rand(B, Hkv, Lq, D), rand(B, Hkv, Lq, D), fetch=False)
    assert c.group_size == gs
    T = c.offset
    q = rand(B, Hkv * r, Lq, D)
    which = rng.choice(["none", "causal", "left_pad", "bool"])
    if which == "none":
        mask = kvhip.MaskMode.none()
    elif which == "causal":
        mask = kvhip.MaskMode.causal()
    elif which == "left_pad":
        pad = torch.from_numpy(rng.integers(0, max(T - Lq, 1), size=B).astype(np.int32))
        mask = kvhip.MaskMode.window_mask(T - Lq, 0, left_pad=pad)
    else:
        keep = rng.random((B, 1, Lq, T)) < 0.7
        keep[..., int(rng.integers(T))] = True
        mask = kvhip.MaskMode.from_array(torch.from_numpy(keep).cuda())
    scale = D ** -0.5
    print(f"seed {seed}: {dtype} D{D} g{gs} {bits}-bit B{B} Hkv{Hkv} r{r} L{Lq} T{T} mask {which}", flush=True)
    lib = kvhip.load()
    try:
        lib.kvhip_set_kernel_policy(1)
        ref = np32(c.attend(q, scale, mask))
        lib.kvhip_set_kernel_policy(0)
        out = np32(c.attend(q, scale, mask))
        chosen = lib.kvhip_last_attend_kernel()
    finally:
        lib.kvhip_set_kernel_policy(0)
    assert chosen != 0, "a quantized cache of a supported head size fell back to the generic kernel"
    assert np.isfinite(ref).all() and np.isfinite(out).all(), f"kernel {chosen}"
    d = np.abs(out.astype(np.float64) - ref.astype(np.float64))
    # two results that each lie within one step of the 16-bit output type of the exact value may
    # differ by two steps (the generic kernel also rounds the probabilities to that type)
    ulp = float(np.abs(ref).max()) * (2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10)
    assert d.max() <= max(MAX_ABS, 2 * ulp) and d.mean() <= max(MEAN_ABS, ulp / 4), \
        f"kernel {chosen}: max-abs {d.max():.3e} mean-abs {d.mean():.3e}"


@pytest.mark.parametrize("seed", range(48))
def test_other_code_widths_against_generic(seed):
    """2-, 3-, 5- and 6-bit caches, mostly at decode row counts: up to 16 query rows per kv head run on the 16-row
    decode kernel where it has an instance for the head and group size, everything else on the prefill tile."""
    rng = np.random.default_rng(7000 + seed)
    bits = [2, 3, 5, 6][seed % 4]
    D = [64, 128, 256][(seed // 4) % 3]
    gs = [32, 64, 128][(seed // 12) % 3]
    if gs > D:
        gs = 32
    dtype = [torch.float16, torch.bfloat16][(seed // 2) % 2]
    B, Hkv, r = int(rng.integers(1, 4)), int(rng.choice([1, 2])), int(rng.choice([1, 3, 4, 8]))
    Lq = int(rng.choice([1, 1, 1, 2, 4, 5, 40]))
    T0 = int(rng.choice([1, 31, 64, 200, 257, 700, 1300, 3100]))
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)

    def rand(*shape):
        return torch.randn(*shape, generator=g, device="cuda").to(dtype)

    c = kvhip.QuantizedKVCache(gs, bits)
    c.update_quantized(rand(B, Hkv, T0, D), rand(B, Hkv, T0, D), fetch=False)
    c.update_quantized(rand(B, Hkv, Lq, D), rand(B, Hkv, Lq, D), fetch=False)
    assert c.group_size == gs
    T = c.offset
    q = rand(B, Hkv * r, Lq, D)
    which = rng.choice(["none", "causal", "left_pad", "lengths", "bool"])
    if which == "none":
        mask = kvhip.MaskMode.none()
    elif which == "causal":
        mask = kvhip.MaskMode.causal()
    elif which == "left_pad":
        pad = torch.from_numpy(rng.integers(0, max(T - Lq, 1), size=B).astype(np.int32))
        mask = kvhip.MaskMode.window_mask(T - Lq, 0, left_pad=pad)
    elif which == "lengths":
        lengths = torch.from_numpy(rng.integers(1, T + 1, size=B).astype(np.int32))
        mask = kvhip.MaskMode.window_mask(T - Lq, 0, lengths=lengths)
    else:
        keep = rng.random((B, 1, Lq, T)) < 0.7
        keep[..., int(rng.integers(T))] = True
        mask = kvhip.MaskMode.from_array(torch.from_numpy(keep).cuda())
    scale = D ** -0.5
    print(f"seed {seed}: {dtype} D{D} g{gs} {bits}-bit B{B} Hkv{Hkv} r{r} L{Lq} T{T} mask {which}", flush=True)
    lib = kvhip.load()
    try:
        lib.kvhip_set_kernel_policy(1)
        ref = np32(c.attend(q, scale, mask))
        lib.kvhip_set_kernel_policy(0)
        out = np32(c.attend(q, scale, mask))
        chosen = lib.kvhip_last_attend_kernel()
    finally:
        lib.kvhip_set_kernel_policy(0)
    decode_shape = (D == 64 and gs in (32, 64)) or D == 128 or (D == 256 and gs == 64)
    assert chosen == (1 if r * Lq <= 16 and decode_shape else 3), chosen
    assert np.isfinite(ref).all() and np.isfinite(out).all(), f"kernel {chosen}"
    d = np.abs(out.astype(np.float64) - ref.astype(np.float64))
    ulp = float(np.abs(ref).max()) * (2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10)
    assert d.max() <= max(MAX_ABS, 2 * ulp) and d.mean() <= max(MEAN_ABS, ulp / 4), \
        f"kernel {chosen}: max-abs {d.max():.3e} mean-abs {d.mean():.3e}"


@pytest.mark.parametrize("seed", range(48))
def test_keys_of_192_values_of_128_against_generic(seed):
    """Keys of 192 with values of 128 (multi-head latent attention) in all three cache kinds, on the prefill tiles
    (quantized caches: up to 16 query rows per kv head on the 16-row decode kernel): the tuned result against the
    generic kernel's."""
    rng = np.random.default_rng(5000 + seed)
    kind = ["simple", "rotating", "quantized"][seed % 3]
    dtype = [torch.float16, torch.bfloat16][(seed // 3) % 2]
    Dk, Dv = 192, 128
    B, Hkv, r = int(rng.integers(1, 4)), int(rng.choice([1, 2, 4])), int(rng.choice([1, 2, 8]))
    Lq = int(rng.choice([1, 1, 3, 16, 40, 70, 130]))
    T0 = int(rng.choice([1, 31, 64, 200, 257, 700, 1300]))
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)

    def rand(*shape):
        return torch.randn(*shape, generator=g, device="cuda").to(dtype)

    if kind == "simple":
        c = kvhip.KVCacheSimple()
    elif kind == "rotating":
        c = kvhip.RotatingKVCache(int(rng.choice([96, 300, 1024])), keep=int(rng.choice([0, 4])))
    else:
        c = kvhip.QuantizedKVCache(int(rng.choice([32, 64])), int(rng.choice([4, 8])))
    upd = c.update_quantized if kind == "quantized" else c.update
    upd(rand(B, Hkv, T0, Dk), rand(B, Hkv, T0, Dv), fetch=False)
    for _ in range(int(rng.integers(0, 40)) if kind == "rotating" else 0):
        upd(rand(B, Hkv, 1, Dk), rand(B, Hkv, 1, Dv), fetch=False)
    upd(rand(B, Hkv, Lq, Dk), rand(B, Hkv, Lq, Dv), fetch=False)
    T = c.presented_length
    Lq = min(Lq, T)
    q = rand(B, Hkv * r, Lq, Dk)
    which = rng.choice(["none", "causal", "window", "left_pad", "bool", "additive"])
    if which == "none":
        mask = kvhip.MaskMode.none()
    elif which == "causal":
        mask = kvhip.MaskMode.causal()
    elif which == "window":
        mask = kvhip.MaskMode.window_mask(T - Lq, int(rng.integers(1, T + 2)))
    elif which == "left_pad":
        pad = torch.from_numpy(rng.integers(0, max(T - Lq, 1), size=B).astype(np.int32))
        mask = kvhip.MaskMode.window_mask(T - Lq, 0, left_pad=pad)
    else:
        shape = [(B, 1, Lq, T), (1, 1, Lq, T)][rng.integers(2)]
        keep = rng.random(shape) < 0.7
        keep[..., int(rng.integers(T))] = True
        if which == "bool":
            mask = kvhip.MaskMode.from_array(torch.from_numpy(keep).cuda())
        else:
            add = np.where(keep, rng.standard_normal(shape).astype(np.float32), -np.inf)
            mask = kvhip.MaskMode.from_array(torch.from_numpy(add).to(dtype).cuda())
    scale = Dk ** -0.5
    print(f"seed {seed}: {kind} {dtype} B{B} Hkv{Hkv} r{r} L{Lq} T{T} mask {which}", flush=True)
    lib = kvhip.load()
    try:
        lib.kvhip_set_kernel_policy(1)
        ref = np32(c.attend(q, scale, mask))
        lib.kvhip_set_kernel_policy(0)
        out = np32(c.attend(q, scale, mask))
        chosen = lib.kvhip_last_attend_kernel()
    finally:
        lib.kvhip_set_kernel_policy(0)
    # (up to 16 query rows per kv head of a quantized cache: the 16-row decode kernel)
    assert chosen == (1 if kind == "quantized" and r * Lq <= 16 else 3) and out.shape == (B, Hkv * r, Lq, Dv)
    assert np.isfinite(ref).all() and np.isfinite(out).all()
    d = np.abs(out.astype(np.float64) - ref.astype(np.float64))
    ulp = float(np.abs(ref).max()) * (2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10)
    assert d.max() <= max(MAX_ABS, 2 * ulp) and d.mean() <= max(MEAN_ABS, ulp / 4), \
        f"max-abs {d.max():.3e} mean-abs {d.mean():.3e}"


@pytest.mark.parametrize("kind,dtype,B,Hkv,L,extra", [
    ("simple", torch.float16, 1, 8, 2048, 0), ("simple", torch.bfloat16, 2, 8, 1024, 512),
    ("quantized", torch.float16, 1, 8, 2048, 0), ("quantized", torch.float16, 2, 8, 1024, 300),
])
def test_causal_grids_of_two_workgroups_per_cu(kind, dtype, B, Hkv, L, extra):
    """A causal prompt chunk whose prefill grid is exactly 512 workgroups (4 query heads per kv head, 128 query
    rows per workgroup): the kernels then pair a long and a short query block on every CU by renumbering the
    workgroups, which must still hand every query block to exactly one of them -- checked against the generic
    kernel over the same device cache."""
    D, r = 128, 4
    g = torch.Generator(device="cuda")
    g.manual_seed(B * 1000 + L)

    def rand(*shape):
        return torch.randn(*shape, generator=g, device="cuda").to(dtype)

    T = L + extra
    if kind == "simple":
        c = kvhip.KVCacheSimple()
        c.update(rand(B, Hkv, T, D), rand(B, Hkv, T, D), fetch=False)
    else:
        c = kvhip.QuantizedKVCache(64, 4)
        c.update_quantized(rand(B, Hkv, T, D), rand(B, Hkv, T, D), fetch=False)
    assert (r * L // 128) * B * Hkv == 512
    q = rand(B, Hkv * r, L, D)
    lib = kvhip.load()
    try:
        lib.kvhip_set_kernel_policy(1)
        ref = np32(c.attend(q, D ** -0.5, kvhip.MaskMode.causal()))
        # (a quantized chunk of this many rows would run dequantize-first: policy 2 keeps it on the quantized tile,
        # whose renumbering this case is about)
        lib.kvhip_set_kernel_policy(2 if kind == "quantized" else 0)
        out = np32(c.attend(q, D ** -0.5, kvhip.MaskMode.causal()))
        assert lib.kvhip_last_attend_kernel() == 3
    finally:
        lib.kvhip_set_kernel_policy(0)
    d = np.abs(out.astype(np.float64) - ref.astype(np.float64))
    ulp = float(np.abs(ref).max()) * (2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10)
    assert np.isfinite(out).all() and d.max() <= max(MAX_ABS, ulp) and d.mean() <= max(MEAN_ABS, ulp / 4), (d.max(), d.mean())
