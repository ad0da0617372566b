"""BASELINE.json configs[2] on its stated data through the C ABI: QuantizedKVCache 4-bit, group 64,
32 query / 8 kv heads, head size 128, batch 32, float16; K and V ~ N(0,1) times a per-channel scale
drawn log-uniform in [0.1, 10], queries ~ N(0,1), seed 0.  Prompt rows go through the whole-tile
quantizer, decode rows through the per-row one, then the fused dequantize + attention kernel
(KVCache.swift:1011-1102, :2351-2447).

The bound, per output element against the CPU oracle (the reference's op sequence with its rounding
points: q*scale, scores and probabilities rounded to float16):

    |out - oracle| <= max(1e-2, one float16 step at |oracle|)      and      mean |out - oracle| <= 1e-3.

On this data the rows are peaked (|V| reaches 60, one key can hold half the weight) and scores reach
|s| = 16..32, where one float16 step is 1.56e-2: a score whose exact value sits on a rounding boundary
moves its key's weight by 1.6 % when it falls to the other side, and the output with it by several
1e-2.  Which side it falls to depends on the float32 summation order inside the score contraction,
which differs between MLX, the oracle and the matrix cores; all of them are the reference's op
sequence.  A query row that exceeds the bound above is therefore accepted only if the test can show
exactly that: the float64 evaluation of the same op sequence, with the near-tie scores of that row
rounded the other way, reproduces the kernel's row within the same bound.  Anything else fails.
"""
import itertools

import numpy as np
import pytest
import torch

import kvhip
from oracle import c_oracle as CO
from oracle import kv_oracle as O

pytestmark = pytest.mark.gpu

B, HQ, HKV, D, GS, BITS = 32, 32, 8, 128, 64, 4
R = HQ // HKV
SCALE = D ** -0.5


def f16_step(x):
    """Spacing of float16 at |x| (float64 numpy)."""
    a = np.maximum(np.abs(x), 2.0 ** -14)
    return 2.0 ** (np.floor(np.log2(a)) - 10)


def draw(T, seed, decode_steps):
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    ch = (10.0 ** (torch.rand(D, generator=g, device=dev) * 2 - 1)).float()
    cache = kvhip.QuantizedKVCache(GS, BITS)
    kept = []
    for t0 in range(0, T, 2048):
        n = min(2048, T - t0)
        k = (torch.randn(B, HKV, n, D, generator=g, device=dev) * ch).half()
        v = (torch.randn(B, HKV, n, D, generator=g, device=dev) * ch).half()
        cache.update_quantized(k, v, fetch=False)
        kept.append((k[:2, :1].cpu(), v[:2, :1].cpu()))   # batch rows 0..1, kv head 0: for the state check
    out = q = None
    for _ in range(decode_steps):
        q = torch.randn(B, HQ, 1, D, generator=g, device=dev).half()
        k = (torch.randn(B, HKV, 1, D, generator=g, device=dev) * ch).half()
        v = (torch.randn(B, HKV, 1, D, generator=g, device=dev) * ch).half()
        out = cache.update_attend(q, k, v, SCALE)
        kept.append((k[:2, :1].cpu(), v[:2, :1].cpu()))
    torch.cuda.synchronize()
    assert kvhip.load().kvhip_last_attend_kernel() == 1, "the quantized matrix-core decode kernel must serve this call"
    return cache, q, out, kept


def unpack_np(wq):
    sh = np.arange(0, 32, BITS, dtype=np.uint32)
    c = (wq[..., None] >> sh) & np.uint32((1 << BITS) - 1)
    return c.reshape(wq.shape[:-1] + (-1,))


def deq64(wq, s, b):
    c = unpack_np(wq).astype(np.float64)
    c = c.reshape(c.shape[:-1] + (s.shape[-1], GS))
    return (c * s.astype(np.float64)[..., None] + b.astype(np.float64)[..., None]).reshape(wq.shape[:-1] + (-1,))


def softmax64(s):
    e = np.exp(s - s.max())
    return e / e.sum()


def tie_flip_explains(got_row, q_row, kq, vq):
    """True if the kernel's output row is, within the bound, the float64 evaluation of the reference's
    op sequence with some of the row's near-tie scores rounded to float16 the other way."""
    K = deq64(*kq)                                        # [T, D]
    V = deq64(*vq)
    qs = O.round_to(q_row.astype(np.float32) * np.float32(SCALE), "float16").astype(np.float64)
    s = K @ qs                                            # exact scores
    r0 = s.astype(np.float16)
    toward = np.where(s >= r0.astype(np.float64), np.float16(np.inf), np.float16(-np.inf))
    r1 = np.nextafter(r0, toward)                         # the float16 neighbour on the other side of s
    r0, r1 = r0.astype(np.float64), r1.astype(np.float64)
    mid = 0.5 * (r0 + r1)
    closeness = np.abs(s - mid) / np.abs(r1 - r0)         # 0: exactly on the rounding boundary
    p0 = softmax64(r0)
    cand = np.nonzero((closeness < 0.02) & (p0 > 1e-4))[0]
    cand = cand[np.argsort(-p0[cand])][:4]
    for k in range(0, len(cand) + 1):
        for flips in itertools.combinations(cand, k):
            r = r0.copy()
            r[list(flips)] = r1[list(flips)]
            out = softmax64(r) @ V
            if np.all(np.abs(got_row - out) <= np.maximum(1e-2, f16_step(out))):
                return True, len(cand), k
    return False, len(cand), -1


@pytest.mark.parametrize("T,seed,steps", [(4096, 0, 3), (32768, 0, 1)])
def test_configs2_on_its_stated_data(T, seed, steps):
    cache, q, out, kept = draw(T, seed, steps)
    assert cache.offset == T + steps
    st = [a.cpu().numpy() for a in cache.state]
    kq = (st[0].view(np.uint32), st[1].astype(np.float32), st[2].astype(np.float32))
    vq = (st[3].view(np.uint32), st[4].astype(np.float32), st[5].astype(np.float32))

    # codes, scales and biases of two (batch row, kv head) pairs against the CPU quantizer: bit-exact
    k_cpu = torch.cat([k for k, _ in kept], dim=2).float().numpy()
    v_cpu = torch.cat([v for _, v in kept], dim=2).float().numpy()
    for plane, src in ((kq, k_cpu), (vq, v_cpu)):
        wq, s, b = CO.affine_quantize(src, GS, BITS, "float16")
        assert np.array_equal(plane[0][:2, :1], wq)
        assert np.array_equal(O.to_bits(plane[1][:2, :1], "float16"), O.to_bits(s, "float16"))
        assert np.array_equal(O.to_bits(plane[2][:2, :1], "float16"), O.to_bits(b, "float16"))

    qn = q.float().cpu().numpy()
    ref = CO.qsdpa(qn, kq, vq, SCALE, None, GS, BITS, "float16").astype(np.float64)
    got = out.float().cpu().numpy().astype(np.float64)
    err = np.abs(got - ref)
    assert err.mean() <= 1e-3, err.mean()
    tol = np.maximum(1e-2, f16_step(ref))
    bad_rows = np.argwhere((err > tol).any(axis=-1)[:, :, 0])
    # every row outside the bound must be explained by float16 ties of its scores, and such rows are rare
    assert len(bad_rows) <= 8, f"{len(bad_rows)} of {B * HQ} query rows exceed max(1e-2, one float16 step)"
    for b, h in bad_rows:
        hk = h // R
        ok, ncand, nflip = tie_flip_explains(
            got[b, h, 0], qn[b, h, 0],
            (kq[0][b, hk], kq[1][b, hk], kq[2][b, hk]), (vq[0][b, hk], vq[1][b, hk], vq[2][b, hk]))
        assert ok, (f"row (batch {b}, head {h}): max |out - oracle| {err[b, h].max():.3e} is not reproduced by "
                    f"rounding any of its {ncand} near-tie scores the other way")

    # against the exact (float64, no intermediate rounding) result the kernel is as good as the
    # reference's own rounding sequence
    dev = out.device
    truth = np.empty_like(got)
    for b in range(B):
        Kb = torch.from_numpy(deq64(kq[0][b], kq[1][b], kq[2][b])).to(dev)   # [Hkv, T, D]
        Vb = torch.from_numpy(deq64(vq[0][b], vq[1][b], vq[2][b])).to(dev)
        qb = (q[b].float() * SCALE).half().double().reshape(HKV, R, D)
        p = torch.softmax(torch.einsum("hrd,htd->hrt", qb, Kb), -1)
        truth[b] = torch.einsum("hrt,htd->hrd", p, Vb).reshape(HQ, 1, D).cpu().numpy()
    e_got, e_ref = np.abs(got - truth).mean(), np.abs(ref - truth).mean()
    assert e_got <= 1.25 * e_ref + 1e-5, (e_got, e_ref)
    assert np.abs(got - truth).max() <= 1.25 * np.abs(ref - truth).max() + 1e-2
