"""Shared helpers for the parity tests: torch <-> oracle array conversion."""
import numpy as np
import torch

from oracle import kv_oracle as O

NAME = {torch.float16: "float16", torch.bfloat16: "bfloat16", torch.float32: "float32"}
TORCH = {v: k for k, v in NAME.items()}


def np32(t):
    """Device tensor -> float32 numpy (exact for 16-bit float types)."""
    if t.dtype == torch.bool:
        return t.cpu().numpy()
    if t.dtype in (torch.int32,):
        return t.cpu().numpy().view(np.uint32)
    return t.detach().to(torch.float32).cpu().numpy()


def dev(a, dtype):
    """float32 numpy holding T-representable values -> device tensor of dtype T."""
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dtype).cuda()


def randn(rng, shape, dtype, scale=1.0):
    """Seeded N(0,1)*scale rounded to dtype; returns (float32 numpy, device tensor)."""
    a = O.round_to(rng.standard_normal(shape).astype(np.float32) * np.float32(scale), NAME[dtype])
    return a, dev(a, dtype)


def bits_equal(t, a32, dtype):
    """Device tensor `t` of dtype T equals oracle float32 array bit for bit."""
    name = NAME[dtype]
    got = O.to_bits(np32(t), name)
    want = O.to_bits(a32, name)
    return np.array_equal(got, want)


def err_stats(got, want):
    d = np.abs(got.astype(np.float64) - want.astype(np.float64))
    return float(d.max()), float(d.mean())


def presented_f64(o):
    """What an oracle cache presents after its last update, as float64 (a quantized cache dequantised exactly:
    scale * code + bias with no rounding)."""
    if isinstance(o, O.QuantizedKVCache):
        def deq(w, sc, bi):
            codes = O.unpack_codes(w, o.bits).astype(np.float64)
            g = codes.reshape(codes.shape[:-1] + (sc.shape[-1], o.group_size))
            return (g * sc[..., None].astype(np.float64) + bi[..., None].astype(np.float64)).reshape(codes.shape)
        qk, qv = o.get_quantized_state()
        return deq(*qk), deq(*qv)
    k, v = o.get_state()
    return k.astype(np.float64), v.astype(np.float64)


def exact_attention(q, k, v, scale, om):
    """softmax(q k^T scale + mask) v in float64 with no intermediate rounding.  q [B,Hq,L,D], k / v [B,Hkv,T,.];
    `om` an oracle Mask (none / causal / array: bool excludes, other dtypes add; [L,T], [B,1,L,T] or [B,Hq,L,T])."""
    B, Hq, L, D = q.shape
    Hkv, T = k.shape[1], k.shape[2]
    r = Hq // Hkv
    kk, vv = np.repeat(k, r, axis=1), np.repeat(v, r, axis=1)
    s = np.einsum("bhld,bhtd->bhlt", q.astype(np.float64), kk) * float(scale)
    if om is not None and om.mode == "causal":
        s = np.where(np.tril(np.ones((L, T), bool), k=T - L), s, -np.inf)
    elif om is not None and om.mode == "array":
        m = om.array
        while m.ndim < 4:
            m = m[None]
        s = np.where(m, s, -np.inf) if m.dtype == np.bool_ else s + m.astype(np.float64)
    s = s - s.max(axis=-1, keepdims=True)
    p = np.exp(s)
    return np.einsum("bhlt,bhtd->bhld", p / p.sum(axis=-1, keepdims=True), vv)


def check_attention(out, ref, dtype, what, exact=None):
    """The bound of the parity tests: max-abs <= 1e-2 and mean-abs <= 1e-3 against the oracle.

    A result outside it is accepted only against a float64 evaluation of the same attention (`exact`, a
    callable): the oracle keeps the reference's intermediate roundings to the cache dtype (one step of bfloat16
    is 7.8e-3 at 1), the kernels keep some of those intermediates with more bits, so where the two differ by more
    than the bound the device result must lie as close to the exact result as the oracle's does -- within 1.25
    times the oracle's own distance plus one rounding step of the output type at the largest output (maximum;
    an eighth of a step for the mean)."""
    got = np32(out) if hasattr(out, "detach") else out
    assert np.isfinite(got).all(), what
    mx, mean = err_stats(got, ref)
    if mx <= 1e-2 and mean <= 1e-3:
        return
    assert exact is not None and dtype != torch.float32, f"{what}: max-abs {mx:.3e} mean-abs {mean:.3e}"
    ex = exact()
    dd, do = np.abs(got.astype(np.float64) - ex), np.abs(ref.astype(np.float64) - ex)
    step = 2.0 ** (np.floor(np.log2(max(float(np.abs(ex).max()), 1e-30))) - (7 if dtype == torch.bfloat16 else 10))
    assert dd.max() <= 1.25 * do.max() + step and dd.mean() <= 1.25 * do.mean() + step / 8, (
        f"{what}: against the oracle max-abs {mx:.3e} mean-abs {mean:.3e}; against float64 device {dd.max():.3e} / "
        f"{dd.mean():.3e}, oracle {do.max():.3e} / {do.mean():.3e}, step {step:.3e}")
