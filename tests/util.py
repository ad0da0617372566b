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
