"""CPU restatement of the rotary embedding the reference applies before the cache write.

TEST INFRASTRUCTURE ONLY: nothing outside tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg may import this module.

The reference's layers end in `MLXFast.RoPE(x, dimensions:, traditional:, base:, scale:,
offset:, freqs:)` (RoPEUtils.swift:139-156, SuScaledRoPE.swift:49-70), called through
`applyRotaryPosition` with `cache.ropeOffset` (Llama.swift:58-60, RoPEApplication.swift:62-74).
`MLXFast.RoPE` lives in mlx-swift (pinned 0.31.6 ..< 0.32.0, not in this tree); its published
definition is restated here: for position p = offset + l, pair i of the first `dims` elements
turns by theta = (p * scale) * inv_freq[i], inv_freq[i] = exp(-i * log(base) / (dims/2)) (or
1 / freqs[i]); pairs are (2i, 2i+1) when `traditional`, else (i, i + dims/2);
out_first = x1 cos - x2 sin, out_second = x1 sin + x2 cos; elements past `dims` pass through.

Pinned by what the mathematics fixes (tests/test_oracle_rope.py): position 0 is the identity,
rotations preserve pair norms, R(p1) R(p2) = R(p1 + p2), the traditional and split layouts are
the same map under the interleaving permutation, dot products depend on the position
difference only, and a hand-computed 2-element case.  What only MLX could pin -- where it
rounds intermediates to the input dtype on its CPU path -- is "parity unpinned": angles and
products are float64 here (from the float32 angle MLX forms) and the result is rounded once.
"""
import numpy as np

from . import kv_oracle as O


def inv_freqs(dims, base=10000.0, freqs=None):
    half = dims // 2
    if freqs is not None:
        return (np.float32(1.0) / np.asarray(freqs, dtype=np.float32)).astype(np.float32)
    # formed in float64 and rounded once (MLX forms it in float32; its last bit is unpinned)
    step = np.log(np.float64(np.float32(base))) / np.float64(half)
    return np.exp(-np.arange(half, dtype=np.float64) * step).astype(np.float32)


def rope(x, dims, traditional=False, base=10000.0, scale=1.0, offset=0, freqs=None, dtype="float32"):
    """x [B, H, L, D] float32 holding values of `dtype` -> rotated, rounded once to `dtype`
    (dtype=None: float64, unrounded).  `offset`: int or [B] ints."""
    x = np.asarray(x)
    B, H, L, D = x.shape
    half = dims // 2
    inv = inv_freqs(dims, base, freqs)
    off = np.broadcast_to(np.asarray(offset, dtype=np.int64).reshape(-1), (B,)) if np.ndim(offset) else np.full((B,), int(offset))
    pos = (off[:, None] + np.arange(L)[None, :]).astype(np.float32) * np.float32(scale)   # [B, L] float32
    theta = (pos[:, :, None] * inv[None, None, :]).astype(np.float32).astype(np.float64)  # [B, L, half]
    cs, sn = np.cos(theta)[:, None], np.sin(theta)[:, None]                               # [B, 1, L, half]
    xf = x.astype(np.float64)
    out = xf.copy()
    if traditional:
        x1, x2 = xf[..., 0:dims:2], xf[..., 1:dims:2]
        out[..., 0:dims:2] = x1 * cs - x2 * sn
        out[..., 1:dims:2] = x1 * sn + x2 * cs
    else:
        x1, x2 = xf[..., :half], xf[..., half:dims]
        out[..., :half] = x1 * cs - x2 * sn
        out[..., half:dims] = x1 * sn + x2 * cs
    if dtype is None:
        return out
    return O.round_to(out.astype(np.float32), dtype)
