"""The rotary-embedding restatement (oracle/rope.py) against what the mathematics fixes:
hand-computed small cases, invariants and identities chosen so that a wrong sign, a wrong
pairing or a wrong frequency exponent fails at least one of them."""
import numpy as np
import pytest

from oracle import rope as R


def rnd(shape, seed=0):
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)


def test_hand_computed_pairs_and_frequencies():
    # split layout, dims 4: pairs (0,2) and (1,3); pair i turns by p * base^(-2i/dims)
    x = np.zeros((1, 1, 1, 4), np.float32)
    x[..., 0] = 1.0
    out = R.rope(x, 4, traditional=False, base=10000.0, offset=1, dtype=None)[0, 0, 0]
    assert np.allclose(out, [np.cos(1.0), 0.0, np.sin(1.0), 0.0], atol=1e-7)   # +sin in the second slot
    x[...] = 0.0
    x[..., 1] = 1.0
    out = R.rope(x, 4, traditional=False, base=10000.0, offset=1, dtype=None)[0, 0, 0]
    th1 = 10000.0 ** (-2.0 / 4.0)                                              # 0.01
    assert np.allclose(out, [0.0, np.cos(th1), 0.0, np.sin(th1)], atol=1e-7)
    # second element of a pair: (x1, x2) = (0, 1) -> (-sin, cos)
    x[...] = 0.0
    x[..., 2] = 1.0
    out = R.rope(x, 4, traditional=False, base=10000.0, offset=1, dtype=None)[0, 0, 0]
    assert np.allclose(out, [-np.sin(1.0), 0.0, np.cos(1.0), 0.0], atol=1e-7)
    # traditional layout: pairs (0,1) and (2,3)
    x[...] = 0.0
    x[..., 2] = 1.0
    out = R.rope(x, 4, traditional=True, base=10000.0, offset=1, dtype=None)[0, 0, 0]
    assert np.allclose(out, [0.0, 0.0, np.cos(th1), np.sin(th1)], atol=1e-7)
    # position scale multiplies the position
    x[...] = 0.0
    x[..., 0] = 1.0
    out = R.rope(x, 4, scale=0.25, offset=2, dtype=None)[0, 0, 0]
    assert np.allclose(out, [np.cos(0.5), 0.0, np.sin(0.5), 0.0], atol=1e-7)


def test_inverse_frequencies_closed_form():
    for dims, base in ((64, 10000.0), (128, 500000.0), (32, 1e6)):
        inv = R.inv_freqs(dims, base)
        want = base ** (-2.0 * np.arange(dims // 2) / dims)
        assert np.allclose(inv, want, rtol=2e-6)
    f = np.array([1.0, 2.0, 8.0, 100.0], np.float32)
    assert np.allclose(R.inv_freqs(8, freqs=f), 1.0 / f, rtol=1e-7)


@pytest.mark.parametrize("traditional", [False, True])
def test_position_zero_is_identity_and_tail_passes_through(traditional):
    x = rnd((2, 3, 1, 64))
    out = R.rope(x, 48, traditional=traditional, offset=0)
    assert np.array_equal(out, x)
    out = R.rope(x, 48, traditional=traditional, offset=5)
    assert np.array_equal(out[..., 48:], x[..., 48:])
    assert not np.allclose(out[..., :48], x[..., :48])


@pytest.mark.parametrize("traditional", [False, True])
def test_rotation_preserves_pair_norms_and_composes(traditional):
    x = rnd((2, 2, 5, 32), 1)
    out = R.rope(x, 32, traditional=traditional, offset=11, dtype=None)
    if traditional:
        n_in = x[..., 0::2].astype(np.float64) ** 2 + x[..., 1::2].astype(np.float64) ** 2
        n_out = out[..., 0::2] ** 2 + out[..., 1::2] ** 2
    else:
        n_in = x[..., :16].astype(np.float64) ** 2 + x[..., 16:].astype(np.float64) ** 2
        n_out = out[..., :16] ** 2 + out[..., 16:] ** 2
    assert np.allclose(n_in, n_out, rtol=1e-12)
    # R(a) R(b) = R(a + b): rotate single rows so that every row sits at the same position
    x1 = x[:, :, :1]
    ab = R.rope(R.rope(x1, 32, traditional=traditional, offset=3, dtype=None), 32, traditional=traditional, offset=5, dtype=None)
    direct = R.rope(x1, 32, traditional=traditional, offset=8, dtype=None)
    assert np.allclose(ab, direct, atol=1e-5)


def test_layouts_agree_under_the_interleaving_permutation():
    x = rnd((1, 2, 4, 16), 2)
    perm = np.empty_like(x)
    perm[..., 0::2] = x[..., :8]
    perm[..., 1::2] = x[..., 8:]
    a = R.rope(x, 16, traditional=False, offset=7, dtype=None)
    b = R.rope(perm, 16, traditional=True, offset=7, dtype=None)
    assert np.allclose(a[..., :8], b[..., 0::2], atol=1e-12)
    assert np.allclose(a[..., 8:], b[..., 1::2], atol=1e-12)


def test_scores_depend_on_the_position_difference_only():
    q, k = rnd((1, 1, 1, 64), 3), rnd((1, 1, 1, 64), 4)
    def score(m, n):
        return float((R.rope(q, 64, offset=m, dtype=None) * R.rope(k, 64, offset=n, dtype=None)).sum())
    assert abs(score(7, 3) - score(14, 10)) < 1e-4
    assert abs(score(7, 3) - score(7, 4)) > 1e-3


def test_row_positions_and_batch_offsets():
    x = rnd((3, 2, 4, 32), 5)
    whole = R.rope(x, 32, offset=10)
    for l in range(4):
        assert np.array_equal(whole[:, :, l:l + 1], R.rope(x[:, :, l:l + 1], 32, offset=10 + l))
    offs = np.array([0, 7, 100])
    batched = R.rope(x, 32, offset=offs)
    for b in range(3):
        assert np.array_equal(batched[b:b + 1], R.rope(x[b:b + 1], 32, offset=int(offs[b])))


def test_freqs_replace_the_base():
    x = rnd((1, 1, 3, 16), 6)
    f = (1.0 / R.inv_freqs(16, 10000.0)).astype(np.float32)
    a = R.rope(x, 16, offset=9, dtype=None)
    b = R.rope(x, 16, offset=9, freqs=f, base=123.0, dtype=None)
    assert np.allclose(a, b, atol=1e-5)


def test_result_is_rounded_to_the_dtype():
    from oracle import kv_oracle as O
    x = O.round_to(rnd((1, 1, 2, 8), 7), "bfloat16")
    out = R.rope(x, 8, offset=3, dtype="bfloat16")
    assert np.array_equal(out, O.round_to(out, "bfloat16"))
    out16 = R.rope(O.round_to(x, "float16"), 8, offset=3, dtype="float16")
    assert np.array_equal(out16, O.round_to(out16, "float16"))
