"""Pins the oracle's dropout pieces: the Philox4x32-10 noise stream against the Random123 library's
known-answer vectors and uniformity statistics, the mask / alpha-dropout arithmetic against closed
forms (lib/LuxLib/test/common_ops/dropout_tests.jl checks the same properties)."""
import numpy as np
import pytest

from oracle import luxlib_oracle as O


def test_philox_known_answers():
    # Random123 kat_vectors, philox4x32 with 10 rounds: (counter, key, expected)
    kat = [((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
           ((0xffffffff,) * 4, (0xffffffff,) * 2, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
           ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
            (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1))]
    for ctr, key, want in kat:
        got = O.philox4x32_10(np.array(ctr, np.uint32), key)
        assert tuple(int(v) for v in got) == want


def test_rand_uniform_stream_layout_and_statistics():
    u = O.rand_uniform(1 << 16, seed=1234, offset=0)
    assert u.dtype == np.float32 and u.min() >= 0 and u.max() < 1
    assert abs(u.mean() - 0.5) < 5e-3 and abs(u.var() - 1 / 12) < 2e-3
    hist = np.histogram(u, bins=16, range=(0, 1))[0]
    assert np.abs(hist - 4096).max() < 5 * 64          # 5 sigma of a binomial bin count
    # element e depends on (seed, offset + e // 4, e % 4) only
    np.testing.assert_array_equal(O.rand_uniform(100, 1234, 3), u[12:112])
    np.testing.assert_array_equal(O.rand_uniform(7, 1234, 0), u[:7])
    assert not np.array_equal(O.rand_uniform(64, 1235, 0), u[:64])
    # the first block of seed 0 is the first known-answer vector
    np.testing.assert_array_equal(O.rand_uniform(4, 0, 0),
                                  (np.array([0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8], np.uint32) >> 8) * np.float32(2.0 ** -24))
    ub = O.rand_uniform(1 << 14, 99, 0, bf16=True)
    np.testing.assert_array_equal(O.round_to_bf16(ub), ub)           # every value is a bf16 number
    assert ub.max() < 1 and abs(ub.mean() - 0.5) < 1e-2


@pytest.mark.parametrize("p", [0.0, 0.25, 0.5, 0.9])
def test_dropout_closed_form(p):
    rng = np.random.default_rng(5)
    x = rng.normal(size=(6, 5, 4)).astype(np.float32)
    invp = 1.0 / (1.0 - p)
    for dims in (None, (1,), (2, 3), (1, 3)):
        ms = O.dropout_shape(x.shape, dims)
        noise = rng.uniform(size=ms).astype(np.float32)
        y, m = O.dropout(noise, x, p, True, invp)
        assert m.shape == ms and set(np.unique(m)) <= {np.float32(0), np.float32(invp)}
        np.testing.assert_array_equal(m != 0, noise > np.float32(p))
        np.testing.assert_array_equal(y, x * m)
        # lib/LuxLib/test/common_ops/dropout_tests.jl: not training returns x untouched
        y2, m2 = O.dropout(noise, x, p, False, invp)
        assert y2 is x and m2 is x
        # a given mask is used as it is when update_mask is false
        y3, m3 = O.dropout(None, x, p, True, invp, mask=m, update_mask=False)
        assert m3 is m
        np.testing.assert_array_equal(y3, y)
        y4, m4 = O.dropout(noise, x, p, True, invp, mask=np.ones(ms, np.float32), update_mask=True)
        np.testing.assert_array_equal(y4, y)
    with pytest.raises(AssertionError):
        O.dropout(None, x, p, True, invp, mask=np.ones((6, 5, 3), np.float32), update_mask=False)


def test_alpha_dropout_closed_form_and_moments():
    p = 0.3
    alpha, A, B = O.alpha_dropout_coefficients(p)
    # the affine map keeps zero mean / unit variance of a standard normal input (Klambauer et al. 2017)
    keep = 1 - p
    mean = A * (keep * 0 + p * alpha) + B
    var = A * A * (keep * 1 + p * alpha ** 2 - (p * alpha) ** 2)
    assert abs(mean) < 1e-12 and abs(var - 1) < 1e-12
    rng = np.random.default_rng(6)
    x = rng.normal(size=(50, 40)).astype(np.float32)
    noise = rng.uniform(size=x.shape).astype(np.float32)
    y = O.alpha_dropout(noise, p, x, alpha, A, B)
    kept = noise > p
    np.testing.assert_allclose(y[kept], x[kept] * np.float32(A) + np.float32(B), rtol=1e-6)
    np.testing.assert_allclose(y[~kept], np.float32(alpha) * np.float32(A) + np.float32(B), rtol=1e-6)
    delta = rng.normal(size=x.shape).astype(np.float32)
    dx = O.alpha_dropout_pullback(noise, p, delta, A)
    np.testing.assert_allclose(dx, np.where(kept, delta * np.float32(A), 0), rtol=1e-6)
    # finite differences of <y, delta> in x
    h = 1e-3
    x64, d64, n64 = x.astype(np.float64), delta.astype(np.float64), noise.astype(np.float64)
    f = lambda xx: (O.alpha_dropout(n64, p, xx, alpha, A, B) * d64).sum()
    e = np.zeros_like(x64)
    e[3, 4] = h
    assert abs((f(x64 + e) - f(x64 - e)) / (2 * h) - O.alpha_dropout_pullback(n64, p, d64, A)[3, 4]) < 1e-8
