"""Tensors just under the library's limit of 2^31 elements (the largest the kernels' 31-bit
element indexing admits): the first, a middle and the last sample are compared with the oracle, and
the parameter gradients, which sum over the whole tensor, with what the input stream fixes.

The inputs are drawn on the device from the Philox stream (host memory never holds a whole
tensor); the oracle's restatement of that stream regenerates any slice of them on the host.
Element e of a stream is lane e % 4 of counter block offset + e // 4, so a sample of a
multiple of four elements starts at a whole block."""
import numpy as np
import pytest

from oracle import luxlib_oracle as O
from tests.util import assert_close, dev, f64

pytestmark = pytest.mark.gpu

SHAPE = (1 << 16, 8, 4095)            # 2^31 - 2^19 elements
PER = SHAPE[0] * SHAPE[1]             # elements per sample
SAMPLES = (0, 2047, 4094)


def stream(gpu, seed, dtype):
    a, _ = gpu.rand_uniform(gpu.PhiloxRNG(seed, 0), SHAPE, dtype)
    return a


def device_sample(gpu, a, n):
    """Sample n of a device tensor as a view (shape (I, C, 1))."""
    return gpu.DeviceArray(SHAPE[:2] + (1,), a.dtype, ptr=a.ptr + n * PER * a.itemsize, base=a)


def host_sample(seed, n, dtype):
    """Sample n of the stream tensor, regenerated on the host."""
    v = O.rand_uniform(PER, seed, n * PER // 4, bf16=(dtype == "bf16"))
    return v.reshape(SHAPE[:2] + (1,), order="F")


def stream_elements(seed, idx, dtype):
    """Elements of the stream at arbitrary flat indices."""
    idx = np.asarray(idx, dtype=np.uint64)
    counter = np.zeros((idx.size, 4), np.uint32)
    blk = idx // np.uint64(4)
    counter[:, 0] = (blk & np.uint64(0xFFFFFFFF)).astype(np.uint32)
    counter[:, 1] = (blk >> np.uint64(32)).astype(np.uint32)
    words = O.philox4x32_10(counter, (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF))
    u = words[np.arange(idx.size), (idx % np.uint64(4)).astype(np.int64)]
    if dtype == "bf16":
        return (u >> np.uint32(24)).astype(np.float64) * 2.0 ** -8
    return (u >> np.uint32(8)).astype(np.float64) * 2.0 ** -24


def expected_sum_above(t, dtype):
    """E[u * (u > t)] for one value u of the stream (t a multiple of 2^-8)."""
    if dtype == "bf16":                                  # u = k / 256, k uniform in 0..255
        k = np.arange(256)
        return float(np.sum(k[k > t * 256]) / 256.0 / 256.0)
    return (1.0 - t * t) / 2.0                           # u = j / 2^24: continuous to 2^-24


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_bias_activation_near_the_element_limit(gpu, dtype):
    x = stream(gpu, 21, dtype)
    bias = -np.arange(8, dtype=np.float32) / 16.0        # relu cuts the stream at t = c / 16
    b = dev(gpu, bias, dtype)
    y, back = gpu.pullback(gpu.bias_activation, "relu", x, b)
    for n in SAMPLES:
        xs = host_sample(21, n, dtype)
        want = O.bias_activation("relu", f64(xs), f64(bias))
        assert_close(device_sample(gpu, y, n).to_numpy(), want, dtype, f"y, sample {n}")
    dx, db = back(x)                                     # the cotangent is the stream itself
    for n in SAMPLES:
        xs = host_sample(21, n, dtype)
        _, wdx, _ = O.bias_activation_pullback("relu", f64(xs), f64(bias), f64(xs))
        assert_close(device_sample(gpu, dx, n).to_numpy(), wdx, dtype, f"dx, sample {n}")
    # db[c] = sum of u (u > c/16) over SHAPE[0] * SHAPE[2] draws: the mean is known, the spread of
    # the sum is 3e-5 of it, so every element must have been counted exactly once
    count = SHAPE[0] * SHAPE[2]
    want_db = np.array([count * expected_sum_above(c / 16.0, dtype) for c in range(8)])
    got = db.to_numpy().astype(np.float64)
    np.testing.assert_allclose(got, want_db, rtol=3e-4 if dtype == "f32" else 1e-2)


def test_groupnorm_near_the_element_limit(gpu):
    dtype = "bf16"
    rng = np.random.default_rng(3)
    x = stream(gpu, 31, dtype)
    gamma = O.round_to_bf16(rng.uniform(0.5, 1.5, size=8).astype(np.float32))
    beta = O.round_to_bf16(rng.normal(size=8).astype(np.float32))
    g, b = dev(gpu, gamma, dtype), dev(gpu, beta, dtype)
    eps = 1e-3
    y, back = gpu.pullback(gpu.groupnorm, x, g, b, 4, "identity", eps)
    delta = stream(gpu, 32, dtype)
    dx, dg, db = back(delta)
    for n in SAMPLES:
        xs, ds = host_sample(31, n, dtype), host_sample(32, n, dtype)
        want = O.groupnorm(f64(xs), f64(gamma), f64(beta), 4, "identity", eps)
        assert_close(device_sample(gpu, y, n).to_numpy(), want, dtype, f"y, sample {n}")
        wdx = O.groupnorm_pullback(f64(xs), f64(gamma), f64(beta), 4, "identity", eps, f64(ds))[0]
        assert_close(device_sample(gpu, dx, n).to_numpy(), wdx, dtype, f"dx, sample {n}", scale=float(np.abs(gamma).max()) * 2.0)
    # dbeta[c] = the sum of the cotangent stream over the channel: mean 127.5/256 per draw
    count = SHAPE[0] * SHAPE[2]
    np.testing.assert_allclose(db.to_numpy().astype(np.float64), np.full(8, count * 127.5 / 256.0), rtol=1e-2)
    assert np.all(np.isfinite(dg.to_numpy()))


def test_layernorm_near_the_element_limit(gpu):
    dtype = "bf16"
    rng = np.random.default_rng(4)
    x = stream(gpu, 41, dtype)
    pshape = SHAPE[:2] + (1,)
    gamma = O.round_to_bf16(rng.uniform(0.5, 1.5, size=pshape).astype(np.float32))
    beta = O.round_to_bf16(rng.normal(size=pshape).astype(np.float32))
    g, b = dev(gpu, gamma, dtype), dev(gpu, beta, dtype)
    eps = 1e-3
    y, back = gpu.pullback(gpu.layernorm, x, g, b, "identity", epsilon=eps)
    delta = stream(gpu, 42, dtype)
    dx, dg, db = back(delta)
    for n in SAMPLES:
        xs, ds = host_sample(41, n, dtype), host_sample(42, n, dtype)
        want = O.layernorm(f64(xs), f64(gamma), f64(beta), "identity", None, eps)
        assert_close(device_sample(gpu, y, n).to_numpy(), want, dtype, f"y, sample {n}")
        wdx = O.layernorm_pullback(f64(xs), f64(gamma), f64(beta), "identity", None, eps, f64(ds))[0]
        assert_close(device_sample(gpu, dx, n).to_numpy(), wdx, dtype, f"dx, sample {n}", scale=2.0)
    # dbeta at a few positions = the sum over all samples of the cotangent there, regenerated exactly
    got = db.to_numpy().reshape(-1, order="F").astype(np.float64)
    for p in (0, 1, 65535, 65536, 300001, PER - 1):
        idx = np.arange(SHAPE[2], dtype=np.uint64) * np.uint64(PER) + np.uint64(p)
        want = stream_elements(42, idx, dtype).sum()
        assert abs(got[p] - want) <= 1e-2 * want, f"dbeta[{p}]: got {got[p]} want {want}"


def test_batchnorm_near_the_element_limit(gpu):
    """Training-mode batchnorm: the statistics run over 2.7e8 draws per channel, so they equal the
    stream's own mean 1/2 - 2^-25 and variance 1/12 to 1e-4; samples are checked against the
    normalisation with those values, at rel 1e-3."""
    dtype = "f32"
    rng = np.random.default_rng(6)
    x = stream(gpu, 61, dtype)
    gamma = rng.uniform(0.5, 1.5, size=8).astype(np.float32)
    beta = rng.normal(size=8).astype(np.float32)
    rm0, rv0 = rng.normal(size=8).astype(np.float32), rng.uniform(0.5, 2.0, size=8).astype(np.float32)
    eps, mom = 1e-5, 0.1
    (y, stats), back = gpu.pullback(gpu.batchnorm, x, dev(gpu, gamma, dtype), dev(gpu, beta, dtype), dev(gpu, rm0, dtype),
                                    dev(gpu, rv0, dtype), True, "identity", mom, eps)
    mu, var = 0.5 - 2.0 ** -25, 1.0 / 12.0
    np.testing.assert_allclose(stats["running_mean"].to_numpy(), (1 - mom) * rm0 + mom * mu, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(stats["running_var"].to_numpy(), (1 - mom) * rv0 + mom * var, rtol=1e-4)
    invstd = 1.0 / np.sqrt(var + eps)
    delta = stream(gpu, 62, dtype)
    dx, dg, db = back(delta)
    gv, bv = f64(gamma).reshape(1, 8, 1), f64(beta).reshape(1, 8, 1)
    for n in SAMPLES:
        xs, ds = f64(host_sample(61, n, dtype)), f64(host_sample(62, n, dtype))
        xhat = (xs - mu) * invstd
        assert_close(device_sample(gpu, y, n).to_numpy(), xhat * gv + bv, dtype, f"y, sample {n}", rel=1e-3)
        # mean(dy) = 1/2 and mean(dy xhat) = 0 for an independent cotangent stream
        assert_close(device_sample(gpu, dx, n).to_numpy(), gv * invstd * (ds - 0.5), dtype, f"dx, sample {n}", rel=1e-3)
    count = SHAPE[0] * SHAPE[2]
    np.testing.assert_allclose(db.to_numpy().astype(np.float64), np.full(8, count * (0.5 - 2.0 ** -25)), rtol=3e-4)
    assert np.all(np.abs(dg.to_numpy()) < 1e-3 * count)       # sum of dy * xhat: zero mean, spread ~ sqrt(count / 12)


def test_dropout_near_the_element_limit(gpu):
    dtype = "bf16"
    x = stream(gpu, 51, dtype)
    y, mask, rng2 = gpu.dropout(gpu.PhiloxRNG(52, 0), x, 0.25, True, 1.0 / 0.75)
    assert rng2.offset == (x.size + 3) // 4
    for n in SAMPLES:
        xs = host_sample(51, n, dtype)
        noise = host_sample(52, n, dtype)
        wy, wm = O.dropout(noise, xs, np.float32(0.25), True, np.float32(1.0 / 0.75))
        assert_close(device_sample(gpu, mask, n).to_numpy(), O.round_to_bf16(wm.astype(np.float32)), dtype, f"mask, sample {n}")
        assert_close(device_sample(gpu, y, n).to_numpy(), wy, dtype, f"y, sample {n}")


def test_two_to_the_31_elements_are_refused(gpu):
    x = gpu.DeviceArray((1 << 16, 8, 4096), "bf16")
    with pytest.raises(gpu.Unsupported):
        gpu.bias_activation("relu", x, None)
    with pytest.raises(gpu.Unsupported):
        gpu.groupnorm(x, None, None, 4)
    with pytest.raises(gpu.Unsupported):
        gpu.layernorm(x, None, None)
    with pytest.raises(gpu.Unsupported):
        gpu.batchnorm(x, None, None, None, None, True)
    # the fused dropout forward indexes with 64 bits and takes the tensor; the broadcast product
    # of the pullback does not
    y, mask, _ = gpu.dropout(gpu.PhiloxRNG(71, 0), x, 0.5, True, 2.0)
    noise = host_sample(71, 4095, "bf16")
    assert_close(device_sample(gpu, mask, 4095).to_numpy(), np.where(noise > 0.5, 2.0, 0.0), "bf16", "mask of the last sample")
    with pytest.raises(gpu.Unsupported):
        gpu.dropout_dot_mul(x, mask)
