"""batchnorm forward (training / inference, running statistics) and pullback on the GPU
against the oracle (mirrors lib/LuxLib/test/normalization/batchnorm_tests.jl:58-178 and the
known-answer test test/core_layers/normalize_tests.jl:10-49 of the reference)."""
import numpy as np
import pytest

from oracle import luxlib_oracle as O
from tests.util import stable_seed, assert_close, dev, f64, host_inputs, rms

pytestmark = pytest.mark.gpu


def dx_scale(x, g, eps, delta, training=True, rvar=None):
    """Magnitude of the leading term delta * gamma / sqrt(var + eps) of the batchnorm input
    gradient: dx is a difference of terms of this size and can be far smaller than them."""
    x = f64(x)
    axes = tuple(i for i in range(x.ndim) if i != x.ndim - 2)
    var = x.var(axis=axes, keepdims=True) if training else f64(rvar).reshape(x.var(axis=axes, keepdims=True).shape)
    gp = (1.0 if g is None else f64(g).reshape(var.shape)) / np.sqrt(var + eps)
    return rms(f64(delta) * gp)


def test_reference_known_answer(gpu):
    x = np.array([[1.0, 3.0, 5.0], [2.0, 4.0, 6.0]], np.float32)
    d = lambda a: gpu.DeviceArray.from_numpy(np.asarray(a, np.float32))
    y, st = gpu.batchnorm(d(x), d(np.ones(2)), d(np.zeros(2)), d(np.zeros(2)), d(np.ones(2)), True, "identity", 0.1, 1e-5)
    np.testing.assert_allclose(y.to_numpy(), [[-1.22474, 0, 1.22474]] * 2, atol=1e-5)
    np.testing.assert_allclose(st["running_mean"].to_numpy(), [0.3, 0.4], rtol=1e-6)
    np.testing.assert_allclose(st["running_var"].to_numpy(), [1.3, 1.3], rtol=1e-6)
    yi, st2 = gpu.batchnorm(d(x), d(np.ones(2)), d(np.zeros(2)), st["running_mean"], st["running_var"], False,
                            "identity", 0.1, 1e-5)
    np.testing.assert_allclose(yi.to_numpy()[0, 0], (1 - 0.3) / np.sqrt(1.3 + 1e-5), rtol=1e-6)
    assert st2["running_mean"] is st["running_mean"]


SHAPES = [(4, 4, 6, 2), (8, 2), (3, 5, 4), (16, 16, 8, 4), (64, 3, 5), (32, 32, 16, 8), (40, 40, 3, 7)]


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("act", ["identity", "relu", "sigmoid_fast", "swish", "gelu", "tanh"])
@pytest.mark.parametrize("affine", [True, False])
@pytest.mark.parametrize("track", [True, False])
def test_training_forward_and_pullback(gpu, bn_path, dtype, act, affine, track):
    rng = np.random.default_rng(stable_seed(dtype, act, affine, track))
    for shape in SHAPES:
        Cc = shape[-2]
        x = O.generate_fixed_array(np.float32, shape) + rng.normal(size=shape) * 0.5
        g = rng.uniform(0.5, 1.5, Cc) if affine else None
        b = rng.normal(size=Cc) * 0.1 if affine else None
        rm = rng.normal(size=Cc) if track else None
        rv = rng.uniform(0.5, 2.0, Cc) if track else None
        delta = rng.normal(size=shape)
        eps = 1e-5 if dtype == "f32" else 1e-3
        for _ in range(50):
            xq, g, b, rm, rv, delta = host_inputs(dtype, x, g, b, rm, rv, delta)
            # keep the pre-activation away from relu's kink (a sign flip is a discontinuity)
            if act != "relu" or np.abs(O.batchnorm(f64(xq), f64(g), f64(b), None, None, True, "identity", 0.1, eps)[0]).min() > 1e-3:
                break
            x = x + rng.normal(size=shape) * 0.05
        x = xq
        args = [dev(gpu, a, dtype) for a in (x, g, b, rm, rv)]
        (y, st), back = gpu.pullback(gpu.batchnorm, *args, True, act, 0.1, eps)
        wy, wrm, wrv = O.batchnorm(f64(x), f64(g), f64(b), f64(rm), f64(rv), True, act, 0.1, eps)
        wy32 = O.batchnorm(x, g, b, rm, rv, True, act, 0.1, eps)[0]
        tag = f"{bn_path} {dtype} {act} {shape} affine={affine} track={track}"
        assert_close(y.to_numpy(), wy, dtype, tag + " y", want32=wy32)
        if track:
            assert_close(st["running_mean"].to_numpy(), wrm, dtype, tag + " running_mean")
            assert_close(st["running_var"].to_numpy(), wrv, dtype, tag + " running_var")
            # inputs are not modified
            np.testing.assert_array_equal(args[3].to_numpy(), rm)
        else:
            assert st["running_mean"] is None and st["running_var"] is None
        gx, gg, gb = back(dev(gpu, delta, dtype))
        wdx, wdg, wdb = O.batchnorm_pullback(f64(x), f64(g), f64(b), act, eps, f64(delta))
        w32 = O.batchnorm_pullback(x, g, b, act, np.float32(eps), delta)
        rel = None
        assert_close(gx.to_numpy(), wdx, dtype, tag + " dx", rel=rel, scale=dx_scale(x, g, eps, delta), want32=w32[0])
        if affine:
            assert_close(gg.to_numpy(), wdg, dtype, tag + " dgamma", rel=rel, scale=rms(delta), want32=w32[1])
            assert_close(gb.to_numpy(), wdb, dtype, tag + " dbeta", rel=rel, scale=rms(delta), want32=w32[2])
        else:
            assert gg is None and gb is None


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("act", ["identity", "relu", "swish"])
def test_inference_forward_and_pullback(gpu, dtype, act):
    rng = np.random.default_rng(3)
    for shape in [(4, 4, 6, 2), (8, 2), (16, 16, 8, 4)]:
        Cc = shape[-2]
        x, g, b, rm, rv, delta = host_inputs(dtype, rng.normal(size=shape), rng.uniform(0.5, 1.5, Cc),
                                             rng.normal(size=Cc), rng.normal(size=Cc) * 0.3, rng.uniform(0.5, 2, Cc),
                                             rng.normal(size=shape))
        eps = 1e-5 if dtype == "f32" else 1e-3
        args = [dev(gpu, a, dtype) for a in (x, g, b, rm, rv)]
        (y, st), back = gpu.pullback(gpu.batchnorm, *args, False, act, 0.1, eps)
        wy, _, _ = O.batchnorm(f64(x), f64(g), f64(b), f64(rm), f64(rv), False, act, 0.1, eps)
        assert_close(y.to_numpy(), wy, dtype, f"infer {act} {shape} y")
        assert st["running_mean"] is args[3]
        gx, gg, gb = back(dev(gpu, delta, dtype))
        wdx, wdg, wdb = O.batchnorm_pullback(f64(x), f64(g), f64(b), act, eps, f64(delta), training=False,
                                             rmean=f64(rm), rvar=f64(rv))
        rel = None
        assert_close(gx.to_numpy(), wdx, dtype, f"infer {act} {shape} dx", rel=rel,
                     scale=dx_scale(x, g, eps, delta, False, rv))
        assert_close(gg.to_numpy(), wdg, dtype, f"infer {act} {shape} dgamma", rel=rel)
        assert_close(gb.to_numpy(), wdb, dtype, f"infer {act} {shape} dbeta", rel=rel)
    # inference without running statistics falls back to batch statistics
    (x,) = host_inputs(dtype, rng.normal(size=(5, 4, 3)))
    y, st = gpu.batchnorm(dev(gpu, x, dtype), None, None, None, None, False, "identity", 0.1, 1e-3)
    assert_close(y.to_numpy(), O.batchnorm(f64(x), None, None, None, None, False, "identity", 0.1, 1e-3)[0], dtype, "no stats")


def test_large_mean_small_variance_is_stable(gpu):
    """single-pass statistics must not cancel catastrophically (mean 1e3, std 1e-1)."""
    rng = np.random.default_rng(9)
    x = (1000.0 + 0.1 * rng.normal(size=(64, 4, 32))).astype(np.float32)
    y, _ = gpu.batchnorm(gpu.DeviceArray.from_numpy(x), None, None, None, None, True, "identity", 0.1, 1e-5)
    want = O.batchnorm(f64(x), None, None, None, None, True, "identity", 0.1, 1e-5)[0]
    # the input itself carries ~6e-5/0.1 relative noise per element after centring
    assert_close(y.to_numpy(), want, "f32", "stability", rel=2e-3)
    assert abs(y.to_numpy().std() - 1) < 1e-2


def test_config2_full_size(gpu, bn_path):
    """benchmark configuration 2 at full size: x 32x32x64x128 ~ N(0.5, 2), train mode.  Checked against
    the fp64 oracle on a channel subset plus size-independent invariants (zero mean / unit
    variance per channel before the affine map; sum(dx) == 0 and sum(dx * xhat) == 0 per
    channel, the two conservation laws of the batchnorm pullback)."""
    rng = np.random.default_rng(1001)
    shape = (32, 32, 64, 128)
    x = (0.5 + 2.0 * rng.standard_normal(size=shape, dtype=np.float32))
    g = rng.uniform(0.5, 1.5, 64).astype(np.float32)
    b = (0.1 * rng.normal(size=64)).astype(np.float32)
    delta = rng.standard_normal(size=shape, dtype=np.float32)
    d = gpu.DeviceArray.from_numpy
    rm, rv = d(np.zeros(64, np.float32)), d(np.ones(64, np.float32))
    (y, st), back = gpu.pullback(gpu.batchnorm, d(x), d(g), d(b), rm, rv, True, "identity", 0.1, 1e-5)
    yh = y.to_numpy()
    xh = (yh - b.reshape(1, 1, 64, 1)) / g.reshape(1, 1, 64, 1)
    assert np.abs(xh.mean(axis=(0, 1, 3), dtype=np.float64)).max() < 1e-5
    assert np.abs(xh.var(axis=(0, 1, 3), dtype=np.float64) - 1).max() < 1e-4
    gx, gg, gb = back(d(delta))
    gxh = gx.to_numpy().astype(np.float64)
    assert np.abs(gxh.sum(axis=(0, 1, 3))).max() < 1e-2        # |sum| of 131072 terms of size ~0.5
    assert np.abs((gxh * xh).sum(axis=(0, 1, 3))).max() < 1e-2
    sub = slice(0, 64, 9)
    wy, wrm, wrv = O.batchnorm(f64(x[:, :, sub]), f64(g[sub]), f64(b[sub]), np.zeros(8), np.ones(8), True, "identity", 0.1, 1e-5)
    assert_close(yh[:, :, sub], wy, "f32", "config2 y")
    assert_close(st["running_mean"].to_numpy()[sub], wrm, "f32", "config2 running_mean")
    assert_close(st["running_var"].to_numpy()[sub], wrv, "f32", "config2 running_var")
    wdx, wdg, wdb = O.batchnorm_pullback(f64(x[:, :, sub]), f64(g[sub]), f64(b[sub]), "identity", 1e-5, f64(delta[:, :, sub]))
    assert_close(gxh[:, :, sub], wdx, "f32", "config2 dx")
    assert_close(gg.to_numpy()[sub], wdg, "f32", "config2 dgamma")
    assert_close(gb.to_numpy()[sub], wdb, "f32", "config2 dbeta")
