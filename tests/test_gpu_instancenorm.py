"""instancenorm forward + pullback (all training / running-statistics combinations) and
fast_activation on the GPU against the oracle
(mirrors lib/LuxLib/test/normalization/instancenorm_tests.jl and common_ops/activation_tests.jl)."""
import numpy as np
import pytest

from oracle import luxlib_oracle as O
from tests.util import stable_seed, assert_close, dev, f64, host_inputs, rms

pytestmark = pytest.mark.gpu

SHAPES = [(4, 4, 6, 2), (7, 3, 4), (3, 2, 2, 5, 3), (16, 16, 8, 3), (33, 65, 2), (96, 96, 4, 2)]


def dx_scale(x, g, eps, delta, var):
    gg = 1.0 if g is None else np.abs(f64(g)).max()
    return rms(f64(delta)) * gg / float(np.sqrt(var.min() + eps))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("act", ["identity", "relu", "swish"])
@pytest.mark.parametrize("affine", [True, False])
@pytest.mark.parametrize("mode", ["train_running", "train_plain", "test_running", "test_plain"])
def test_forward_and_pullback(gpu, dtype, act, affine, mode):
    rng = np.random.default_rng(stable_seed(dtype, act, affine, mode))
    training = mode.startswith("train")
    running = mode.endswith("running")
    for shape in SHAPES:
        Cc = shape[-2]
        eps = 1e-5 if dtype == "f32" else 1e-3
        x, g, b, rm, rv, delta = host_inputs(
            dtype, rng.normal(size=shape) * 1.5 + 0.3, rng.uniform(0.8, 1.2, Cc) if affine else None,
            rng.normal(size=Cc) * 0.05 if affine else None, rng.normal(size=Cc) * 0.3 if running else None,
            rng.uniform(0.5, 2.0, Cc) if running else None, rng.normal(size=shape))
        pre = O.instancenorm(f64(x), f64(g), f64(b), f64(rm), f64(rv), training, "identity", 0.1, eps)[0]
        if act == "relu":
            # a sign flip of a pre-activation next to relu's kink is a discontinuity, not a rounding
            # difference: no cotangent flows into those elements
            delta[np.abs(pre) < 1e-3] = 0
        tag = f"{mode} {dtype} {act} {shape} affine={affine}"
        args = [dev(gpu, a, dtype) for a in (x, g, b, rm, rv)]
        (y, stats), back = gpu.pullback(gpu.instancenorm, *args, training, act, 0.1, eps)
        wy, wrm, wrv = O.instancenorm(f64(x), f64(g), f64(b), f64(rm), f64(rv), training, act, 0.1, eps)
        assert_close(y.to_numpy(), wy, dtype, tag + " y",
                     want32=O.instancenorm(x, g, b, rm, rv, training, act, np.float32(0.1), np.float32(eps))[0])
        y2, stats2 = gpu.instancenorm(*args, training, act, 0.1, eps)
        np.testing.assert_array_equal(y2.to_numpy(), y.to_numpy())
        if running:
            for st in (stats, stats2):
                assert_close(st["running_mean"].to_numpy(), wrm, dtype, tag + " running_mean")
                assert_close(st["running_var"].to_numpy(), wrv, dtype, tag + " running_var")
            if not training:
                assert stats["running_mean"] is args[3] and stats["running_var"] is args[4]
        else:
            assert stats["running_mean"] is None and stats["running_var"] is None
        gx, gg, gb = back(dev(gpu, delta, dtype))
        kw = dict(training=training, rmean=f64(rm), rvar=f64(rv))
        wdx, wdg, wdb = O.instancenorm_pullback(f64(x), f64(g), f64(b), act, eps, f64(delta), **kw)
        w32 = O.instancenorm_pullback(x, g, b, act, np.float32(eps), delta, training=training, rmean=rm, rvar=rv)
        var = f64(rv) if (running and not training) else f64(x).var(axis=tuple(range(len(shape) - 2)))
        rel = None
        assert_close(gx.to_numpy(), wdx, dtype, tag + " dx", rel=rel, scale=dx_scale(x, g, eps, delta, var), want32=w32[0])
        if affine:
            sc = rms(delta) * max(1.0, float(np.abs(pre).max()))
            assert_close(gg.to_numpy(), wdg, dtype, tag + " dgamma", rel=rel, scale=sc, want32=w32[1])
            assert_close(gb.to_numpy(), wdb, dtype, tag + " dbeta", rel=rel, scale=rms(delta), want32=w32[2])
        else:
            assert gg is None and gb is None


def test_argument_errors(gpu):
    d = lambda *s: gpu.DeviceArray.from_numpy(np.ones(s, np.float32))
    with pytest.raises(AssertionError):
        gpu.instancenorm(d(4, 3), None, None, None, None, True)
    with pytest.raises(gpu.ArgumentError):
        gpu.instancenorm(d(4, 3, 2), d(4), d(4), None, None, True)
    with pytest.raises(gpu.ArgumentError):
        gpu.instancenorm(d(4, 3, 2), None, None, d(3), None, True)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("act", ["identity", "relu", "tanh", "sigmoid_fast", "swish", "gelu", "softplus"])
def test_fast_activation(gpu, dtype, act):
    """fast_activation, fast_activation!! and the activation pullback
    (lib/LuxLib/test/common_ops/activation_tests.jl:1-60)."""
    rng = np.random.default_rng(stable_seed(dtype, act))
    for shape in [(4,), (5, 3), (3, 4, 2, 2), (1000, 33), (0, 4)]:
        x, delta = host_inputs(dtype, rng.normal(size=shape) * 2, rng.normal(size=shape))
        if act == "relu":
            x[np.abs(x) < 1e-3] = 0.5
        y, back = gpu.pullback(gpu.fast_activation, act, dev(gpu, x, dtype))
        want = O.act_value(act, f64(x))
        assert_close(y.to_numpy(), want, dtype, f"{act} {shape} y")
        np.testing.assert_array_equal(gpu.fast_activation(act, dev(gpu, x, dtype)).to_numpy(), y.to_numpy())
        xin = dev(gpu, x, dtype)
        assert gpu.fast_activation_inplace(act, xin) is xin
        np.testing.assert_array_equal(xin.to_numpy(), y.to_numpy())
        (dx,) = back(dev(gpu, delta, dtype))
        yq = f64(O.round_to_bf16(want.astype(np.float32))) if dtype == "bf16" else want
        assert_close(dx.to_numpy(), O.grad_activation(f64(delta), yq, act, f64(x)), dtype, f"{act} {shape} dx",
                     rel=None)


def test_separate_running_statistics_call_matches_the_fused_forward(gpu):
    """luxhip_groupnorm_fwd with G = C followed by luxhip_instancenorm_running_stats (the two-call form of the C
    ABI) gives the running statistics that luxhip_instancenorm_fwd computes in its own launch."""
    rng = np.random.default_rng(77)
    shape = (9, 7, 12, 5)
    I, Cc, N = 63, 12, 5
    x = rng.normal(size=shape).astype(np.float32) * 2 + 0.3
    rm, rv = rng.normal(size=Cc).astype(np.float32), rng.uniform(0.5, 2.0, Cc).astype(np.float32)
    d = gpu.DeviceArray.from_numpy
    dx_, drm, drv = d(x), d(rm), d(rv)
    (y, stats) = gpu.instancenorm(dx_, None, None, drm, drv, True, "identity", 0.2, 1e-5)
    y2 = gpu.DeviceArray(shape, "f32")
    sm, si = gpu.StatArray(Cc * N), gpu.StatArray(Cc * N)
    s = gpu.current_stream()
    gpu._lib.call("luxhip_groupnorm_fwd", s, 0, 0, I, Cc, Cc, N, dx_.ptr, None, None, 1e-5, y2.ptr, sm.ptr, si.ptr)
    rm2, rv2 = gpu.DeviceArray((Cc,), "f32"), gpu.DeviceArray((Cc,), "f32")
    gpu._lib.call("luxhip_instancenorm_running_stats", s, 0, I, Cc, N, sm.ptr, si.ptr, 1e-5, 0.2, drm.ptr, drv.ptr, rm2.ptr, rv2.ptr)
    np.testing.assert_array_equal(y2.to_numpy(), y.to_numpy())
    np.testing.assert_allclose(rm2.to_numpy(), stats["running_mean"].to_numpy(), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(rv2.to_numpy(), stats["running_var"].to_numpy(), rtol=1e-6)
    want = O.instancenorm(x.astype(np.float64), None, None, rm.astype(np.float64), rv.astype(np.float64), True, "identity", 0.2, 1e-5)
    np.testing.assert_allclose(rm2.to_numpy(), want[1], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(rv2.to_numpy(), want[2], rtol=1e-5)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_running_variance_of_a_constant_channel(gpu, dtype):
    """A channel whose slices are constant (variance 0, far below eps) and one with a variance of 1e-9: the
    running variance moves towards that variance, never below (1 - momentum) * running_var."""
    rng = np.random.default_rng(5)
    shape = (16, 8, 3, 4)
    x = rng.normal(size=shape).astype(np.float32)
    x[:, :, 0, :] = 3.0
    x[:, :, 1, :] = 2.0 + (3e-5 * rng.normal(size=(16, 8, 4))).astype(np.float32)
    (x,) = host_inputs(dtype, x)
    rm, rv = np.zeros(3, np.float32), np.ones(3, np.float32)
    (_, stats) = gpu.instancenorm(dev(gpu, x, dtype), None, None, dev(gpu, rm, dtype), dev(gpu, rv, dtype), True, "identity", 0.1, 1e-5)
    want = O.instancenorm(f64(x), None, None, f64(rm), f64(rv), True, "identity", 0.1, 1e-5)
    got = stats["running_var"].to_numpy().astype(np.float64)
    assert got[0] == pytest.approx(0.9, rel=1e-2 if dtype == "bf16" else 1e-6) and (got >= 0.9 * (1 - 4e-3)).all()
    assert_close(got, want[2], dtype, "running_var")
