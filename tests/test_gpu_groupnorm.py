"""groupnorm forward + pullback on the GPU against the oracle
(mirrors lib/LuxLib/test/normalization/groupnorm_tests.jl:48-115 of the reference)."""
import numpy as np
import pytest

from oracle import luxlib_oracle as O
from tests.util import stable_seed, assert_close, dev, f64, host_inputs, rms

pytestmark = pytest.mark.gpu

CASES = [((6, 2), 2), ((4, 4, 6, 2), 3), ((2, 2, 6, 2), 2), ((5, 12, 3), 4), ((16, 16, 8, 3), 2), ((64, 6, 2), 3),
         ((32, 32, 12, 2), 1), ((8, 8, 16, 2), 16), ((96, 96, 4, 2), 1),
         # slices that two workgroups share (fp32: 19200 elements per slice, bf16: 65536)
         ((40, 40, 24, 2), 2), ((64, 64, 32, 2), 2),
         # 72 channels per group: more than the kernels' LDS tables of channel parameters hold
         ((4, 4, 144, 2), 2)]


@pytest.fixture(params=["wait", "no_wait"])
def gn_path(gpu, request):
    """Slices shared by two workgroups exchange partial statistics with a bounded wait; "no_wait"
    cuts the wait to zero polls, so every workgroup recomputes its peer's share itself."""
    gpu.set_option("bn_spin_limit", 0 if request.param == "no_wait" else 1 << 22)
    yield request.param
    gpu.set_option("bn_spin_limit", 1 << 22)


def dx_scale(x, g, groups, eps, delta):
    xv, Cg = O._gn_view(f64(x), groups)
    axes = tuple(range(xv.ndim - 2))
    var = xv.var(axis=axes, keepdims=True)
    gg = 1.0 if g is None else np.abs(f64(g)).max()
    return rms(f64(delta)) * gg / float(np.sqrt(var.min() + eps))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("act", ["identity", "relu", "sigmoid_fast", "swish", "gelu"])
@pytest.mark.parametrize("affine", [True, False])
def test_forward_and_pullback(gpu, gn_path, dtype, act, affine):
    rng = np.random.default_rng(stable_seed(dtype, act, affine))
    for shape, groups in CASES:
        Cc = shape[-2]
        eps = 1e-5 if dtype == "f32" else 1e-3
        for _ in range(50):
            x, g, b, delta = host_inputs(dtype, rng.normal(size=shape), rng.uniform(0.8, 1.2, Cc) if affine else None,
                                         rng.normal(size=Cc) * 0.05 if affine else None, rng.normal(size=shape))
            # keep the pre-activation away from relu's kink: a sign flip there is a discontinuity,
            # not a rounding difference
            if act != "relu" or np.abs(O.groupnorm(f64(x), f64(g), f64(b), groups, "identity", eps)).min() > 1e-3:
                break
        tag = f"{gn_path} {dtype} {act} {shape} G={groups} affine={affine}"
        y, back = gpu.pullback(gpu.groupnorm, dev(gpu, x, dtype), dev(gpu, g, dtype), dev(gpu, b, dtype), groups, act, eps)
        wy = O.groupnorm(f64(x), f64(g), f64(b), groups, act, eps)
        assert_close(y.to_numpy(), wy, dtype, tag + " y", want32=O.groupnorm(x, g, b, groups, act, np.float32(eps)))
        y2 = gpu.groupnorm(dev(gpu, x, dtype), dev(gpu, g, dtype), dev(gpu, b, dtype), groups, act, eps)
        np.testing.assert_array_equal(y2.to_numpy(), y.to_numpy())
        gx, gg, gb = back(dev(gpu, delta, dtype))
        wdx, wdg, wdb = O.groupnorm_pullback(f64(x), f64(g), f64(b), groups, act, eps, f64(delta))
        w32 = O.groupnorm_pullback(x, g, b, groups, act, np.float32(eps), delta)
        rel = None
        assert_close(gx.to_numpy(), wdx, dtype, tag + " dx", rel=rel, scale=dx_scale(x, g, groups, eps, delta), want32=w32[0])
        if affine:
            assert_close(gg.to_numpy(), wdg, dtype, tag + " dgamma", rel=rel, scale=rms(delta), want32=w32[1])
            assert_close(gb.to_numpy(), wdb, dtype, tag + " dbeta", rel=rel, scale=rms(delta), want32=w32[2])
        else:
            assert gg is None and gb is None


def test_argument_errors(gpu):
    d = lambda *s: gpu.DeviceArray.from_numpy(np.ones(s, np.float32))
    with pytest.raises(gpu.ArgumentError):
        gpu.groupnorm(d(4, 6, 2), d(6), d(6), 4)
    with pytest.raises(gpu.ArgumentError):
        gpu.groupnorm(d(4, 6, 2), d(5), d(5), 2)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_config3_full_size(gpu, gn_path, dtype):
    """benchmark configuration 3 at full size: x 64x64x256x16, 32 groups, swish.  Oracle comparison on
    two samples; whole-tensor invariants: per-(group, sample) slices of dx sum to zero and are
    orthogonal to xhat (the two conservation laws of the normalisation pullback)."""
    rng = np.random.default_rng(1002)
    shape, G = (64, 64, 256, 16), 32
    x = rng.standard_normal(size=shape, dtype=np.float32)
    g = rng.uniform(0.8, 1.2, 256).astype(np.float32)
    b = (0.05 * rng.standard_normal(256)).astype(np.float32)
    delta = rng.standard_normal(size=shape, dtype=np.float32)
    x, g, b, delta = host_inputs(dtype, x, g, b, delta)
    eps = 1e-5
    y, back = gpu.pullback(gpu.groupnorm, dev(gpu, x, dtype), dev(gpu, g, dtype), dev(gpu, b, dtype), G, "swish", eps)
    gx, gg, gb = back(dev(gpu, delta, dtype))
    yh, gxh = y.to_numpy(), gx.to_numpy().astype(np.float64)
    sub = [0, 11]
    wy = O.groupnorm(f64(x[..., sub]), f64(g), f64(b), G, "swish", eps)
    assert_close(yh[..., sub], wy, dtype, "config3 y")
    wdx, _, _ = O.groupnorm_pullback(f64(x[..., sub]), f64(g), f64(b), G, "swish", eps, f64(delta[..., sub]))
    assert_close(gxh[..., sub], wdx, dtype, "config3 dx")
    # conservation laws on every slice
    xs = f64(x).reshape(64 * 64 * 8, 32, 16, order="F")
    ds = gxh.reshape(64 * 64 * 8, 32, 16, order="F")
    xh = (xs - xs.mean(axis=0)) / np.sqrt(xs.var(axis=0) + eps)
    tol = 1e-2 if dtype == "f32" else 3.0
    assert np.abs(ds.sum(axis=0)).max() < tol
    assert np.abs((ds * xh).sum(axis=0)).max() < tol
    # parameter gradients against an fp64 reduction of the full tensors
    _, wdg, wdb = O.groupnorm_pullback(f64(x), f64(g), f64(b), G, "swish", eps, f64(delta))
    assert_close(gg.to_numpy(), wdg, dtype, "config3 dgamma", scale=rms(delta) * 10)
    assert_close(gb.to_numpy(), wdb, dtype, "config3 dbeta", scale=rms(delta) * 10)


@pytest.mark.parametrize("scale", [1e6, 3e-6, 1e-20, "uneven"])
@pytest.mark.parametrize("act", ["identity", "swish"])
def test_pullback_with_scaled_cotangents_bf16(gpu, act, scale):
    """bf16 cotangents far outside and far below the fp16 range, and cotangents whose magnitude differs by 1e4 between
    the halves of a slice: the pullback keeps an intermediate as scaled fp16 in registers where it can, and must neither
    saturate large values nor lose small ones (the result scales with the cotangent)."""
    rng = np.random.default_rng(99)
    shape, groups, eps = (16, 16, 8, 3), 2, 1e-3
    if scale == "uneven":
        factor = np.where(np.arange(8) % 4 >= 2, 1e4, 1.0).reshape(1, 1, 8, 1)
    else:
        factor = scale
    x, g, b, delta = host_inputs("bf16", rng.normal(size=shape), rng.uniform(0.8, 1.2, 8), rng.normal(size=8) * 0.05,
                                 rng.normal(size=shape) * factor)
    y, back = gpu.pullback(gpu.groupnorm, dev(gpu, x, "bf16"), dev(gpu, g, "bf16"), dev(gpu, b, "bf16"), groups, act, eps)
    gx, gg, gb = back(dev(gpu, delta, "bf16"))
    wdx, wdg, wdb = O.groupnorm_pullback(f64(x), f64(g), f64(b), groups, act, eps, f64(delta))
    tag = f"bf16 {act} cotangent x {scale}"
    assert_close(gx.to_numpy(), wdx, "bf16", tag + " dx", rel=1e-2, scale=dx_scale(x, g, groups, eps, delta))
    assert_close(gg.to_numpy(), wdg, "bf16", tag + " dgamma", rel=1e-2, scale=rms(delta))
    assert_close(gb.to_numpy(), wdb, "bf16", tag + " dbeta", rel=1e-2, scale=rms(delta))
