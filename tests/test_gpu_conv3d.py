"""Convolutions with three spatial dims (x (W, H, D, C, N), w (kW, kH, kD, C/groups, Cout)) on the
GPU against the oracle's N-d convolution (the reference's conv tests run 3-d cases through the same
entry points, lib/LuxLib/test/common_ops/conv_tests.jl; layers: test/core_layers/conv_tests.jl)."""
import numpy as np
import pytest

from oracle import luxlib_oracle as O
from tests.util import stable_seed, assert_close, dev, f64, host_inputs, rms

pytestmark = pytest.mark.gpu

CASES = [
    # x shape, w shape, stride, pad, dilation, groups, flip
    ((6, 5, 4, 3, 2), (2, 2, 2, 3, 4), 1, 0, 1, 1, False),
    ((6, 5, 7, 4, 2), (3, 2, 3, 4, 6), 1, 1, 1, 1, False),
    ((7, 6, 8, 4, 2), (2, 3, 3, 2, 6), (1, 2, 2), (1, 0, 2, 1, 1, 2), (2, 1, 2), 2, False),
    ((7, 6, 8, 4, 2), (2, 3, 3, 2, 6), (2, 1, 3), (0, 1, 1, 1, 2, 0), (1, 2, 1), 2, True),
    ((8, 8, 6, 16, 3), (3, 3, 3, 16, 32), 1, 1, 1, 1, False),            # planes of 16-byte multiples
    ((8, 4, 5, 32, 2), (3, 3, 2, 8, 64), (1, 1, 2), 1, 1, 4, True),
    ((5, 5, 3, 2, 1), (1, 1, 5, 2, 3), 1, (0, 0, 0, 0, 2, 2), 1, 1, False),   # more depth taps than slices
]


def cdims(gpu, xs, ws, **kw):
    return gpu.DenseConvDims(xs, ws, **kw), O.ConvDimsND(xs, ws, **kw)


def test_impulse_response_orientation(gpu):
    d = lambda a: gpu.DeviceArray.from_numpy(np.asarray(a, np.float32))
    x = np.zeros((5, 5, 5, 1, 1), np.float32)
    x[2, 2, 2, 0, 0] = 1
    w = np.random.default_rng(1).normal(size=(3, 3, 3, 1, 1)).astype(np.float32)
    gd, _ = cdims(gpu, x.shape, w.shape)
    y = gpu.fused_conv_bias_activation("identity", d(w), d(x), None, gd).to_numpy()
    assert y.shape == (3, 3, 3, 1, 1)
    np.testing.assert_array_equal(y[..., 0, 0], w[..., 0, 0])                  # true convolution
    gd, _ = cdims(gpu, x.shape, w.shape, flipkernel=True)
    y = gpu.fused_conv_bias_activation("identity", d(w), d(x), None, gd).to_numpy()
    np.testing.assert_array_equal(y[..., 0, 0], w[::-1, ::-1, ::-1, 0, 0])     # cross-correlation


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("case", range(len(CASES)))
def test_conv_and_gradients(gpu, dtype, case):
    xs, ws, stride, pad, dil, groups, flip = CASES[case]
    rng = np.random.default_rng(300 + case)
    gd, od = cdims(gpu, xs, ws, stride=stride, padding=pad, dilation=dil, groups=groups, flipkernel=flip)
    assert gd.out_spatial == od.out_spatial
    fan_in = ws[0] * ws[1] * ws[2] * ws[3]
    x, w, dy = host_inputs(dtype, rng.normal(size=xs), rng.normal(size=ws) * np.sqrt(2.0 / fan_in), rng.normal(size=gd.y_shape))
    tag = f"{dtype} case {case}"
    y = gpu.conv(dev(gpu, x, dtype), dev(gpu, w, dtype), gd)
    assert_close(y.to_numpy(), O.conv_nd(f64(x), f64(w), od), dtype, tag + " conv")
    dx = gpu.conv_data_grad(dev(gpu, dy, dtype), dev(gpu, w, dtype), gd)
    assert_close(dx.to_numpy(), O.conv_nd_data_grad(f64(dy), f64(w), od), dtype, tag + " dgrad")
    dw = gpu.conv_filter_grad(dev(gpu, x, dtype), dev(gpu, dy, dtype), gd)
    assert_close(dw.to_numpy(), O.conv_nd_filter_grad(f64(x), f64(dy), od), dtype, tag + " wgrad")


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("act", ["identity", "gelu", "relu"])
def test_fused_conv_pullback(gpu, dtype, act):
    rng = np.random.default_rng(stable_seed("conv3d", dtype, act))
    for case in (1, 2, 3, 4, 5):
        xs, ws, stride, pad, dil, groups, flip = CASES[case]
        gd, od = cdims(gpu, xs, ws, stride=stride, padding=pad, dilation=dil, groups=groups, flipkernel=flip)
        fan_in = ws[0] * ws[1] * ws[2] * ws[3]
        for with_bias in (True, False):
            x, w, b, delta = host_inputs(dtype, rng.normal(size=xs), rng.normal(size=ws) * np.sqrt(2.0 / fan_in),
                                         rng.normal(size=ws[4]) * 0.1 if with_bias else None, rng.normal(size=gd.y_shape))
            tag = f"{dtype} {act} case {case} bias={with_bias}"
            y, back = gpu.pullback(gpu.fused_conv_bias_activation, act, dev(gpu, w, dtype), dev(gpu, x, dtype), dev(gpu, b, dtype), gd)
            wy, wdw, wdx, wdb = O.fused_conv_nd_pullback(act, f64(w), f64(x), f64(b), od, f64(delta))
            assert_close(y.to_numpy(), wy, dtype, tag + " y")
            gw, gx, gb = back(dev(gpu, delta, dtype))
            if dtype == "bf16":
                # y, the pre-activation and dz are stored in bf16 between the passes
                pre = O.bias_add(O.conv_nd(f64(x), f64(w), od), f64(b))
                yq, preq = (f64(O.round_to_bf16(a.astype(np.float32))) for a in (wy, pre))
                dzx = O.grad_activation(f64(delta), yq, act, preq)
                dz = f64(O.round_to_bf16(dzx.astype(np.float32)))
                wdw, wdx = O.conv_nd_filter_grad(f64(x), dz, od), O.conv_nd_data_grad(dz, f64(w), od)
                wdb = O.grad_bias_add(b, dzx)
            dzr = rms(delta)
            assert gw.shape == tuple(ws) and gx.shape == tuple(xs)
            assert_close(gw.to_numpy(), wdw, dtype, tag + " dw", scale=np.sqrt(np.prod(gd.y_shape) / ws[4]) * dzr * rms(x) * 0.5)
            assert_close(gx.to_numpy(), wdx, dtype, tag + " dx", scale=np.sqrt(ws[0] * ws[1] * ws[2] * ws[4] / groups) * dzr * rms(w) * 0.5)
            if with_bias:
                assert_close(gb.to_numpy(), wdb, dtype, tag + " db", rel=None)
            else:
                assert gb is None


def test_depth_of_one_equals_the_two_dimensional_problem(gpu):
    """(W, H, 1, C, N) with a (kW, kH, 1, ., .) weight is the 2-d problem bit for bit."""
    rng = np.random.default_rng(9)
    x = rng.normal(size=(9, 8, 1, 6, 3)).astype(np.float32)
    w = rng.normal(size=(3, 3, 1, 6, 10)).astype(np.float32)
    g3 = gpu.DenseConvDims(x.shape, w.shape, stride=1, padding=(1, 1, 1, 1, 0, 0))
    g2 = gpu.DenseConvDims((9, 8, 6, 3), (3, 3, 6, 10), stride=1, padding=1)
    y3 = gpu.conv(dev(gpu, x, "f32"), dev(gpu, w, "f32"), g3).to_numpy()
    y2 = gpu.conv(dev(gpu, x[:, :, 0], "f32"), dev(gpu, w[:, :, 0], "f32"), g2).to_numpy()
    np.testing.assert_array_equal(y3[:, :, 0], y2)
