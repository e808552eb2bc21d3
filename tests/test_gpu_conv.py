"""fused_conv_bias_activation forward + pullback (fprop, dgrad, wgrad) on the GPU against the
oracle (mirrors lib/LuxLib/test/common_ops/conv_tests.jl:25-117 and the known answers of
test/core_layers/conv_tests.jl:54-69,145-190 of the reference)."""
import numpy as np
import pytest

from oracle import luxlib_oracle as O
from tests.util import stable_seed, assert_close, dev, f64, host_inputs, rms

pytestmark = pytest.mark.gpu


def cdims(gpu, xs, ws, **kw):
    return gpu.DenseConvDims(xs, ws, **kw), O.ConvDims(xs, ws, **kw)


def test_reference_known_answers(gpu):
    d = lambda a: gpu.DeviceArray.from_numpy(np.asarray(a, np.float32))
    # impulse response => true convolution orientation
    x = np.zeros((7, 7, 1, 1), np.float32)
    x[3, 3, 0, 0] = 1
    w = np.random.default_rng(1).normal(size=(3, 3, 1, 1)).astype(np.float32)
    gd, _ = cdims(gpu, x.shape, w.shape)
    y = gpu.fused_conv_bias_activation("identity", d(w), d(x), None, gd).to_numpy()
    assert y.shape == (5, 5, 1, 1)
    np.testing.assert_array_equal(y[1:4, 1:4, 0, 0], w[:, :, 0, 0])
    gd, _ = cdims(gpu, x.shape, w.shape, flipkernel=True)
    yc = gpu.fused_conv_bias_activation("identity", d(w), d(x), None, gd).to_numpy()
    np.testing.assert_array_equal(yc[1:4, 1:4, 0, 0], w[::-1, ::-1, 0, 0])
    # asymmetric padding, all ones, relu, zero bias
    x = np.ones((28, 28, 1, 1), np.float32)
    w = np.ones((3, 3, 1, 1), np.float32)
    gd, _ = cdims(gpu, x.shape, w.shape, padding=(0, 1, 1, 2))
    y = gpu.fused_conv_bias_activation("relu", d(w), d(x), d(np.zeros(1)), gd).to_numpy()[:, :, 0, 0]
    assert y.shape == (27, 29)
    assert (y[0, 0], y[1, 1], y[26, 0], y[0, 28], y[0, 27], y[26, 28]) == (6.0, 9.0, 4.0, 3.0, 6.0, 2.0)


CASES = [
    # x shape, w shape, stride, pad, dilation, groups, flip
    ((6, 5, 4, 2), (2, 2, 4, 6), 1, 0, 1, 1, False),
    ((6, 5, 4, 2), (2, 2, 4, 6), 2, 1, 1, 1, False),
    ((6, 5, 4, 2), (2, 2, 2, 6), 1, 1, 1, 2, False),
    ((7, 8, 3, 2), (3, 3, 3, 5), (2, 1), (0, 1, 2, 1), (1, 2), 1, False),
    ((7, 8, 3, 2), (3, 2, 3, 5), 1, 1, 1, 1, True),
    ((16, 16, 16, 4), (3, 3, 16, 32), 1, 1, 1, 1, False),
    ((14, 14, 64, 3), (3, 3, 64, 128), 1, 1, 1, 1, False),
    ((15, 13, 32, 2), (3, 3, 8, 64), 2, 1, 1, 4, False),
    ((12, 12, 24, 2), (5, 5, 24, 40), 1, 2, 2, 1, True),
    ((9, 9, 8, 5), (1, 1, 8, 16), 1, 0, 1, 1, False),
    # channel counts per group that are multiples of the K stage (whole-tap kernels), with
    # strides, dilation, asymmetric padding, groups, partial column tiles and > 128 columns
    ((13, 11, 64, 3), (3, 2, 32, 64), (2, 1), (1, 0, 2, 1), (1, 2), 2, True),
    ((10, 12, 64, 2), (3, 3, 32, 96), 1, (2, 1, 0, 2), 2, 2, False),
    ((8, 8, 32, 5), (3, 3, 32, 320), 1, 1, 1, 1, False),
    # output planes of a multiple of 32 positions (bf16 filter gradient straight from the WHCN cotangent)
    ((16, 8, 32, 3), (3, 3, 16, 48), 1, 1, 1, 2, False),
    ((16, 8, 16, 2), (3, 3, 16, 24), (2, 1), (1, 1, 1, 1), 1, 1, True),
]


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("case", range(len(CASES)))
def test_conv_and_gradients(gpu, dtype, case):
    xs, ws, stride, pad, dil, groups, flip = CASES[case]
    rng = np.random.default_rng(100 + case)
    gd, od = cdims(gpu, xs, ws, stride=stride, padding=pad, dilation=dil, groups=groups, flipkernel=flip)
    fan_in = ws[0] * ws[1] * ws[2]
    x, w, dy = host_inputs(dtype, rng.normal(size=xs), rng.normal(size=ws) * np.sqrt(2.0 / fan_in), rng.normal(size=od.y_shape()))
    tag = f"{dtype} case {case}"
    y = gpu.conv(dev(gpu, x, dtype), dev(gpu, w, dtype), gd)
    assert_close(y.to_numpy(), O.conv(f64(x), f64(w), od), dtype, tag + " conv")
    dx = gpu.conv_data_grad(dev(gpu, dy, dtype), dev(gpu, w, dtype), gd)
    assert_close(dx.to_numpy(), O.conv_data_grad(f64(dy), f64(w), od), dtype, tag + " dgrad")
    dw = gpu.conv_filter_grad(dev(gpu, x, dtype), dev(gpu, dy, dtype), gd)
    assert_close(dw.to_numpy(), O.conv_filter_grad(f64(x), f64(dy), od), dtype, tag + " wgrad")


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("act", ["identity", "sigmoid", "gelu", "relu"])
def test_fused_conv_pullback(gpu, dtype, act):
    rng = np.random.default_rng(stable_seed(dtype, act))
    for case in (1, 2, 5, 7, 10, 11, 13):
        xs, ws, stride, pad, dil, groups, flip = CASES[case]
        gd, od = cdims(gpu, xs, ws, stride=stride, padding=pad, dilation=dil, groups=groups, flipkernel=flip)
        fan_in = ws[0] * ws[1] * ws[2]
        for with_bias in (True, False):
            x, w, b, delta = host_inputs(dtype, rng.normal(size=xs), rng.normal(size=ws) * np.sqrt(2.0 / fan_in),
                                         rng.normal(size=ws[3]) * 0.1 if with_bias else None, rng.normal(size=od.y_shape()))
            tag = f"{dtype} {act} case {case} bias={with_bias}"
            y, back = gpu.pullback(gpu.fused_conv_bias_activation, act, dev(gpu, w, dtype), dev(gpu, x, dtype), dev(gpu, b, dtype), gd)
            wy, wdw, wdx, wdb = O.fused_conv_pullback(act, f64(w), f64(x), f64(b), od, f64(delta))
            assert_close(y.to_numpy(), wy, dtype, tag + " y")
            gw, gx, gb = back(dev(gpu, delta, dtype))
            if dtype == "bf16":
                # y, the pre-activation and dz are stored in bf16 between the passes
                pre = O.bias_add(O.conv(f64(x), f64(w), od), f64(b))
                yq, preq = (f64(O.round_to_bf16(a.astype(np.float32))) for a in (wy, pre))
                dzx = O.grad_activation(f64(delta), yq, act, preq)
                dz = f64(O.round_to_bf16(dzx.astype(np.float32)))
                wdw, wdx = O.conv_filter_grad(f64(x), dz, od), O.conv_data_grad(dz, f64(w), od)
                wdb = O.grad_bias_add(b, dzx)
            dzr = rms(delta)
            assert_close(gw.to_numpy(), wdw, dtype, tag + " dw", scale=np.sqrt(np.prod(od.y_shape()) / ws[3]) * dzr * rms(x) * 0.5)
            assert_close(gx.to_numpy(), wdx, dtype, tag + " dx", scale=np.sqrt(ws[0] * ws[1] * ws[3] / groups) * dzr * rms(w) * 0.5)
            if with_bias:
                assert_close(gb.to_numpy(), wdb, dtype, tag + " db", rel=None)
            else:
                assert gb is None


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("xs,ws,stride,pad,dil,groups,flip", [
    ((12, 4, 2), (3, 4, 6), 1, (1, 1), 1, 1, False), ((13, 6, 3), (4, 3, 4), 2, (0, 2), 2, 2, False),
    ((9, 2, 2), (2, 2, 3), 1, (1, 0), 1, 1, True), ((200, 64, 4), (5, 64, 96), 1, 2, 1, 1, False)])
def test_one_spatial_dim(gpu, dtype, xs, ws, stride, pad, dil, groups, flip):
    """x (W, C, N), w (K, C/groups, Cout) (lib/LuxLib/test/common_ops/conv_tests.jl runs 1-d cases too)."""
    rng = np.random.default_rng(stable_seed(dtype, xs, ws))
    gd = gpu.DenseConvDims(xs, ws, stride=stride, padding=pad, dilation=dil, groups=groups, flipkernel=flip)
    od = O.ConvDims.one_spatial_dim(xs, ws, stride, pad, dil, groups, flip)
    assert gd.y_shape == (od.y_shape()[0],) + od.y_shape()[2:]
    x, w, b, delta = host_inputs(dtype, rng.normal(size=xs), rng.normal(size=ws) * np.sqrt(2.0 / (ws[0] * ws[1])),
                                 rng.normal(size=ws[2]) * 0.1, rng.normal(size=gd.y_shape))
    y, back = gpu.pullback(gpu.fused_conv_bias_activation, "tanh", dev(gpu, w, dtype), dev(gpu, x, dtype), dev(gpu, b, dtype), gd)
    x4, w4, d4 = f64(x).reshape(od.x_shape), f64(w).reshape(od.w_shape), f64(delta).reshape(od.y_shape())
    wy, wdw, wdx, wdb = O.fused_conv_pullback("tanh", w4, x4, f64(b), od, d4)
    assert_close(y.to_numpy(), wy.reshape(gd.y_shape), dtype, "1-d y")
    gw, gx, gb = back(dev(gpu, delta, dtype))
    if dtype == "bf16":                      # y and dz are stored in bf16 between the passes
        yq = f64(O.round_to_bf16(wy.astype(np.float32)))
        dzx = O.grad_activation(d4, yq, "tanh", None)
        dz = f64(O.round_to_bf16(dzx.astype(np.float32)))
        wdw, wdx, wdb = O.conv_filter_grad(x4, dz, od), O.conv_data_grad(dz, w4, od), O.grad_bias_add(b, dzx)
    assert gw.shape == tuple(ws) and gx.shape == tuple(xs)
    assert_close(gw.to_numpy(), wdw.reshape(ws), dtype, "1-d dw", scale=np.sqrt(np.prod(gd.y_shape) / ws[2]) * rms(delta) * rms(x) * 0.5)
    assert_close(gx.to_numpy(), wdx.reshape(xs), dtype, "1-d dx", scale=np.sqrt(ws[0] * ws[2] / groups) * rms(delta) * rms(w) * 0.5)
    assert_close(gb.to_numpy(), wdb, dtype, "1-d db", rel=None)
    with pytest.raises(gpu.Unsupported):
        gpu.DenseConvDims((4, 4, 4, 4, 2, 1), (2, 2, 2, 2, 2, 3))       # four spatial dims


def test_dimension_mismatch(gpu):
    with pytest.raises(gpu.DimensionMismatch):
        gpu.DenseConvDims((8, 8, 4, 2), (3, 3, 3, 6))
    d = lambda *s: gpu.DeviceArray.from_numpy(np.ones(s, np.float32))
    gd = gpu.DenseConvDims((8, 8, 4, 2), (3, 3, 4, 6))
    with pytest.raises(gpu.DimensionMismatch):
        gpu.fused_conv_bias_activation("relu", d(3, 3, 4, 6), d(8, 8, 4, 3), None, gd)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_config5_full_size(gpu, dtype):
    """benchmark configuration 5 at full size: x 56x56x128x64, w 3x3x128x128 Kaiming-normal, stride 1,
    pad 1, relu.  Forward and input gradient: fp64 oracle on two images.  Filter gradient: the
    adjoint identity <dw, w'> == <dz, conv(x, w')> against the (checked) forward kernel, an
    fp64 oracle on a two-image batch and the fp64 oracle on the whole batch.  Bias gradient: fp64 channel sums."""
    rng = np.random.default_rng(1004)
    xs, ws = (56, 56, 128, 64), (3, 3, 128, 128)
    gd, od = cdims(gpu, xs, ws, padding=1)
    x = rng.standard_normal(size=xs, dtype=np.float32)
    w = (np.sqrt(2.0 / 1152) * rng.standard_normal(size=ws, dtype=np.float32))
    b = (0.01 * rng.standard_normal(128)).astype(np.float32)
    delta = rng.standard_normal(size=xs[:2] + (128, 64), dtype=np.float32)
    x, w, b, delta = host_inputs(dtype, x, w, b, delta)
    dx_, dw_, db_, dd_ = (dev(gpu, a, dtype) for a in (x, w, b, delta))
    y, back = gpu.pullback(gpu.fused_conv_bias_activation, "relu", dw_, dx_, db_, gd)
    gw, gx, gb = back(dd_)
    yh = y.to_numpy()
    sub = [3, 63]          # the last image lies in the rows that the fp32 kernels give to a second launch
    od2 = O.ConvDims(xs[:3] + (2,), ws, padding=1)
    wy = O.fused_conv_bias_activation("relu", f64(w), f64(x[..., sub]), f64(b), od2)
    assert_close(yh[..., sub], wy, dtype, "config5 y")
    dz = f64(delta) * (yh > 0)                                    # relu: derivative from the stored output
    if dtype == "bf16":
        dz = f64(O.round_to_bf16(dz.astype(np.float32)))
    assert_close(gx.to_numpy()[..., sub], O.conv_data_grad(dz[..., sub], f64(w), od2), dtype, "config5 dx")
    assert_close(gb.to_numpy(), (f64(delta) * (yh > 0)).sum(axis=(0, 1, 3)), dtype, "config5 db", scale=rms(delta) * 300)
    # adjoint identity for the filter gradient
    wp = host_inputs(dtype, rng.standard_normal(size=ws, dtype=np.float32))[0]
    cwp = gpu.conv(dx_, dev(gpu, wp, dtype), gd).to_numpy().astype(np.float64)
    lhs = float((gw.to_numpy().astype(np.float64) * f64(wp)).sum())
    rhs = float((dz * cwp).sum())
    assert abs(lhs - rhs) <= (2e-4 if dtype == "f32" else 1e-2) * max(abs(rhs), np.sqrt(dz.size)), (lhs, rhs)
    # and an oracle check of the same kernel on a two-image batch
    gd2 = gpu.DenseConvDims(xs[:3] + (2,), ws, padding=1)
    dzq = dz[..., sub].astype(np.float32)
    gw2 = gpu.conv_filter_grad(dev(gpu, x[..., sub], dtype), dev(gpu, dzq, dtype), gd2)
    assert_close(gw2.to_numpy(), O.conv_filter_grad(f64(x[..., sub]), f64(dzq), od2), dtype, "config5 dw (2 images)")
    # the full-size filter gradient itself (in bf16 a kernel of its own: one partial sum per image): every element
    assert_close(gw.to_numpy(), O.conv_filter_grad(f64(x), dz, od), dtype, "config5 dw (all images)")


# Shapes that the bf16 kernel with the tile's input window in LDS takes (3 x 3, unit stride and dilation, output as
# large as the input, channels per group in multiples of 64), chosen for its special cases:
WINDOW_CASES = [
    # x shape, w shape, pad, groups, flip
    ((20, 12, 128, 5), (3, 3, 128, 192), 1, 1, True),              # two 64-channel parts; two column tiles, the second half empty
    ((12, 10, 128, 3), (3, 3, 64, 128), 1, 2, False),              # groups: 64 channels in, 64 columns out per group
    ((14, 14, 64, 3), (3, 3, 64, 80), (0, 2, 2, 0), 1, False),     # asymmetric padding, 80 columns (a partial fragment row of channels)
    ((56, 56, 64, 1), (3, 3, 64, 64), 1, 1, False),                # one image: 196 fragments on 13 workgroups (15 or 16 each)
    ((6, 6, 64, 2), (3, 3, 64, 16), 1, 1, False),                  # 72 positions: one partial tile, rows past the last position
    ((32, 34, 64, 64), (3, 3, 64, 64), 1, 1, True),                # 4352 fragments = 17 per compute unit: tiles with a seventeenth fragment
    ((12, 10, 128, 3), (3, 3, 128, 48), 1, 1, False),              # two 64-channel parts into 48 columns (the kernel for at most 64)
]


@pytest.mark.parametrize("case", range(len(WINDOW_CASES)))
def test_window_kernel_shapes(gpu, case):
    """fprop and dgrad on those shapes against the fp64 oracle (the larger problems on a few images, whose results
    do not depend on the other images) and against the gather-per-tap kernels that the `conv_tile` switch selects."""
    xs, ws, pad, groups, flip = WINDOW_CASES[case]
    rng = np.random.default_rng(300 + case)
    gd, od = cdims(gpu, xs, ws, padding=pad, groups=groups, flipkernel=flip)
    assert od.y_shape()[:2] == xs[:2]
    fan_in = 9 * ws[2]
    x, w, b, dy = host_inputs("bf16", rng.normal(size=xs), rng.normal(size=ws) * np.sqrt(2.0 / fan_in), rng.normal(size=ws[3]) * 0.1,
                              rng.normal(size=od.y_shape()))
    dx_, dw_, db_, ddy_ = (dev(gpu, a, "bf16") for a in (x, w, b, dy))
    y = gpu.fused_conv_bias_activation("relu", dw_, dx_, db_, gd).to_numpy()
    gx = gpu.conv_data_grad(ddy_, dw_, gd).to_numpy()
    gpu.set_option("conv_tile", 84)
    try:
        y_tap = gpu.fused_conv_bias_activation("relu", dw_, dx_, db_, gd).to_numpy()
        gx_tap = gpu.conv_data_grad(ddy_, dw_, gd).to_numpy()
    finally:
        gpu.set_option("conv_tile", 0)
    imgs = sorted({0, xs[3] // 2, xs[3] - 1})
    sub = O.ConvDims(xs[:3] + (len(imgs),), ws, padding=pad, groups=groups, flipkernel=flip)
    want_y = O.fused_conv_bias_activation("relu", f64(w), f64(x[..., imgs]), f64(b), sub)
    want_gx = O.conv_data_grad(f64(dy[..., imgs]), f64(w), sub)
    tag = f"window case {case} "
    assert_close(y[..., imgs], want_y, "bf16", tag + "y")
    assert_close(gx[..., imgs], want_gx, "bf16", tag + "dgrad")
    # the two kernels add the same products in a different order: equal up to the bf16 rounding of the result
    assert_close(y, f64(y_tap), "bf16", tag + "y vs gather kernel")
    assert_close(gx, f64(gx_tap), "bf16", tag + "dgrad vs gather kernel")
    # both window kernels on every shape, whichever the library would pick: tiles of 64 (1) and of 128 (2) output channels
    for forced in (1, 2):
        gpu.set_option("conv_tile", forced)
        try:
            y_f = gpu.fused_conv_bias_activation("relu", dw_, dx_, db_, gd).to_numpy()
            gx_f = gpu.conv_data_grad(ddy_, dw_, gd).to_numpy()
        finally:
            gpu.set_option("conv_tile", 0)
        assert_close(y_f[..., imgs], want_y, "bf16", tag + f"y, column tiles {64 * forced}")
        assert_close(gx_f[..., imgs], want_gx, "bf16", tag + f"dgrad, column tiles {64 * forced}")


@pytest.mark.parametrize("xs,ws", [((16, 16, 128, 36), (3, 3, 128, 128)),      # 36 images: the last group of eight is incomplete
                                   ((16, 8, 64, 136), (3, 3, 64, 64))])        # one 64 x 64 channel part per image, 17 groups of eight
def test_filter_gradient_window_kernel_batches(gpu, xs, ws):
    """bf16 filter gradient with the input window of an image in LDS (one workgroup per image and 64 x 64 channel
    part, the parts of eight images dealt to the eight XCDs) against the fp64 oracle and against the gather kernel."""
    rng = np.random.default_rng(777 + xs[3])
    gd, od = cdims(gpu, xs, ws, padding=1)
    x, dy = host_inputs("bf16", rng.normal(size=xs), rng.normal(size=od.y_shape()))
    dx_, ddy_ = dev(gpu, x, "bf16"), dev(gpu, dy, "bf16")
    dw = gpu.conv_filter_grad(dx_, ddy_, gd).to_numpy()
    gpu.set_option("conv_tile", 84)
    try:
        dw_gather = gpu.conv_filter_grad(dx_, ddy_, gd).to_numpy()
    finally:
        gpu.set_option("conv_tile", 0)
    want = O.conv_filter_grad(f64(x), f64(dy), od)
    assert_close(dw, want, "bf16", f"window wgrad N={xs[3]}")
    assert_close(dw_gather, want, "bf16", f"gather wgrad N={xs[3]}")


@pytest.mark.parametrize("xs,ws", [((16, 16, 128, 300), (3, 3, 128, 128)),     # 4 parts x 300 images: 128 workgroups per part, 2-3 images each
                                   ((8, 8, 256, 200), (3, 3, 256, 256))])       # 16 parts x 200 images: 32 per part, 6-7 images each
def test_filter_gradient_window_kernel_large_batches(gpu, xs, ws):
    """Batches so large that one workgroup per image and channel part would be more than two per compute unit: a workgroup
    then walks several images and the number of fp32 partial sums (and the scratch memory for them) stays bounded.  Against
    the gather kernel on the whole gradient and against the fp64 oracle on the first eight output channels."""
    rng = np.random.default_rng(778 + xs[3])
    gd, od = cdims(gpu, xs, ws, padding=1)
    x, dy = host_inputs("bf16", rng.normal(size=xs), rng.normal(size=od.y_shape()))
    dx_, ddy_ = dev(gpu, x, "bf16"), dev(gpu, dy, "bf16")
    dw = gpu.conv_filter_grad(dx_, ddy_, gd).to_numpy()
    gpu.set_option("conv_tile", 84)
    try:
        dw_gather = gpu.conv_filter_grad(dx_, ddy_, gd).to_numpy()
    finally:
        gpu.set_option("conv_tile", 0)
    assert_close(dw, f64(dw_gather), "bf16", f"window against gather wgrad N={xs[3]}")
    _, od8 = cdims(gpu, xs, ws[:3] + (8,), padding=1)
    want = O.conv_filter_grad(f64(x), f64(dy[:, :, :8]), od8)
    assert_close(dw[..., :8], want, "bf16", f"window wgrad N={xs[3]}, first output channels")


def _random_window_shapes(count, seed):
    """Shapes that the 3 x 3 window kernels accept (unit stride, output as large as the input, channels per group in
    multiples of 64, W * H a multiple of 4), drawn with a fixed seed."""
    rng = np.random.default_rng(seed)
    shapes = []
    while len(shapes) < count:
        W, H = int(rng.integers(3, 61)), int(rng.integers(3, 41))
        if (W * H) % 4 != 0:
            continue
        groups = int(rng.choice([1, 1, 2]))
        cin = 64 * groups * int(rng.integers(1, 3))
        cout = groups * int(rng.choice([8, 16, 48, 64, 72, 128, 136]))
        N = int(rng.integers(1, 8))
        pad = [(1, 1, 1, 1), (0, 2, 2, 0), (2, 0, 1, 1), (1, 1, 0, 2)][int(rng.integers(0, 4))]
        shapes.append(((W, H, cin, N), (3, 3, cin // groups, cout), pad, groups, bool(rng.integers(0, 2))))
    return shapes


@pytest.mark.parametrize("case", range(16))
def test_window_kernels_random_shapes(gpu, case):
    """fprop (with bias and relu) and dgrad of both window kernels against the gather-per-tap kernels, which the other
    tests pin against the oracle: the same products in another order, so equal up to the bf16 rounding of the result."""
    xs, ws, pad, groups, flip = _random_window_shapes(16, 4242)[case]
    rng = np.random.default_rng(900 + case)
    gd, od = cdims(gpu, xs, ws, padding=pad, groups=groups, flipkernel=flip)
    assert od.y_shape()[:2] == xs[:2]
    x, w, b, dy = host_inputs("bf16", rng.normal(size=xs), rng.normal(size=ws) * np.sqrt(2.0 / (9 * ws[2])), rng.normal(size=ws[3]) * 0.1,
                              rng.normal(size=od.y_shape()))
    dx_, dw_, db_, ddy_ = (dev(gpu, a, "bf16") for a in (x, w, b, dy))
    out = {}
    for tile in (84, 1, 2, 0):
        gpu.set_option("conv_tile", tile)
        try:
            out[tile] = (gpu.fused_conv_bias_activation("relu", dw_, dx_, db_, gd).to_numpy(), gpu.conv_data_grad(ddy_, dw_, gd).to_numpy())
        finally:
            gpu.set_option("conv_tile", 0)
    tag = f"random window shape {xs} {ws} pad {pad} groups {groups} flip {flip}: "
    for tile in (1, 2, 0):
        assert_close(out[tile][0], f64(out[84][0]), "bf16", tag + f"y, conv_tile {tile}")
        assert_close(out[tile][1], f64(out[84][1]), "bf16", tag + f"dgrad, conv_tile {tile}")


# Shapes of the bf16 pullback's single pass over delta (dz as it lies, its channel-contiguous copy, the bias gradient's
# partial sums, the repacked filter): positions and channels in multiples of 8.  Chosen for its special cases.
ONE_PASS_CASES = [
    # x shape, w shape, stride, pad, groups
    ((24, 20, 16, 3), (3, 3, 16, 72), 1, 1, 1),        # 480 positions: a partial last tile; 72 channels: a partial second channel tile
    ((8, 8, 8, 2), (1, 1, 8, 8), 1, 0, 1),             # one partial tile in both directions
    ((32, 30, 32, 9), (3, 3, 16, 64), 1, 1, 2),        # 960 positions: fifteen tiles; groups
    ((64, 64, 8, 16), (3, 3, 8, 128), 1, 1, 1),        # 2048 tiles: a workgroup walks two of them and keeps the channel sums in registers
    ((16, 16, 8, 2), (2, 2, 8, 200), 2, 0, 1),         # 64 positions, four channel tiles (the last with 8 channels), strided
]


@pytest.mark.parametrize("case", range(len(ONE_PASS_CASES)))
@pytest.mark.parametrize("act", ["relu", "gelu", "identity"])
def test_pullback_single_pass_over_delta(gpu, case, act):
    """with and without a bias (the partial sums), with the identity (dz is delta itself) and with activations that
    take their derivative from the output (relu) or from the pre-activation (gelu)"""
    xs, ws, stride, pad, groups = ONE_PASS_CASES[case]
    rng = np.random.default_rng(stable_seed("one pass", case, act))
    gd, od = cdims(gpu, xs, ws, stride=stride, padding=pad, groups=groups)
    assert (od.y_shape()[0] * od.y_shape()[1]) % 8 == 0 and ws[3] % 8 == 0
    fan_in = ws[0] * ws[1] * ws[2]
    for with_bias in (True, False):
        x, w, b, delta = host_inputs("bf16", rng.normal(size=xs), rng.normal(size=ws) * np.sqrt(2.0 / fan_in),
                                     rng.normal(size=ws[3]) * 0.1 if with_bias else None, rng.normal(size=od.y_shape()))
        tag = f"bf16 {act} one-pass case {case} bias={with_bias}"
        y, back = gpu.pullback(gpu.fused_conv_bias_activation, act, dev(gpu, w, "bf16"), dev(gpu, x, "bf16"), dev(gpu, b, "bf16"), gd)
        wy, _, _, _ = O.fused_conv_pullback(act, f64(w), f64(x), f64(b), od, f64(delta))
        gw, gx, gb = back(dev(gpu, delta, "bf16"))
        # y, the pre-activation and dz are stored in bf16 between the passes
        pre = O.bias_add(O.conv(f64(x), f64(w), od), f64(b))
        yq, preq = (f64(O.round_to_bf16(a.astype(np.float32))) for a in (wy, pre))
        dzx = O.grad_activation(f64(delta), yq, act, preq)
        dz = f64(O.round_to_bf16(dzx.astype(np.float32)))
        dzr = rms(delta)
        assert_close(gw.to_numpy(), O.conv_filter_grad(f64(x), dz, od), "bf16", tag + " dw",
                     scale=np.sqrt(np.prod(od.y_shape()) / ws[3]) * dzr * rms(x) * 0.5)
        assert_close(gx.to_numpy(), O.conv_data_grad(dz, f64(w), od), "bf16", tag + " dx",
                     scale=np.sqrt(ws[0] * ws[1] * ws[3] / groups) * dzr * rms(w) * 0.5)
        if with_bias:
            assert_close(gb.to_numpy(), O.grad_bias_add(b, dzx), "bf16", tag + " db")
        else:
            assert gb is None
