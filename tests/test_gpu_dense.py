"""matmul / fused_dense_bias_activation forward + pullback on the GPU against the oracle
(mirrors lib/LuxLib/test/common_ops/dense_tests.jl:13-93 and the Dense known answers of
test/core_layers/basic_tests.jl:151-194 of the reference)."""
import ctypes as C

import numpy as np
import pytest

from oracle import luxlib_oracle as O
from tests.util import stable_seed, assert_close, dev, f64, host_inputs, rms

pytestmark = pytest.mark.gpu


def test_reference_known_answers(gpu):
    d = lambda a: gpu.DeviceArray.from_numpy(np.asarray(a, np.float32))
    y = gpu.fused_dense_bias_activation("identity", d(np.ones((1, 10))), d(np.ones((10, 1))), None)
    assert y.to_numpy().tolist() == [[10.0]]
    y = gpu.fused_dense_bias_activation("identity", d(np.ones((2, 10))), d(np.array([np.ones(10), 2 * np.ones(10)]).T), None)
    assert y.to_numpy().tolist() == [[10.0, 20.0], [10.0, 20.0]]
    y = gpu.fused_dense_bias_activation("identity", d(np.ones((2, 10))), d(np.ones((10, 1))), d(np.ones(2)))
    assert y.to_numpy().tolist() == [[11.0], [11.0]]
    y = gpu.fused_dense_bias_activation("relu", d(-np.ones((1, 10))), d(np.ones((10, 1))), None)
    assert y.to_numpy().tolist() == [[0.0]]


MNK = [(4, 3, 32), (32, 3, 4), (33, 17, 65), (128, 128, 128), (130, 70, 257), (256, 64, 128), (300, 520, 96), (64, 64, 8)]


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("transA", [False, True])
@pytest.mark.parametrize("transB", [False, True])
def test_matmul_all_layouts(gpu, dtype, transA, transB):
    rng = np.random.default_rng(17)
    for (M, N, K) in MNK:
        for with_bias in (False, True):
            A = rng.normal(size=(K, M) if transA else (M, K))
            B = rng.normal(size=(N, K) if transB else (K, N))
            bias = rng.normal(size=M) if with_bias else None
            A, B, bias = host_inputs(dtype, A, B, bias)
            got = gpu.matmul(dev(gpu, A, dtype), dev(gpu, B, dtype), dev(gpu, bias, dtype), transA, transB).to_numpy()
            want = (f64(A).T if transA else f64(A)) @ (f64(B).T if transB else f64(B))
            if with_bias:
                want = want + f64(bias)[:, None]
            assert_close(got, want, dtype, f"{dtype} matmul {M}x{N}x{K} tA={transA} tB={transB} bias={with_bias}")


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("act", ["identity", "tanh", "sigmoid_fast", "relu", "gelu", "swish"])
def test_fused_dense_forward_and_pullback(gpu, dtype, act):
    rng = np.random.default_rng(stable_seed(dtype, act))
    for (M, K, N, with_bias) in [(4, 4, 3, True), (4, 32, 3, False), (32, 4, 3, True), (32, 32, 3, True), (200, 136, 72, True),
                                 (96, 264, 130, False)]:
        W = rng.normal(size=(M, K)) / np.sqrt(K)
        x = rng.normal(size=(K, N))
        b = rng.normal(size=M) * 0.1 if with_bias else None
        delta = rng.normal(size=(M, N))
        W, x, b, delta = host_inputs(dtype, W, x, b, delta)
        tag = f"{dtype} {act} dense {M}x{K}x{N} bias={with_bias}"
        y = gpu.fused_dense_bias_activation(act, dev(gpu, W, dtype), dev(gpu, x, dtype), dev(gpu, b, dtype))
        wy, wdW, wdx, wdb = O.fused_dense_pullback(act, f64(W), f64(x), f64(b), f64(delta))
        assert_close(y.to_numpy(), wy, dtype, tag + " y")
        y2, back = gpu.pullback(gpu.fused_dense_bias_activation, act, dev(gpu, W, dtype), dev(gpu, x, dtype), dev(gpu, b, dtype))
        np.testing.assert_array_equal(y2.to_numpy(), y.to_numpy())
        gW, gx, gb = back(dev(gpu, delta, dtype))
        if dtype == "bf16":
            # the rrule keeps y (and the pre-activation) in bf16 and the activation gradient dz is
            # stored in bf16 before the two gradient GEMMs (impl/dense.jl:83-103): restate that
            pre = O.matmuladd(f64(W), f64(x), f64(b))
            yq = f64(O.round_to_bf16(wy.astype(np.float32)))
            preq = f64(O.round_to_bf16(pre.astype(np.float32)))
            dz = f64(O.round_to_bf16(O.grad_activation(f64(delta), yq, act, preq).astype(np.float32)))
            wdW, wdx = dz @ f64(x).T, f64(W).T @ dz
            wdb = None if b is None else O.grad_activation(f64(delta), yq, act, preq).sum(axis=1)
        # magnitude of the summed terms (the sums can cancel): sqrt(#terms) * rms * rms
        dzr = rms(O.grad_activation(f64(delta), wy, act, O.matmuladd(f64(W), f64(x), f64(b))))
        assert_close(gW.to_numpy(), wdW, dtype, tag + " dW", scale=np.sqrt(N) * dzr * rms(x))
        assert_close(gx.to_numpy(), wdx, dtype, tag + " dx", scale=np.sqrt(M) * dzr * rms(W))
        if with_bias:
            assert_close(gb.to_numpy(), wdb, dtype, tag + " db", rel=None)
        else:
            assert gb is None


def test_dimension_mismatch(gpu):
    d = lambda *s: gpu.DeviceArray.from_numpy(np.ones(s, np.float32))
    with pytest.raises(gpu.DimensionMismatch):
        gpu.fused_dense_bias_activation("relu", d(3, 4), d(5, 2), None)
    with pytest.raises(gpu.DimensionMismatch):
        gpu.fused_dense_bias_activation("relu", d(3, 4), d(4, 2), d(4))
    with pytest.raises(gpu.DimensionMismatch):
        gpu.matmul(d(3, 4), d(5, 2))


def test_views_with_leading_dimension(gpu):
    """Operands that are views of larger arrays (leading dimension > rows), through the C ABI."""
    rng = np.random.default_rng(23)
    M, K, N, ldw, ldx, ldy = 37, 29, 21, 48, 40, 64
    Wb = rng.normal(size=(ldw, K)).astype(np.float32)
    xb = rng.normal(size=(ldx, N)).astype(np.float32)
    b = rng.normal(size=M).astype(np.float32)
    d = gpu.DeviceArray.from_numpy
    dW, dx_, db = d(Wb), d(xb), d(b)
    y = d(np.full((ldy, N), 7.0, np.float32))
    gpu._lib.call("luxhip_fused_dense_fwd", gpu.current_stream(), 0, gpu._lib.ACT_IDS["tanh"], M, K, N, dW.ptr, ldw, dx_.ptr, ldx,
                  db.ptr, y.ptr, ldy, None)
    got = y.to_numpy()
    want = np.tanh(f64(Wb[:M]) @ f64(xb[:K]) + f64(b)[:, None])
    assert_close(got[:M], want, "f32", "view y")
    np.testing.assert_array_equal(got[M:], 7.0)          # rows outside the view are untouched


def test_config1(gpu):
    """benchmark configuration 1: W 256x128 Glorot-uniform, x 128x64, bias 256, tanh, fp32."""
    rng = np.random.default_rng(1000)
    lim = np.sqrt(6.0 / 384.0)
    W = rng.uniform(-lim, lim, size=(256, 128)).astype(np.float32)
    x = rng.standard_normal(size=(128, 64)).astype(np.float32)
    b = (0.01 * rng.standard_normal(256)).astype(np.float32)
    delta = rng.standard_normal(size=(256, 64)).astype(np.float32)
    d = gpu.DeviceArray.from_numpy
    y, back = gpu.pullback(gpu.fused_dense_bias_activation, "tanh", d(W), d(x), d(b))
    gW, gx, gb = back(d(delta))
    wy, wdW, wdx, wdb = O.fused_dense_pullback("tanh", f64(W), f64(x), f64(b), f64(delta))
    w32 = O.fused_dense_pullback("tanh", W, x, b, delta)
    assert_close(y.to_numpy(), wy, "f32", "config1 y", want32=w32[0])
    assert_close(gW.to_numpy(), wdW, "f32", "config1 dW", want32=w32[1])
    assert_close(gx.to_numpy(), wdx, "f32", "config1 dx", want32=w32[2])
    assert_close(gb.to_numpy(), wdb, "f32", "config1 db", want32=w32[3])


def test_config4_dense_full_size(gpu):
    """benchmark configuration 4's first dense layer at full size (4096 -> 11008, 8192 tokens, gelu,
    bf16 storage / fp32 accumulation): output rows, weight-gradient rows and input-gradient
    columns are spot-checked against the fp64 oracle; linearity of the pullback in the
    cotangent is checked on the whole tensors."""
    rng = np.random.default_rng(1003)
    K, M, N = 4096, 11008, 8192
    std = np.sqrt(2.0 / (K + M))
    W = (std * rng.standard_normal(size=(M, K), dtype=np.float32))
    x = rng.standard_normal(size=(K, N), dtype=np.float32)
    b = np.zeros(M, np.float32)
    delta = (0.02 * rng.standard_normal(size=(M, N), dtype=np.float32))
    W, x, b, delta = host_inputs("bf16", W, x, b, delta)
    dW_, dx_, db_, dd_ = (dev(gpu, a, "bf16") for a in (W, x, b, delta))
    y, back = gpu.pullback(gpu.fused_dense_bias_activation, "gelu", dW_, dx_, db_)
    gW, gx, gb = back(dd_)
    rows = rng.choice(M, 24, replace=False)
    cols = rng.choice(N, 24, replace=False)
    yh = y.to_numpy()
    pre_rows = f64(W[rows]) @ f64(x)
    assert_close(yh[rows], O.act_value("gelu", pre_rows), "bf16", "config4 y rows")
    # dz as the device computes it: from the bf16-stored pre-activation and bf16-rounded
    pre_q = f64(O.round_to_bf16(pre_rows.astype(np.float32)))
    dz_rows = f64(O.round_to_bf16((f64(delta[rows]) * O.act_derivative("gelu", O.act_value("gelu", pre_q), pre_q)).astype(np.float32)))
    assert_close(gW.to_numpy()[rows], dz_rows @ f64(x).T, "bf16", "config4 dW rows")
    pre_cols = f64(W) @ f64(x[:, cols])
    pre_cq = f64(O.round_to_bf16(pre_cols.astype(np.float32)))
    dz_cols = f64(O.round_to_bf16((f64(delta[:, cols]) * O.act_derivative("gelu", O.act_value("gelu", pre_cq), pre_cq)).astype(np.float32)))
    assert_close(gx.to_numpy()[:, cols], f64(W).T @ dz_cols, "bf16", "config4 dx cols")
    assert_close(gb.to_numpy()[rows], (f64(delta[rows]) * O.act_derivative("gelu", O.act_value("gelu", pre_q), pre_q)).sum(axis=1),
                 "bf16", "config4 db rows", scale=rms(delta) * 90)
    # linearity: pullback(2 * delta) == 2 * pullback(delta) (exact: scaling by 2 commutes with rounding)
    gW2, gx2, _ = back(dev(gpu, 2 * delta, "bf16"))
    np.testing.assert_array_equal(gW2.to_numpy()[rows], 2 * gW.to_numpy()[rows])
    np.testing.assert_array_equal(gx2.to_numpy()[:, cols], 2 * gx.to_numpy()[:, cols])


@pytest.mark.parametrize("ragged", ["m", "n"])
def test_ragged_tile_rounds_bf16(gpu, ragged):
    """43 x 32 tiles of 256 x 256 do not fill whole rounds of one tile per compute unit: the
    library cuts such a problem into a part of whole rounds and a rest on smaller tiles.  Rows and
    columns on both sides of the cut and at the far end are compared with the fp64 oracle."""
    rng = np.random.default_rng(77)
    M, N = (11008, 8192) if ragged == "m" else (8192, 11008)
    K = 64
    A, B, bias = host_inputs("bf16", rng.normal(size=(M, K)), rng.normal(size=(K, N)), rng.normal(size=M))
    got = gpu.matmul(dev(gpu, A, "bf16"), dev(gpu, B, "bf16"), dev(gpu, bias, "bf16")).to_numpy()
    want = lambda r, c: f64(A[r]) @ f64(B[:, c]) + f64(bias[r])[:, None]
    full = slice(None)
    cut = 10240   # 40 of the 43 tiles along the ragged dimension keep the big tiles
    edge = np.r_[0:4, cut - 130:cut + 130, (M if ragged == "m" else N) - 4:(M if ragged == "m" else N)]
    if ragged == "m":
        assert_close(got[edge], want(edge, full), "bf16", "ragged m rows")
    else:
        assert_close(got[:, edge], want(full, edge), "bf16", "ragged n cols")


@pytest.mark.parametrize("transA,transB", [(False, False), (False, True), (True, True)])
@pytest.mark.parametrize("pretranspose", [1, 0])
def test_large_bf16_operand_layouts(gpu, transA, transB, pretranspose):
    """Large bf16 products whose operands are contiguous along m or n: by default such operands are
    first copied into the k-contiguous layout (switch gemm_pretranspose); both routes against the
    fp64 oracle on a band of rows and columns."""
    rng = np.random.default_rng(78)
    M, N, K = 4096, 4096, 2048
    A, B, bias = host_inputs("bf16", rng.normal(size=(K, M) if transA else (M, K)), rng.normal(size=(N, K) if transB else (K, N)),
                             rng.normal(size=M))
    gpu.set_option("gemm_pretranspose", pretranspose)
    try:
        got = gpu.matmul(dev(gpu, A, "bf16"), dev(gpu, B, "bf16"), dev(gpu, bias, "bf16"), transA=transA, transB=transB).to_numpy()
    finally:
        gpu.set_option("gemm_pretranspose", 1)
    Am, Bm = (f64(A).T if transA else f64(A)), (f64(B).T if transB else f64(B))
    rows = np.r_[0:130, 2040:2060, M - 130:M]
    assert_close(got[rows], Am[rows] @ Bm + f64(bias[rows])[:, None], "bf16", "rows", scale=np.sqrt(K))
    assert_close(got[:, rows], Am @ Bm[:, rows] + f64(bias)[:, None], "bf16", "cols", scale=np.sqrt(K))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("with_derivative", [False, True])
def test_closure_activation(gpu, dtype, with_derivative):
    """An activation without a device kernel (the reference's dense tests use `x -> x^3`, dense_tests.jl; rule branch 3,
    impl/dense.jl:103-112): the product and the bias run on the device, the closure and its derivative on a staged host
    copy; with and without a derivative supplied by the caller (central differences otherwise)."""
    rng = np.random.default_rng(stable_seed("closure", dtype))
    w, x, b, delta = host_inputs(dtype, rng.normal(size=(24, 16)) / 4, rng.normal(size=(16, 10)), rng.normal(size=24),
                                 rng.normal(size=(24, 10)))
    cube = lambda z: z ** 3
    if with_derivative:
        def cube(z):
            return z ** 3
        cube.derivative = lambda z: 3.0 * z ** 2
    y, back = gpu.pullback(gpu.fused_dense_bias_activation, cube, dev(gpu, w, dtype), dev(gpu, x, dtype), dev(gpu, b, dtype))
    y2 = gpu.fused_dense_bias_activation(cube, dev(gpu, w, dtype), dev(gpu, x, dtype), dev(gpu, b, dtype))
    z = f64(w) @ f64(x) + f64(b)[:, None]
    if dtype == "bf16":                                   # the device stores z, the closure reads the stored values
        z = f64(O.round_to_bf16(z.astype(np.float32)))
    assert_close(y.to_numpy(), z ** 3, dtype, "y")
    np.testing.assert_array_equal(y2.to_numpy(), y.to_numpy())
    dz = f64(delta) * 3.0 * z ** 2
    if dtype == "bf16":
        dz = f64(O.round_to_bf16(dz.astype(np.float32)))
    dw, dx, db = back(dev(gpu, delta, dtype))
    assert_close(dw.to_numpy(), dz @ f64(x).T, dtype, "dw")
    assert_close(dx.to_numpy(), f64(w).T @ dz, dtype, "dx")
    assert_close(db.to_numpy(), dz.sum(axis=1), dtype, "db")
    # the same closure through bias_activation, fast_activation and a convolution
    xb, bb, db_ = host_inputs(dtype, rng.normal(size=(5, 4, 6, 3)), rng.normal(size=6), rng.normal(size=(5, 4, 6, 3)))
    yb, backb = gpu.pullback(gpu.bias_activation, cube, dev(gpu, xb, dtype), dev(gpu, bb, dtype))
    zb = f64(xb) + f64(bb).reshape(1, 1, 6, 1)
    if dtype == "bf16":
        zb = f64(O.round_to_bf16(zb.astype(np.float32)))
    assert_close(yb.to_numpy(), zb ** 3, dtype, "bias_activation y")
    gxb, gbb = backb(dev(gpu, db_, dtype))
    dzb = f64(db_) * 3.0 * zb ** 2
    if dtype == "bf16":
        dzb = f64(O.round_to_bf16(dzb.astype(np.float32)))
    assert_close(gxb.to_numpy(), dzb, dtype, "bias_activation dx")
    assert_close(gbb.to_numpy(), dzb.sum(axis=(0, 1, 3)), dtype, "bias_activation db")
    yf, backf = gpu.pullback(gpu.fast_activation, cube, dev(gpu, xb, dtype))
    assert_close(yf.to_numpy(), f64(xb) ** 3, dtype, "fast_activation y")
    assert_close(backf(dev(gpu, db_, dtype))[0].to_numpy(), f64(db_) * 3.0 * f64(xb) ** 2, dtype, "fast_activation dx")
    cw, cx, cb, cd_ = host_inputs(dtype, rng.normal(size=(3, 3, 4, 6)) / 6, rng.normal(size=(8, 7, 4, 2)), rng.normal(size=6),
                                  rng.normal(size=(8, 7, 6, 2)))
    cdims = gpu.DenseConvDims(cx.shape, cw.shape, padding=1)
    yc, backc = gpu.pullback(gpu.fused_conv_bias_activation, cube, dev(gpu, cw, dtype), dev(gpu, cx, dtype), dev(gpu, cb, dtype), cdims)
    od = O.ConvDims(cx.shape, cw.shape, 1, 1, 1)
    zc = O.fused_conv_bias_activation("identity", f64(cw), f64(cx), f64(cb), od)
    if dtype == "bf16":
        zc = f64(O.round_to_bf16(zc.astype(np.float32)))
    assert_close(yc.to_numpy(), zc ** 3, dtype, "conv y")
    dzc = f64(cd_) * 3.0 * zc ** 2
    if dtype == "bf16":
        dzc = f64(O.round_to_bf16(dzc.astype(np.float32)))
    gw, gx, gb = backc(dev(gpu, cd_, dtype))
    assert_close(gw.to_numpy(), O.conv_filter_grad(f64(cx), dzc, od), dtype, "conv dw")
    assert_close(gx.to_numpy(), O.conv_data_grad(dzc, f64(cw), od), dtype, "conv dx")
    assert_close(gb.to_numpy(), dzc.sum(axis=(0, 1, 3)), dtype, "conv db")


def test_mixed_storage_types_are_promoted(gpu):
    """A bf16 weight with fp32 activations (and the other way round): the operands are promoted to fp32, as
    the reference promotes mixed element types (ext/CUDAExt/cublaslt.jl:46-63; dense_tests.jl:226-228 runs
    the mixed combinations); the result is fp32 and each gradient comes back in its operand's own type."""
    import warnings
    rng = np.random.default_rng(41)
    w = O.round_to_bf16(rng.normal(size=(24, 16)).astype(np.float32) / 4)
    x = rng.normal(size=(16, 10)).astype(np.float32)
    b = O.round_to_bf16(rng.normal(size=24).astype(np.float32))
    delta = rng.normal(size=(24, 10)).astype(np.float32)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        y, back = gpu.pullback(gpu.fused_dense_bias_activation, "tanh", dev(gpu, w, "bf16"), dev(gpu, x, "f32"), dev(gpu, b, "bf16"))
        y2 = gpu.fused_dense_bias_activation("tanh", dev(gpu, w, "bf16"), dev(gpu, x, "f32"), dev(gpu, b, "bf16"))
    wy, wdw, wdx, wdb = O.fused_dense_pullback("tanh", f64(w), f64(x), f64(b), f64(delta))
    assert y.dtype == "f32" and y2.dtype == "f32"
    assert_close(y.to_numpy(), wy, "f32", "y")
    np.testing.assert_array_equal(y2.to_numpy(), y.to_numpy())
    dw, dx, db = back(dev(gpu, delta, "f32"))
    assert (dw.dtype, dx.dtype, db.dtype) == ("bf16", "f32", "bf16")
    assert_close(dw.to_numpy(), wdw, "bf16", "dw")
    assert_close(dx.to_numpy(), wdx, "f32", "dx")
    assert_close(db.to_numpy(), wdb, "bf16", "db")
    # convolution: fp32 weight, bf16 input
    cw = rng.normal(size=(3, 3, 4, 6)).astype(np.float32) / 6
    cx = O.round_to_bf16(rng.normal(size=(8, 7, 4, 2)).astype(np.float32))
    cd = gpu.DenseConvDims(cx.shape, cw.shape, padding=1)
    od = O.ConvDims(cx.shape, cw.shape, 1, 1, 1)
    cdelta = rng.normal(size=cd.y_shape).astype(np.float32)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        cy, cback = gpu.pullback(gpu.fused_conv_bias_activation, "relu", dev(gpu, cw, "f32"), dev(gpu, cx, "bf16"), None, cd)
    wy, wdw, wdx, _ = O.fused_conv_pullback("relu", f64(cw), f64(cx), None, od, f64(cdelta))
    assert cy.dtype == "f32"
    assert_close(cy.to_numpy(), wy, "f32", "conv y")
    gw, gx, gb = cback(dev(gpu, cdelta, "f32"))
    assert (gw.dtype, gx.dtype, gb) == ("f32", "bf16", None)
    assert_close(gw.to_numpy(), wdw, "f32", "conv dw", scale=1.0)
    assert_close(gx.to_numpy(), wdx, "bf16", "conv dx", scale=1.0)
