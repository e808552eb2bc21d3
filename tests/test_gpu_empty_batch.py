"""Zero-sized batches through every operator of the path: the reference's tests feed empty
arrays to bias_activation (lib/LuxLib/test/common_ops/bias_act_tests.jl:119-131) and its layers
accept a batch of zero samples; here every operator and its pullback must return arrays of the
right (empty) shape, parameter gradients that are exactly zero, and leave the library usable."""
import numpy as np
import pytest

from tests.util import dev

pytestmark = pytest.mark.gpu


def _zeros(a):
    return a.to_numpy().astype(np.float64)


def _check_zero(a, shape, what):
    assert tuple(a.shape) == tuple(shape), f"{what}: shape {a.shape} != {shape}"
    h = _zeros(a)
    assert np.all(h == 0), f"{what}: not zero"


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_dense_empty_batch(gpu, dtype):
    rng = np.random.default_rng(1)
    w, b = dev(gpu, rng.normal(size=(6, 5)), dtype), dev(gpu, rng.normal(size=6), dtype)
    x = gpu.DeviceArray((5, 0), dtype)
    y = gpu.fused_dense_bias_activation("gelu", w, x, b)
    assert y.shape == (6, 0)
    y2, back = gpu.pullback(gpu.fused_dense_bias_activation, "gelu", w, x, b)
    dw, dx, db = back(gpu.DeviceArray((6, 0), dtype))
    _check_zero(dw, (6, 5), "dw")
    assert dx.shape == (5, 0)
    _check_zero(db, (6,), "db")


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_norms_empty_batch(gpu, dtype):
    rng = np.random.default_rng(2)
    C = 8
    g, b = dev(gpu, rng.normal(size=C), dtype), dev(gpu, rng.normal(size=C), dtype)
    x = gpu.DeviceArray((4, 3, C, 0), dtype)
    delta = gpu.DeviceArray((4, 3, C, 0), dtype)
    # groupnorm
    y, back = gpu.pullback(gpu.groupnorm, x, g, b, 4, "relu")
    assert y.shape == (4, 3, C, 0)
    dx, dg, db = back(delta)
    assert dx.shape == (4, 3, C, 0)
    _check_zero(dg, (C,), "groupnorm dgamma")
    _check_zero(db, (C,), "groupnorm dbeta")
    # instancenorm without running statistics
    y, back = gpu.pullback(gpu.instancenorm, x, g, b, None, None, True, "relu")
    y = y[0] if isinstance(y, tuple) else y
    assert y.shape == (4, 3, C, 0)
    dx, dg, db = back(delta)[:3]
    assert dx.shape == (4, 3, C, 0)
    _check_zero(dg, (C,), "instancenorm dgamma")
    _check_zero(db, (C,), "instancenorm dbeta")
    # batchnorm in inference mode (training statistics of no samples are undefined)
    rm, rv = dev(gpu, rng.normal(size=C), dtype), dev(gpu, rng.uniform(0.5, 2, size=C), dtype)
    out = gpu.batchnorm(x, g, b, rm, rv, False, "relu")
    y = out[0] if isinstance(out, tuple) else out
    assert y.shape == (4, 3, C, 0)
    # layernorm over the first dimensions with a per-position affine transform
    xs = gpu.DeviceArray((4, 3, 0), dtype)
    gs, bs = dev(gpu, rng.normal(size=(4, 3, 1)), dtype), dev(gpu, rng.normal(size=(4, 3, 1)), dtype)
    y, back = gpu.pullback(gpu.layernorm, xs, gs, bs, "tanh", (1, 2))
    assert y.shape == (4, 3, 0)
    dx, dg, db = back(gpu.DeviceArray((4, 3, 0), dtype))
    assert dx.shape == (4, 3, 0)
    _check_zero(dg, (4, 3, 1), "layernorm dgamma")
    _check_zero(db, (4, 3, 1), "layernorm dbeta")


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_conv_empty_batch(gpu, dtype):
    rng = np.random.default_rng(3)
    w, b = dev(gpu, rng.normal(size=(3, 3, 4, 6)), dtype), dev(gpu, rng.normal(size=6), dtype)
    x = gpu.DeviceArray((9, 8, 4, 0), dtype)
    cd = gpu.DenseConvDims(x.shape, w.shape, stride=1, padding=1)
    y, back = gpu.pullback(gpu.fused_conv_bias_activation, "relu", w, x, b, cd)
    assert y.shape == (9, 8, 6, 0)
    dw, dx, db = back(gpu.DeviceArray((9, 8, 6, 0), dtype))
    _check_zero(dw, (3, 3, 4, 6), "conv dw")
    assert dx.shape == (9, 8, 4, 0)
    _check_zero(db, (6,), "conv db")


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_dropout_batched_matmul_attention_empty_batch(gpu, dtype):
    rng = gpu.PhiloxRNG(7)
    x = gpu.DeviceArray((5, 4, 0), dtype)
    out = gpu.dropout(rng, x, 0.5, True, 2.0)
    assert out[0].shape == (5, 4, 0) and out[1].shape == (5, 4, 0)
    a = gpu.DeviceArray((5, 4, 0), dtype)
    b = gpu.DeviceArray((4, 3, 0), dtype)
    z, back = gpu.pullback(gpu.batched_matmul, a, b)
    assert z.shape == (5, 3, 0)
    da, db = back(gpu.DeviceArray((5, 3, 0), dtype))
    assert da.shape == (5, 4, 0) and db.shape == (4, 3, 0)
    q = gpu.DeviceArray((8, 2, 6, 0), dtype)
    k = gpu.DeviceArray((8, 2, 7, 0), dtype)
    v = gpu.DeviceArray((8, 2, 7, 0), dtype)
    (o, wts), back = gpu.pullback(gpu.scaled_dot_product_attention, q, k, v)
    assert o.shape == (8, 2, 6, 0) and wts.shape == (7, 6, 2, 0)
    dq, dk, dv = back(gpu.DeviceArray((8, 2, 6, 0), dtype))[:3]
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape


def test_library_still_works_after_empty_calls(gpu):
    rng = np.random.default_rng(5)
    x = rng.normal(size=(6, 5, 3)).astype(np.float32)
    y = gpu.bias_activation("relu", dev(gpu, x, "f32"), None)
    np.testing.assert_array_equal(y.to_numpy(), np.maximum(x, 0))
