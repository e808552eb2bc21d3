"""Operands that start in the middle of an allocation (contiguous views such as Julia's
`view(x, 2:n)`): pointers that are aligned to the element size only.  Shapes are the ones that
would take the 16-byte vector paths, so the pointer alone decides; every operator and pullback must
give what it gives on aligned copies of the same data."""
import numpy as np
import pytest

from tests.util import assert_close, host_inputs

pytestmark = pytest.mark.gpu


def shifted(gpu, a, dtype, offset=1):
    """The array on the device, starting `offset` elements into a larger allocation."""
    if a is None:
        return None
    a = np.asarray(a, np.float32)
    flat = np.concatenate([np.full(offset, 7.0, np.float32), a.ravel(order="F"), np.full(3, 9.0, np.float32)])
    base = gpu.DeviceArray.from_numpy(flat, dtype)
    return gpu.DeviceArray(a.shape, dtype, ptr=base.ptr + offset * base.itemsize, base=base)


def aligned(gpu, a, dtype):
    return None if a is None else gpu.DeviceArray.from_numpy(np.asarray(a, np.float32), dtype)


def run_both(gpu, dtype, fn, arrays, delta_shape_of=None, rel=None):
    """fn(*device arrays) -> (outputs tuple, back or None); compares the shifted run with the aligned one."""
    outs = []
    for put in (aligned, shifted):
        dev_arrays = [put(gpu, a, dtype) for a in arrays]
        res, back = fn(*dev_arrays)
        res = res if isinstance(res, (tuple, list)) else (res,)
        got = [r.to_numpy() for r in res if hasattr(r, "to_numpy")]
        if back is not None:
            rng = np.random.default_rng(17)
            (delta,) = host_inputs(dtype, rng.normal(size=res[0].shape))
            grads = back(put(gpu, delta, dtype))
            got += [g.to_numpy() for g in grads if g is not None]
        outs.append(got)
    assert len(outs[0]) == len(outs[1])
    for i, (a, b) in enumerate(zip(*outs)):
        scale = float(np.sqrt(np.mean(np.square(a.astype(np.float64))))) if a.size else 0.0
        assert_close(b, a.astype(np.float64), dtype, f"result {i}", rel=rel, scale=scale)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_bias_activation_and_norms(gpu, dtype):
    rng = np.random.default_rng(1)
    x, g, b = host_inputs(dtype, rng.normal(size=(16, 8, 16, 4)), rng.uniform(0.5, 1.5, 16), rng.normal(size=16))
    rel = None
    run_both(gpu, dtype, lambda x_, b_: gpu.pullback(gpu.bias_activation, "gelu", x_, b_), [x, b], rel=rel)
    run_both(gpu, dtype, lambda x_, g_, b_: (lambda r: (r[0][0], r[1]))(
        gpu.pullback(gpu.batchnorm, x_, g_, b_, None, None, True, "relu", 0.1, 1e-3)), [x, g, b], rel=rel)
    run_both(gpu, dtype, lambda x_, g_, b_: gpu.pullback(gpu.groupnorm, x_, g_, b_, 4, "swish", 1e-3), [x, g, b], rel=rel)
    run_both(gpu, dtype, lambda x_, g_, b_: (lambda r: (r[0][0], r[1]))(
        gpu.pullback(gpu.instancenorm, x_, g_, b_, None, None, True, "relu", 0.1, 1e-3)), [x, g, b], rel=rel)
    gl, bl = host_inputs(dtype, rng.uniform(0.5, 1.5, (16, 8, 16, 1)), rng.normal(size=(16, 8, 16, 1)))
    run_both(gpu, dtype, lambda x_, g_, b_: gpu.pullback(gpu.layernorm, x_, g_, b_, "tanh", gpu.DEFAULT_DIMS, 1e-3), [x, gl, bl], rel=rel)
    x2, g2, b2 = host_inputs(dtype, rng.normal(size=(256, 96)), rng.uniform(0.5, 1.5, (256, 1)), rng.normal(size=(256, 1)))
    run_both(gpu, dtype, lambda x_, g_, b_: gpu.pullback(gpu.layernorm, x_, g_, b_, "identity", gpu.DEFAULT_DIMS, 1e-3), [x2, g2, b2], rel=rel)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_dense_conv_and_products(gpu, dtype):
    rng = np.random.default_rng(2)
    rel = None
    w, x, b = host_inputs(dtype, rng.normal(size=(128, 64)) / 8, rng.normal(size=(64, 96)), rng.normal(size=128))
    run_both(gpu, dtype, lambda w_, x_, b_: gpu.pullback(gpu.fused_dense_bias_activation, "gelu", w_, x_, b_), [w, x, b], rel=rel)
    w, x, b = host_inputs(dtype, rng.normal(size=(256, 256)) / 16, rng.normal(size=(256, 256)), rng.normal(size=256))
    run_both(gpu, dtype, lambda w_, x_, b_: gpu.pullback(gpu.fused_dense_bias_activation, "relu", w_, x_, b_), [w, x, b], rel=rel)
    cw, cx, cb = host_inputs(dtype, rng.normal(size=(3, 3, 32, 64)) / 17, rng.normal(size=(16, 16, 32, 4)), rng.normal(size=64))
    cd = gpu.DenseConvDims(cx.shape, cw.shape, padding=1)
    run_both(gpu, dtype, lambda w_, x_, b_: gpu.pullback(gpu.fused_conv_bias_activation, "relu", w_, x_, b_, cd), [cw, cx, cb], rel=rel)
    a, bm = host_inputs(dtype, rng.normal(size=(64, 32, 6)), rng.normal(size=(32, 48, 6)))
    run_both(gpu, dtype, lambda a_, b_: gpu.pullback(gpu.batched_matmul, a_, b_), [a, bm], rel=rel)
    q, k, v = host_inputs(dtype, rng.normal(size=(32, 4, 64, 2)), rng.normal(size=(32, 2, 128, 2)), rng.normal(size=(32, 2, 128, 2)))
    rel_a = None
    run_both(gpu, dtype, lambda q_, k_, v_: (lambda r: (r[0][0], r[1]))(
        gpu.pullback(gpu.scaled_dot_product_attention, q_, k_, v_, 1, 3, None, None, True)), [q, k, v], rel=rel_a)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_dropout(gpu, dtype):
    rng = np.random.default_rng(3)
    (x,) = host_inputs(dtype, rng.normal(size=(64, 32, 8)))
    for dims in (None, (1, 2)):
        def f(x_):
            (y, mask, _), back = gpu.pullback(gpu.dropout, gpu.PhiloxRNG(5, 3), x_, 0.4, True, 1.0 / 0.6, dims)
            return (y, mask), back
        run_both(gpu, dtype, f, [x])
    def g(x_):
        (y, _), back = gpu.pullback(gpu.alpha_dropout, gpu.PhiloxRNG(9, 0), x_, 0.3, True)
        return (y,), back
    run_both(gpu, dtype, g, [x])
