"""bias_activation forward + pullback on the GPU against the oracle
(mirrors lib/LuxLib/test/common_ops/bias_act_tests.jl:16-131 and activation_tests.jl:9-67)."""
import numpy as np
import pytest

from oracle import luxlib_oracle as O
from tests.util import stable_seed, assert_close, dev, f64, host_inputs

pytestmark = pytest.mark.gpu

ACTS = ["identity", "relu", "sigmoid", "sigmoid_fast", "softplus", "logsigmoid", "gelu", "swish", "lisht", "tanh",
        "tanh_fast"]
SHAPES = [(2, 2, 3, 4), (4, 5), (7, 3, 5), (64, 8, 4), (16, 16, 6, 3), (1024, 16, 8), (5,), (1, 24, 7), (8, 640)]


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("act", ACTS)
def test_forward_and_pullback(gpu, act, dtype):
    rng = np.random.default_rng(stable_seed(act, dtype))
    for shape in SHAPES:
        nb = shape[0] if len(shape) == 1 else shape[-2]
        x, b, delta = host_inputs(dtype, rng.normal(size=shape) * 1.5, rng.normal(size=nb), rng.normal(size=shape))
        dx_, db_ = dev(gpu, x, dtype), dev(gpu, b, dtype)
        y = gpu.bias_activation(act, dx_, db_)
        want = O.bias_activation(act, f64(x), f64(b))
        assert_close(y.to_numpy(), want, dtype, f"{act} {shape} y")
        y2, back = gpu.pullback(gpu.bias_activation, act, dx_, db_)
        gx, gb = back(dev(gpu, delta, dtype))
        _, wdx, wdb = O.bias_activation_pullback(act, f64(x), f64(b), f64(delta))
        if dtype == "bf16" and O.ACT_NEEDS[O.canonical_act(act)] == "out":
            # the rrule keeps only the output, in the array's storage type
            # (impl/bias_activation.jl:76-84): the derivative sees the bf16-rounded y
            wdx = O.grad_activation(f64(delta), f64(O.round_to_bf16(want.astype(np.float32))), act, None)
            wdb = O.grad_bias_add(b, wdx)
        assert_close(y2.to_numpy(), want, dtype, f"{act} {shape} y (rrule)")
        assert_close(gx.to_numpy(), wdx, dtype, f"{act} {shape} dx")
        # the bias gradient is a long sum of rounded terms in bf16 storage: compare at the
        # same relative bar against the magnitude of the summed terms
        assert_close(gb.to_numpy(), wdb, dtype, f"{act} {shape} db",
                     rel=None)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_no_bias_inplace_and_empty(gpu, dtype):
    rng = np.random.default_rng(5)
    (x,) = host_inputs(dtype, rng.normal(size=(6, 5, 3)))
    d = dev(gpu, x, dtype)
    y = gpu.bias_activation("relu", d, None)
    assert_close(y.to_numpy(), np.maximum(x, 0), dtype, "relu no bias")
    (b,) = host_inputs(dtype, rng.normal(size=5))
    r = gpu.bias_activation_inplace("tanh", d, dev(gpu, b, dtype))
    assert r is d
    assert_close(d.to_numpy(), O.bias_activation("tanh", f64(x), f64(b)), dtype, "in place")
    # zero-sized arrays (bias_act_tests.jl:119-131)
    e = gpu.DeviceArray((4, 3, 2, 0), dtype)
    out = gpu.bias_activation("relu", e, dev(gpu, np.ones(2), dtype))
    assert out.shape == (4, 3, 2, 0) and out.to_numpy().size == 0
    y0, back = gpu.pullback(gpu.bias_activation, "relu", e, dev(gpu, np.ones(2), dtype))
    gx, gb = back(gpu.DeviceArray((4, 3, 2, 0), dtype))
    assert gx.shape == (4, 3, 2, 0)
    np.testing.assert_array_equal(gb.to_numpy(), np.zeros(2))


def test_argument_errors(gpu):
    x = gpu.DeviceArray.from_numpy(np.ones((3, 4), np.float32))
    with pytest.raises(AssertionError):
        gpu.bias_activation("relu", x, gpu.DeviceArray.from_numpy(np.ones(4, np.float32)))
    with pytest.raises(gpu.Unsupported):
        gpu.bias_activation("cube", x, None)


def test_full_size_properties(gpu):
    """benchmark configuration 2's bias_activation(relu) at full size (1024, 64, 128): checked through
    size-independent properties (idempotence of relu, linearity of the pullback, the bias
    gradient equals the channel sums of dx)."""
    rng = np.random.default_rng(11)
    shape = (32, 32, 64, 128)
    x = rng.normal(size=shape).astype(np.float32)
    b = rng.normal(size=64).astype(np.float32)
    delta = rng.normal(size=shape).astype(np.float32)
    dx_, db_, dd = (gpu.DeviceArray.from_numpy(a) for a in (x, b, delta))
    y, back = gpu.pullback(gpu.bias_activation, "relu", dx_, db_)
    yh = y.to_numpy()
    np.testing.assert_array_equal(yh, np.maximum(x + b.reshape(1, 1, 64, 1), 0))      # exact in fp32
    y2 = gpu.bias_activation("relu", y, None)
    np.testing.assert_array_equal(y2.to_numpy(), yh)                                    # idempotent
    gx, gb = back(dd)
    gxh = gx.to_numpy()
    np.testing.assert_array_equal(gxh, delta * (yh > 0))
    assert_close(gb.to_numpy(), gxh.astype(np.float64).sum(axis=(0, 1, 3)), "f32", "db full size")
