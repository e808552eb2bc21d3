"""luxhip_bias_activation_bwd_noalloc (partial sums and arrival counters in a fixed device block, no
allocation) against luxhip_bias_activation_bwd, which takes them from the stream's workspace, and
against the oracle: two calls in a row on the same device, the second on a smaller input, so that the
block still holds the first call's contents."""
import numpy as np
import pytest

from oracle import luxlib_oracle as O
from tests.util import assert_close, dev, f64, host_inputs, stable_seed

pytestmark = pytest.mark.gpu

# (first shape, second smaller shape): the "channel" kernel (I >= 64: partial sums per channel and slice,
# arrival counters), the "plane" kernel (dense layout: partial sums per batch slice) and a mixed pair
PAIRS = [
    ((32, 32, 64, 16), (16, 8, 24, 3)),
    ((1, 512, 96), (1, 40, 7)),
    ((24, 24, 130, 5), (3, 3, 7, 2)),
    ((8, 4096), (128, 12, 4)),
]


def _run(gpu, entry, act, dtype, x, b, delta):
    """y = act(x + b) through the library, then the pullback through `entry`; returns host arrays."""
    I = int(np.prod(x.shape[:-2])) if x.ndim > 2 else 1
    Cc, N = x.shape[-2], x.shape[-1]
    dx_, db_ = dev(gpu, x, dtype), dev(gpu, b, dtype)
    y = gpu.DeviceArray(x.shape, dtype)
    pre = gpu.DeviceArray(x.shape, dtype)
    s = gpu.current_stream()
    gpu._lib.call("luxhip_bias_activation_fwd", s, y.code, gpu._lib.ACT_IDS[act], I, Cc, N, dx_.ptr, db_.ptr, y.ptr, pre.ptr)
    dd = dev(gpu, delta, dtype)
    gx, gb = gpu.DeviceArray(x.shape, dtype), gpu.DeviceArray((Cc,), dtype)
    gpu._lib.call(entry, s, y.code, gpu._lib.ACT_IDS[act], I, Cc, N, dd.ptr, y.ptr, pre.ptr, gx.ptr, gb.ptr)
    return y.to_numpy(), gx.to_numpy(), gb.to_numpy()


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("act", ["relu", "swish", "identity"])
@pytest.mark.parametrize("pair", range(len(PAIRS)))
def test_two_calls_in_a_row_match_the_allocating_entry_point(gpu, pair, act, dtype):
    rng = np.random.default_rng(stable_seed("noalloc", pair, act, dtype))
    for shape in PAIRS[pair]:                                   # large first, then the smaller one
        x, b, delta = host_inputs(dtype, rng.normal(size=shape) * 1.5, rng.normal(size=shape[-2]), rng.normal(size=shape))
        y0, gx0, gb0 = _run(gpu, "luxhip_bias_activation_bwd", act, dtype, x, b, delta)
        y1, gx1, gb1 = _run(gpu, "luxhip_bias_activation_bwd_noalloc", act, dtype, x, b, delta)
        tag = f"{act} {dtype} {shape}"
        np.testing.assert_array_equal(gx1, gx0, err_msg=tag + " dx")
        # the same kernels with the same split of the sums: identical bits
        np.testing.assert_array_equal(gb1, gb0, err_msg=tag + " dbias")
        # and both against the oracle, from the output and pre-activation the device holds
        yq = f64(y1)
        pre = f64(x) + f64(b).reshape((-1, 1))
        if dtype == "bf16":
            pre = f64(O.round_to_bf16(pre.astype(np.float32)))
        wdx = O.grad_activation(f64(delta), yq, act, pre)
        assert_close(gx1, wdx, dtype, tag + " dx vs oracle")
        assert_close(gb1, O.grad_bias_add(b, wdx), dtype, tag + " dbias vs oracle", rel=None if dtype == "f32" else 2e-2)


def test_sizes_beyond_the_fixed_block_are_refused(gpu):
    """Dense layout with 2^20 features and a batch of 64: two batch slices of 4 MiB of partial sums each."""
    shape = (1 << 20, 64)
    d = gpu.DeviceArray(shape, "f32")
    gb = gpu.DeviceArray((shape[0],), "f32")
    s = gpu.current_stream()
    with pytest.raises(gpu._lib.LuxHipError) as ei:
        gpu._lib.call("luxhip_bias_activation_bwd_noalloc", s, 0, 1, 1, shape[0], shape[1], d.ptr, d.ptr, None, d.ptr, gb.ptr)
    assert ei.value.status == gpu._lib.INVALID and "scratch" in str(ei.value)
    # the allocating entry point takes the same shape
    gpu._lib.call("luxhip_bias_activation_bwd", s, 0, 1, 1, shape[0], shape[1], d.ptr, d.ptr, None, d.ptr, gb.ptr)
    gpu.synchronize()
