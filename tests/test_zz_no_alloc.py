"""luxhip_bias_activation_bwd_noalloc (partial sums and arrival counters in a fixed device block, no
allocation) against luxhip_bias_activation_bwd, which takes them from the stream's workspace, and
against the oracle: two calls in a row on the same device, the second on a smaller input, so that the
block still holds the first call's contents."""
import ctypes as C

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
        assert_close(gb1, O.grad_bias_add(b, wdx), dtype, tag + " dbias vs oracle")


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


def test_no_allocation_on_a_stream_without_workspace_also_while_it_records(gpu):
    """What the entry point is for: on a stream that has never had scratch memory (the allocating entry point
    would have to create it, and refuses to while the stream records a graph) the call succeeds eagerly and
    under capture, the device's free memory does not change, and the replayed graph gives the same bits."""
    hip = C.CDLL("libamdhip64.so")
    hip.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
    hip.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
    hip.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
    hip.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_char_p, C.c_size_t]
    hip.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
    hip.hipGraphExecDestroy.argtypes = [C.c_void_p]
    hip.hipGraphDestroy.argtypes = [C.c_void_p]

    def free_bytes():
        f, t = C.c_size_t(), C.c_size_t()
        assert hip.hipMemGetInfo(C.byref(f), C.byref(t)) == 0
        return f.value

    rng = np.random.default_rng(5)
    shape = (16, 16, 48, 6)
    I, Cc, N = 256, 48, 6
    x, b, delta = host_inputs("f32", rng.normal(size=shape), rng.normal(size=Cc), rng.normal(size=shape))
    _, gx0, gb0 = _run(gpu, "luxhip_bias_activation_bwd", "relu", "f32", x, b, delta)      # reference bits, main stream
    y = dev(gpu, np.maximum(x + b.reshape(1, 1, -1, 1), 0), "f32")
    dd = dev(gpu, delta, "f32")
    gx, gb = gpu.DeviceArray(shape, "f32"), gpu.DeviceArray((Cc,), "f32")
    fresh = C.c_void_p()
    gpu._lib.call("luxhip_stream_create", C.byref(fresh))
    graph, graph_exec = C.c_void_p(), C.c_void_p()
    try:
        gpu.synchronize()
        call = lambda: gpu._lib.call("luxhip_bias_activation_bwd_noalloc", fresh, 0, gpu._lib.ACT_IDS["relu"], I, Cc, N, dd.ptr, y.ptr,
                                     None, gx.ptr, gb.ptr)
        before = free_bytes()
        call()
        gpu._lib.call("luxhip_stream_synchronize", fresh)
        assert free_bytes() == before
        np.testing.assert_array_equal(gb.to_numpy(), gb0)
        np.testing.assert_array_equal(gx.to_numpy(), gx0)
        # the allocating entry point on the same stream, while it records: refused (no workspace yet)
        assert hip.hipStreamBeginCapture(fresh, 1) == 0
        try:
            with pytest.raises(gpu._lib.LuxHipError):
                gpu._lib.call("luxhip_bias_activation_bwd", fresh, 0, gpu._lib.ACT_IDS["relu"], I, Cc, N, dd.ptr, y.ptr, None, gx.ptr, gb.ptr)
            call()                                              # recorded
        finally:
            rc = hip.hipStreamEndCapture(fresh, C.byref(graph))
        assert rc == 0 and graph.value
        assert free_bytes() == before
        assert hip.hipGraphInstantiate(C.byref(graph_exec), graph, None, None, 0) == 0
        zero_b = dev(gpu, np.zeros(Cc, np.float32), "f32")
        for _ in range(2):
            gpu._lib.call("luxhip_memcpy_d2d", gb.ptr, zero_b.ptr, Cc * 4, fresh)
            assert hip.hipGraphLaunch(graph_exec, fresh) == 0
            gpu._lib.call("luxhip_stream_synchronize", fresh)
            np.testing.assert_array_equal(gb.to_numpy(), gb0)
            np.testing.assert_array_equal(gx.to_numpy(), gx0)
    finally:
        if graph_exec.value:
            hip.hipGraphExecDestroy(graph_exec)
        if graph.value:
            hip.hipGraphDestroy(graph)
        gpu._lib.call("luxhip_stream_destroy", fresh)
