"""The part of the C ABI that owns device buffers, streams and events (what the reference gets from
its GPU array package): streams keep their work ordered and their scratch memory apart, the pooled
allocator reuses blocks, events time a stream, the per-kernel profile names the kernels that ran,
and errors come back as status codes with a message."""
import ctypes as C
import json

import numpy as np
import pytest

from oracle import luxlib_oracle as O
from tests.util import assert_close, dev, f64

pytestmark = pytest.mark.gpu


def _new_stream(gpu):
    s = C.c_void_p()
    gpu._lib.call("luxhip_stream_create", C.byref(s))
    return s


def test_device_info(gpu):
    info = gpu.device_info()
    assert info["compute_units"] > 0 and info["total_mem"] > 0 and info["name"]


def test_two_streams_keep_their_scratch_apart(gpu):
    """batchnorm (arrival counters, exchange words, partial sums in the per-stream workspace) and
    groupnorm pullbacks issued alternately on two streams that are not synchronised with each other:
    every result equals the one computed alone."""
    rng = np.random.default_rng(3)
    main = gpu.current_stream()
    other = _new_stream(gpu)
    shapes = [(16, 16, 8, 4), (32, 32, 16, 8), (6, 5, 12, 3)]
    cases = []
    for shape in shapes:
        Cc = shape[2]
        x, d = rng.normal(size=shape).astype(np.float32), rng.normal(size=shape).astype(np.float32)
        g, b = rng.uniform(0.5, 1.5, Cc).astype(np.float32), rng.normal(size=Cc).astype(np.float32)
        cases.append((x, d, g, b))
    results = {0: [], 1: []}
    keep = []            # a block that goes back to the pool may be handed to the other stream at once: nothing
    # is released before both streams have finished
    try:
        for rep in range(3):
            for x, d, g, b in cases:
                for which, stream in ((0, main), (1, other)):
                    gpu.set_stream(stream)
                    xs = x if which == 0 else -x          # different data per stream
                    dx_, dd_, dg_, db_ = dev(gpu, xs, "f32"), dev(gpu, d, "f32"), dev(gpu, g, "f32"), dev(gpu, b, "f32")
                    (y, _), back = gpu.pullback(gpu.batchnorm, dx_, dg_, db_, None, None, True, "relu", 0.1, 1e-5)
                    grads = back(dd_)
                    y2, back2 = gpu.pullback(gpu.groupnorm, dx_, dg_, db_, 2, "identity", 1e-5)
                    grads2 = back2(dd_)
                    keep.append((dx_, dd_, dg_, db_, back, back2))
                    results[which].append((xs, d, g, b, y, grads, y2, grads2))
        for stream in (main, other):
            gpu._lib.call("luxhip_stream_synchronize", stream)
    finally:
        gpu.set_stream(main)
    for which in (0, 1):
        for xs, d, g, b, y, grads, y2, grads2 in results[which]:
            want_y = O.batchnorm(f64(xs), f64(g), f64(b), None, None, True, "relu", 0.1, 1e-5)[0]
            assert_close(y.to_numpy(), want_y, "f32", "batchnorm y")
            assert_close(y2.to_numpy(), O.groupnorm(f64(xs), f64(g), f64(b), 2, "identity", 1e-5), "f32", "groupnorm y")
            wg = O.groupnorm_pullback(f64(xs), f64(g), f64(b), 2, "identity", 1e-5, f64(d))
            for got, w_, name in zip(grads2, wg, ("dx", "dgamma", "dbeta")):
                assert_close(got.to_numpy(), w_, "f32", "groupnorm " + name, scale=float(np.abs(d).mean()) * 4)
            # batchnorm: the same call alone on the main stream gives the same bits
            (y_alone, _), back = gpu.pullback(gpu.batchnorm, dev(gpu, xs, "f32"), dev(gpu, g, "f32"), dev(gpu, b, "f32"),
                                              None, None, True, "relu", 0.1, 1e-5)
            alone = back(dev(gpu, d, "f32"))
            np.testing.assert_array_equal(y.to_numpy(), y_alone.to_numpy())
            for got, ref in zip(grads, alone):
                np.testing.assert_array_equal(got.to_numpy(), ref.to_numpy())
    gpu._lib.call("luxhip_stream_destroy", other)


def test_pooled_allocator_reuses_blocks(gpu):
    gpu.synchronize()
    gpu._lib.call("luxhip_trim")                          # start from an empty pool
    a = gpu.DeviceArray((1 << 20,), "f32")
    ptr = a.ptr
    del a
    b = gpu.DeviceArray((1 << 20,), "f32")
    assert b.ptr == ptr                                   # the block came back from the pool
    del b
    gpu._lib.call("luxhip_trim")                          # the pool goes back to the driver; the library keeps working
    x = np.arange(12, dtype=np.float32).reshape(3, 4)
    np.testing.assert_array_equal(gpu.DeviceArray.from_numpy(x).to_numpy(), x)
    p = C.c_void_p()
    gpu._lib.call("luxhip_malloc", C.byref(p), 0)         # zero bytes: a valid call
    gpu._lib.call("luxhip_free", p)
    with pytest.raises(gpu.LuxHipError):
        gpu._lib.call("luxhip_free", C.c_void_p(0x1000))  # not a block of the pool


def test_events_time_the_stream(gpu):
    x = gpu.DeviceArray((1 << 24,), "f32")
    e0, e1 = gpu.Event(), gpu.Event()
    e0.record()
    for _ in range(10):
        gpu.bias_activation("relu", x.reshape(1 << 12, 1 << 12), None)
    e1.record()
    ms = e0.elapsed_ms(e1)
    assert 0.0 < ms < 1000.0


def test_profile_reports_the_kernels_that_ran(gpu):
    rng = np.random.default_rng(1)
    x = dev(gpu, rng.normal(size=(64, 32, 8)), "f32")
    gpu._lib.call("luxhip_profile_enable", 1)
    try:
        gpu.bias_activation("relu", x, None)
        gpu.groupnorm(x, None, None, 4)
        buf = C.create_string_buffer(1 << 16)
        gpu._lib.call("luxhip_profile_report", buf, len(buf))
    finally:
        gpu._lib.call("luxhip_profile_enable", 0)
    rows = json.loads(buf.value.decode())
    names = {r["kernel"] for r in rows}
    assert "bias_act_fwd_kernel" in names and "gn_fwd_kernel" in names
    for r in rows:
        assert r["count"] >= 1 and 0.0 < r["min_ms"] <= r["max_ms"] and r["total_ms"] >= r["max_ms"] * 0.999
    # the log was cleared by the report
    buf2 = C.create_string_buffer(1 << 12)
    gpu._lib.call("luxhip_profile_report", buf2, len(buf2))
    assert json.loads(buf2.value.decode()) == []


def test_errors_carry_a_status_and_a_message(gpu):
    with pytest.raises(gpu.LuxHipError) as err:
        gpu.set_option("no_such_option", 1)
    assert "no_such_option" in str(err.value)
    x = gpu.DeviceArray.from_numpy(np.ones((4, 6, 2), np.float32))
    with pytest.raises(gpu.Unsupported) as err:
        gpu._lib.call("luxhip_bias_activation_fwd", gpu.current_stream(), 7, 0, 4, 6, 2, x.ptr, None, x.ptr, None)   # dtype 7
    assert err.value.status == -1 and "dtype" in str(err.value)
    with pytest.raises(gpu.LuxHipError) as err:           # 6 channels do not divide into 4 groups
        gpu._lib.call("luxhip_groupnorm_fwd", gpu.current_stream(), 0, 0, 4, 6, 4, 2, x.ptr, None, None, 1e-5, x.ptr, None, None)
    assert "divisible" in str(err.value)
    # the library is still usable after the errors
    np.testing.assert_array_equal(gpu.bias_activation("relu", x, None).to_numpy(), np.ones((4, 6, 2), np.float32))


def test_exchange_word_epoch_wraps(gpu):
    """The resident batchnorm kernels and the split groupnorm pullback tag the words they exchange with a
    32-bit per-stream epoch.  Across the wrap (forced here through the test option) the words are
    cleared and results stay right, call after call."""
    rng = np.random.default_rng(21)
    shape = (32, 32, 16, 8)
    x, d = rng.normal(size=shape).astype(np.float32), rng.normal(size=shape).astype(np.float32)
    g, b = rng.uniform(0.5, 1.5, 16).astype(np.float32), rng.normal(size=16).astype(np.float32)
    want_y = O.batchnorm(f64(x), f64(g), f64(b), None, None, True, "identity", 0.1, 1e-5)[0]
    want_g = O.batchnorm_pullback(f64(x), f64(g), f64(b), "identity", 1e-5, f64(d))
    gshape = (64, 64, 16, 2)                                 # slices of 64*64*8 elements: split between two workgroups
    xg, dg_ = rng.normal(size=gshape).astype(np.float32), rng.normal(size=gshape).astype(np.float32)
    want_gn = O.groupnorm_pullback(f64(xg), f64(g), f64(b), 2, "identity", 1e-5, f64(dg_))
    dx_, dd_, dgam, dbet = dev(gpu, x, "f32"), dev(gpu, d, "f32"), dev(gpu, g, "f32"), dev(gpu, b, "f32")
    dxg, ddg = dev(gpu, xg, "f32"), dev(gpu, dg_, "f32")
    gpu.bias_activation("relu", dx_, None)                  # the stream has its workspace
    gpu.set_option("workspace_epoch", (1 << 32) - 6)
    for it in range(12):
        (y, _), back = gpu.pullback(gpu.batchnorm, dx_, dgam, dbet, None, None, True, "identity", 0.1, 1e-5)
        grads = back(dd_)
        assert_close(y.to_numpy(), want_y, "f32", f"call {it}: y")
        for got, want, name in zip(grads, want_g, ("dx", "dgamma", "dbeta")):
            assert_close(got.to_numpy(), want, "f32", f"call {it}: {name}", scale=1.0)
        _, back_g = gpu.pullback(gpu.groupnorm, dxg, dgam, dbet, 2, "identity", 1e-5)
        for got, want, name in zip(back_g(ddg), want_gn, ("dx", "dgamma", "dbeta")):
            assert_close(got.to_numpy(), want, "f32", f"call {it}: groupnorm {name}", scale=1.0)


def test_plain_c_client_of_the_abi(gpu):
    """lux.jl_amd/csrc/examples/c_client.c: a C program (no Python, no C++) that links the library and
    reproduces the Dense and BatchNorm known answers of the reference's layer tests."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(gpu.__file__), "luxhip_c_client")
    assert os.path.exists(exe), "build() compiles it next to the library"
    gpu.synchronize()
    res = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    assert res.returncode == 0 and res.stdout.strip() == "OK", res.stdout + res.stderr


def test_workspace_growth_does_not_wait_for_the_stream(gpu):
    """The stream's scratch memory grows while earlier work is still queued: the call that grows it
    returns while that work is still pending (the outgrown block is retired behind an event, nothing
    synchronises), and the operators before and after the growth give the right results."""
    rng = np.random.default_rng(11)
    hip = C.CDLL("libamdhip64.so")
    hip.hipEventQuery.argtypes = [C.c_void_p]
    HIP_ERROR_NOT_READY = 600
    stream = _new_stream(gpu)
    main = gpu.current_stream()
    gpu.set_stream(stream)
    try:
        n = 4096
        a = dev(gpu, rng.normal(size=(n, n)).astype(np.float32), "f32")
        b = dev(gpu, rng.normal(size=(n, n)).astype(np.float32), "f32")
        c = gpu.DeviceArray((n, n), "f32")
        shape = (1, 96, 4000)                      # dense layout: partial sums in the workspace
        x = rng.normal(size=shape).astype(np.float32)
        dd, dy = dev(gpu, x, "f32"), dev(gpu, np.maximum(x, 0), "f32")
        gx, gb = gpu.DeviceArray(shape, "f32"), gpu.DeviceArray((96,), "f32")
        call = lambda: gpu._lib.call("luxhip_bias_activation_bwd", stream, 0, 1, 1, 96, 4000, dd.ptr, dy.ptr, None, gx.ptr, gb.ptr)
        gpu._lib.call("luxhip_reserve", stream, 1 << 20)      # first block
        call()
        gpu._lib.call("luxhip_stream_synchronize", stream)
        want_gb = gb.to_numpy().copy()
        queued = C.c_void_p()
        gpu._lib.call("luxhip_event_create", C.byref(queued))
        # about 80 ms of fp32 products (137 GFLOP each) queued on the stream, an event behind them
        for _ in range(60):
            gpu._lib.call("luxhip_matmul", stream, 0, 0, 0, n, n, n, a.ptr, n, b.ptr, n, None, c.ptr, n)
        gpu._lib.call("luxhip_event_record", queued, stream)
        call()                                                 # uses the small block, queued behind the products
        gpu._lib.call("luxhip_reserve", stream, 96 << 20)     # outgrows it while that work is pending
        call()                                                 # runs out of the new block
        # the products queued before the growth have not finished: nothing above waited for the stream
        assert hip.hipEventQuery(queued) == HIP_ERROR_NOT_READY
        gpu._lib.call("luxhip_stream_synchronize", stream)
        assert hip.hipEventQuery(queued) == 0
        gpu._lib.call("luxhip_event_destroy", queued)
        np.testing.assert_array_equal(gb.to_numpy(), want_gb)
        # a third growth after everything has finished recycles the retired blocks through the pool
        gpu._lib.call("luxhip_reserve", stream, 200 << 20)
        call()
        gpu._lib.call("luxhip_stream_synchronize", stream)
        np.testing.assert_array_equal(gb.to_numpy(), want_gb)
    finally:
        gpu.set_stream(main)
        gpu._lib.call("luxhip_stream_destroy", stream)


def test_a_recorded_graph_keeps_its_workspace_block_after_growth(gpu):
    """A graph recorded on a stream has the address of that stream's scratch block in its kernels.  When a
    later eager call outgrows the block, the block must not go back to the allocator: a replay would write
    partial sums into whatever tensor received it."""
    hip = C.CDLL("libamdhip64.so")
    hip.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
    hip.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
    hip.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_char_p, C.c_size_t]
    hip.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
    hip.hipGraphExecDestroy.argtypes = [C.c_void_p]
    hip.hipGraphDestroy.argtypes = [C.c_void_p]
    rng = np.random.default_rng(12)
    stream = _new_stream(gpu)
    main = gpu.current_stream()
    gpu.set_stream(stream)
    graph, graph_exec = C.c_void_p(), C.c_void_p()
    try:
        shape = (1, 96, 4000)                      # dense layout: partial sums in the workspace
        x = rng.normal(size=shape).astype(np.float32)
        dd, dy = dev(gpu, x, "f32"), dev(gpu, np.maximum(x, 0), "f32")
        gx, gb = gpu.DeviceArray(shape, "f32"), gpu.DeviceArray((96,), "f32")
        call = lambda: gpu._lib.call("luxhip_bias_activation_bwd", stream, 0, 1, 1, 96, 4000, dd.ptr, dy.ptr, None, gx.ptr, gb.ptr)
        first = 8 << 20                            # the smallest block the workspace takes
        gpu._lib.call("luxhip_reserve", stream, first)
        call()
        gpu._lib.call("luxhip_stream_synchronize", stream)
        want_gb = gb.to_numpy().copy()
        assert hip.hipStreamBeginCapture(stream, 1) == 0
        try:
            call()
        finally:
            rc = hip.hipStreamEndCapture(stream, C.byref(graph))
        assert rc == 0 and graph.value
        assert hip.hipGraphInstantiate(C.byref(graph_exec), graph, None, None, 0) == 0
        gpu._lib.call("luxhip_reserve", stream, 64 << 20)     # eager growth after the recording
        call()
        gpu._lib.call("luxhip_stream_synchronize", stream)
        # tensors of the outgrown block's size: had the block been pooled, one of them would be it
        sentinels = [gpu.DeviceArray.from_numpy(np.full(first // 4, 7.0, np.float32)) for _ in range(4)]
        gb2 = gpu.DeviceArray.from_numpy(np.zeros(96, np.float32))
        gpu._lib.call("luxhip_memcpy_d2d", gb.ptr, gb2.ptr, 96 * 4, stream)       # clear the result
        for _ in range(2):
            assert hip.hipGraphLaunch(graph_exec, stream) == 0
            gpu._lib.call("luxhip_stream_synchronize", stream)
            np.testing.assert_array_equal(gb.to_numpy(), want_gb)
            for t in sentinels:
                assert (t.to_numpy() == 7.0).all()
    finally:
        if graph_exec.value:
            hip.hipGraphExecDestroy(graph_exec)
        if graph.value:
            hip.hipGraphDestroy(graph)
        gpu.set_stream(main)
        gpu._lib.call("luxhip_stream_destroy", stream)


@pytest.mark.parametrize("n,offset", [(4096, 0), (4099, 0), (8 * 1000 + 8, 1), (7, 0), (8 * 70000, 0)])
def test_storage_conversion_every_access_path(gpu, n, offset):
    """fp32 -> bf16 (round to nearest even) and back: lengths that are and are not multiples of the eight elements a
    thread converts at once, and a source that starts one element into its allocation (the element-wise kernel)."""
    rng = np.random.default_rng(n + offset)
    h = (rng.normal(size=n + offset) * 10.0 ** rng.integers(-3, 4, n + offset)).astype(np.float32)
    base = gpu.DeviceArray.from_numpy(h, "f32")
    src = gpu.DeviceArray((n,), "f32", ptr=base.ptr + offset * 4, base=base) if offset else base
    lo = gpu.DeviceArray((n,), "bf16")
    gpu._lib.call("luxhip_convert", gpu.current_stream(), src.code, lo.code, n, src.ptr, lo.ptr)
    want = O.round_to_bf16(h[offset:])
    got = lo.to_numpy()
    assert np.array_equal(np.asarray(got, np.float32), np.asarray(want, np.float32))
    back = gpu.DeviceArray((n,), "f32")
    gpu._lib.call("luxhip_convert", gpu.current_stream(), lo.code, back.code, n, lo.ptr, back.ptr)
    assert np.array_equal(back.to_numpy(), np.asarray(want, np.float32))
