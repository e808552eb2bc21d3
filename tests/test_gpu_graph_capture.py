"""The operators enqueue on the caller's stream without synchronising or allocating from the driver
(after a warm-up has sized the stream's workspace), so a caller can record a training step into a HIP
graph and replay it.  One step of every fused operator (forward + pullback) is captured once and
replayed with new input data, with eager work and synchronisations between the replays; every replay
is checked against the oracle.  While a stream captures, batchnorm and groupnorm take the code paths
that do not tag exchange words with the per-call epoch (a replay would find its own words again)."""
import ctypes as C

import numpy as np
import pytest

from oracle import luxlib_oracle as O
from tests.util import assert_close, f64

pytestmark = pytest.mark.gpu

THREAD_LOCAL = 1      # hipStreamCaptureModeThreadLocal


def _hip():
    hip = C.CDLL("libamdhip64.so")
    hip.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
    hip.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
    hip.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_char_p, C.c_size_t]
    hip.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
    hip.hipGraphExecDestroy.argtypes = [C.c_void_p]
    hip.hipGraphDestroy.argtypes = [C.c_void_p]
    return hip


def _upload(gpu, arr, host):
    host = np.ascontiguousarray(np.asarray(host, np.float32).ravel(order="F"))
    gpu._lib.call("luxhip_memcpy_h2d", arr.ptr, host.ctypes.data, host.nbytes, gpu.current_stream())


def test_a_training_step_replays_from_a_graph(gpu):
    hip = _hip()
    rng = np.random.default_rng(31)
    d = lambda a: gpu.DeviceArray.from_numpy(np.asarray(a, np.float32))
    shape = (32, 32, 16, 8)                       # batchnorm: resident kernels when run eagerly
    gshape = (64, 64, 16, 2)                      # groupnorm pullback: split slices when run eagerly
    host = {
        "x": rng.normal(size=shape), "delta": rng.normal(size=shape), "g": rng.uniform(0.5, 1.5, 16), "b": rng.normal(size=16),
        "bias": rng.normal(size=16), "xg": rng.normal(size=gshape), "dg": rng.normal(size=gshape),
        "w": rng.normal(size=(96, 64)) / 8, "xd": rng.normal(size=(64, 40)), "bd": rng.normal(size=96), "dd": rng.normal(size=(96, 40)),
        "xl": rng.normal(size=(128, 48)), "gl": rng.uniform(0.5, 1.5, (128, 1)), "bl": rng.normal(size=(128, 1)), "dl": rng.normal(size=(128, 48)),
        "cw": rng.normal(size=(3, 3, 8, 16)) / 8, "cx": rng.normal(size=(12, 12, 8, 3)), "cb": rng.normal(size=16),
        "cd": rng.normal(size=(12, 12, 16, 3)),
    }
    host = {k: np.asarray(v, np.float32) for k, v in host.items()}
    dev_ = {k: d(v) for k, v in host.items()}
    cdims = gpu.DenseConvDims(host["cx"].shape, host["cw"].shape, padding=1)

    def step():
        out = {}
        (y, _), bn_back = gpu.pullback(gpu.batchnorm, dev_["x"], dev_["g"], dev_["b"], None, None, True, "identity", 0.1, 1e-5)
        z, act_back = gpu.pullback(gpu.bias_activation, "relu", y, dev_["bias"])
        dy, out["dbias"] = act_back(dev_["delta"])
        out["z"] = z
        out["bn_dx"], out["bn_dg"], out["bn_db"] = bn_back(dy)
        out["gn_y"], gn_back = gpu.pullback(gpu.groupnorm, dev_["xg"], dev_["g"], dev_["b"], 2, "swish", 1e-5)
        out["gn_dx"], out["gn_dg"], out["gn_db"] = gn_back(dev_["dg"])
        out["dense_y"], dense_back = gpu.pullback(gpu.fused_dense_bias_activation, "gelu", dev_["w"], dev_["xd"], dev_["bd"])
        out["dense_dw"], out["dense_dx"], out["dense_db"] = dense_back(dev_["dd"])
        out["ln_y"], ln_back = gpu.pullback(gpu.layernorm, dev_["xl"], dev_["gl"], dev_["bl"], "tanh", gpu.DEFAULT_DIMS, 1e-5)
        out["ln_dx"], out["ln_dg"], out["ln_db"] = ln_back(dev_["dl"])
        out["conv_y"], conv_back = gpu.pullback(gpu.fused_conv_bias_activation, "relu", dev_["cw"], dev_["cx"], dev_["cb"], cdims)
        out["conv_dw"], out["conv_dx"], out["conv_db"] = conv_back(dev_["cd"])
        return out, (bn_back, act_back, gn_back, dense_back, ln_back, conv_back, y, dy)

    def expected():
        h = {k: f64(v) for k, v in host.items()}
        e = {}
        y = O.batchnorm(h["x"], h["g"], h["b"], None, None, True, "identity", 0.1, 1e-5)[0]
        e["z"], dy, e["dbias"] = O.bias_activation_pullback("relu", y, h["bias"], h["delta"])
        e["bn_dx"], e["bn_dg"], e["bn_db"] = O.batchnorm_pullback(h["x"], h["g"], h["b"], "identity", 1e-5, dy)
        e["gn_y"] = O.groupnorm(h["xg"], h["g"], h["b"], 2, "swish", 1e-5)
        e["gn_dx"], e["gn_dg"], e["gn_db"] = O.groupnorm_pullback(h["xg"], h["g"], h["b"], 2, "swish", 1e-5, h["dg"])
        e["dense_y"], e["dense_dw"], e["dense_dx"], e["dense_db"] = O.fused_dense_pullback("gelu", h["w"], h["xd"], h["bd"], h["dd"])
        e["ln_y"] = O.layernorm(h["xl"], h["gl"], h["bl"], "tanh", (0,), 1e-5)
        e["ln_dx"], e["ln_dg"], e["ln_db"] = O.layernorm_pullback(h["xl"], h["gl"], h["bl"], "tanh", (0,), 1e-5, h["dl"])
        od = O.ConvDims(host["cx"].shape, host["cw"].shape, 1, 1, 1)
        e["conv_y"], e["conv_dw"], e["conv_dx"], e["conv_db"] = O.fused_conv_pullback("relu", h["cw"], h["cx"], h["cb"], od, h["cd"])
        return e

    def compare(outs, what):
        want = expected()
        for k, got in outs.items():
            w = want[k]
            assert_close(got.to_numpy(), w, "f32", f"{what}: {k}", scale=float(np.sqrt(np.mean(np.square(w)))) + 1e-3)

    stream = gpu.current_stream()
    # everything the program allocates is allocated before the capture: blocks that the host layer
    # releases while it records (its temporaries) go back to the pool, and what the pool hands out
    # afterwards may be memory that the graph writes on every replay
    other = d(rng.normal(size=(64, 64, 8)))
    for _ in range(2):                            # warm-up: sizes the workspace, fills the pool with the blocks a step needs
        outs, keep = step()
        gpu.synchronize()
    compare(outs, "eager")
    del outs, keep
    assert hip.hipStreamBeginCapture(stream, THREAD_LOCAL) == 0
    try:
        outs, keep = step()                       # recorded, not run; the arrays stay alive as long as the graph
    finally:
        graph = C.c_void_p()
        rc = hip.hipStreamEndCapture(stream, C.byref(graph))
    assert rc == 0 and graph.value
    graph_exec = C.c_void_p()
    assert hip.hipGraphInstantiate(C.byref(graph_exec), graph, None, None, 0) == 0
    try:
        for replay in range(3):
            for k in ("x", "delta", "xg", "dg", "xd", "dd", "xl", "dl", "cx", "cd"):     # new data in the same buffers
                host[k] = rng.normal(size=host[k].shape).astype(np.float32)
                _upload(gpu, dev_[k], host[k])
            gpu.groupnorm(other, None, None, 4)   # the program's own eager work between replays
            gpu.synchronize()
            assert hip.hipGraphLaunch(graph_exec, stream) == 0
            gpu.synchronize()
            compare(outs, f"replay {replay}")
    finally:
        hip.hipGraphExecDestroy(graph_exec)
        hip.hipGraphDestroy(graph)
