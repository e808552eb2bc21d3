"""Pins the C restatement (oracle/luxlib_cpu.c, the benchmark's CPU baseline) against the
numpy oracle and the reference's batchnorm known-answer test."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

from oracle import luxlib_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SO = os.path.join(ROOT, "oracle", "libluxcpu.so")


@pytest.fixture(scope="module")
def cpu():
    if not os.path.exists(SO):
        subprocess.run(["make", "-C", os.path.join(ROOT, "oracle")], check=True)
    return C.CDLL(SO)


def P(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def F(a):
    return np.asfortranarray(a, dtype=np.float32)


@pytest.mark.parametrize("act,aid", [("identity", 0), ("relu", 1), ("tanh", 2), ("sigmoid", 3), ("swish", 4), ("gelu", 5)])
def test_bias_activation(cpu, act, aid):
    rng = np.random.default_rng(4)
    shape = (5, 3, 6, 4)
    I, Cc, N = 15, 6, 4
    x, b, delta = F(rng.normal(size=shape)), rng.normal(size=Cc).astype(np.float32), F(rng.normal(size=shape))
    y = np.empty(shape, np.float32, order="F")
    cpu.luxcpu_bias_activation_fwd(aid, C.c_int64(I), C.c_int64(Cc), C.c_int64(N), P(x), P(b), P(y))
    wy, wdx, wdb = O.bias_activation_pullback(act, x.astype(np.float64), b.astype(np.float64), delta.astype(np.float64))
    np.testing.assert_allclose(y, wy, rtol=2e-6, atol=2e-6)
    pre = F(x + b.reshape(1, 1, Cc, 1))
    dx, db = np.empty(shape, np.float32, order="F"), np.empty(Cc, np.float32)
    cpu.luxcpu_bias_activation_bwd(aid, C.c_int64(I), C.c_int64(Cc), C.c_int64(N), P(delta), P(y), P(pre), P(dx), P(db))
    np.testing.assert_allclose(dx, wdx, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(db, wdb, rtol=1e-5, atol=1e-4)


def test_batchnorm_known_answer_and_oracle(cpu):
    # test/core_layers/normalize_tests.jl:10-49 of the reference
    x = F(np.array([[1.0, 3.0, 5.0], [2.0, 4.0, 6.0]]))
    y = np.empty((2, 3), np.float32, order="F")
    g, b, rm, rv = np.ones(2, np.float32), np.zeros(2, np.float32), np.zeros(2, np.float32), np.ones(2, np.float32)
    rmo, rvo, mean, var = (np.empty(2, np.float32) for _ in range(4))
    cpu.luxcpu_batchnorm_train_fwd(0, C.c_int64(1), C.c_int64(2), C.c_int64(3), P(x), P(g), P(b), P(rm), P(rv),
                                   C.c_float(0.1), C.c_float(1e-5), P(y), P(rmo), P(rvo), P(mean), P(var))
    np.testing.assert_allclose(y, [[-1.22474, 0, 1.22474]] * 2, atol=1e-5)
    np.testing.assert_allclose(rmo, [0.3, 0.4], rtol=1e-6)
    np.testing.assert_allclose(rvo, [1.3, 1.3], rtol=1e-6)

    rng = np.random.default_rng(8)
    shape = (6, 5, 4, 7)
    I, Cc, N = 30, 4, 7
    x = F(0.5 + 2 * rng.normal(size=shape))
    g, b = rng.uniform(0.5, 1.5, Cc).astype(np.float32), rng.normal(size=Cc).astype(np.float32)
    rm, rv = rng.normal(size=Cc).astype(np.float32), rng.uniform(0.5, 2, Cc).astype(np.float32)
    dy = F(rng.normal(size=shape))
    y = np.empty(shape, np.float32, order="F")
    rmo, rvo, mean, var, dg, db = (np.empty(Cc, np.float32) for _ in range(6))
    cpu.luxcpu_batchnorm_train_fwd(0, C.c_int64(I), C.c_int64(Cc), C.c_int64(N), P(x), P(g), P(b), P(rm), P(rv),
                                   C.c_float(0.1), C.c_float(1e-5), P(y), P(rmo), P(rvo), P(mean), P(var))
    f8 = lambda a: a.astype(np.float64)
    wy, wrm, wrv = O.batchnorm(f8(x), f8(g), f8(b), f8(rm), f8(rv), True, "identity", 0.1, 1e-5)
    np.testing.assert_allclose(y, wy, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(rmo, wrm, rtol=1e-5)
    np.testing.assert_allclose(rvo, wrv, rtol=1e-5)
    dx = np.empty(shape, np.float32, order="F")
    cpu.luxcpu_batchnorm_train_bwd(C.c_int64(I), C.c_int64(Cc), C.c_int64(N), P(dy), P(x), P(g), P(mean), P(var),
                                   C.c_float(1e-5), P(dx), P(dg), P(db))
    wdx, wdg, wdb = O.batchnorm_pullback(f8(x), f8(g), f8(b), "identity", 1e-5, f8(dy))
    np.testing.assert_allclose(dx, wdx, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(dg, wdg, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(db, wdb, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("act,aid", [("identity", 0), ("relu", 1), ("swish", 4)])
def test_groupnorm_against_the_numpy_oracle(cpu, act, aid):
    """The C port of groupnorm (benchmark baseline of the groupnorm workload) against the numpy oracle,
    which torch's group_norm and finite differences pin."""
    rng = np.random.default_rng(21)
    shape = (5, 4, 6, 3)
    I, Cc, G, N = 20, 6, 3, 3
    x, delta = F(rng.normal(size=shape) * 1.5 + 0.2), F(rng.normal(size=shape))
    g, b = rng.uniform(0.8, 1.2, Cc).astype(np.float32), (0.05 * rng.normal(size=Cc)).astype(np.float32)
    y, dx = np.empty(shape, np.float32, order="F"), np.empty(shape, np.float32, order="F")
    mean, var = np.empty(G * N, np.float32), np.empty(G * N, np.float32)
    dg, db = np.empty(Cc, np.float32), np.empty(Cc, np.float32)
    i64 = C.c_int64
    cpu.luxcpu_groupnorm_fwd(aid, i64(I), i64(Cc // G), i64(G), i64(N), P(x), P(g), P(b), C.c_float(1e-5), P(y), P(mean), P(var))
    f8 = lambda a: a.astype(np.float64)
    wy = O.groupnorm(f8(x), f8(g), f8(b), G, act, 1e-5)
    np.testing.assert_allclose(y, wy, rtol=2e-5, atol=2e-5)
    if act == "relu":
        pre = O.groupnorm(f8(x), f8(g), f8(b), G, "identity", 1e-5)
        delta[np.abs(pre) < 1e-3] = 0
    cpu.luxcpu_groupnorm_bwd(aid, i64(I), i64(Cc // G), i64(G), i64(N), P(delta), P(x), P(g), P(b), P(mean), P(var), C.c_float(1e-5),
                             P(dx), P(dg), P(db))
    wdx, wdg, wdb = O.groupnorm_pullback(f8(x), f8(g), f8(b), G, act, 1e-5, f8(delta))
    np.testing.assert_allclose(dx, wdx, rtol=2e-4, atol=2e-5)
    np.testing.assert_allclose(dg, wdg, rtol=2e-4, atol=2e-4)
    np.testing.assert_allclose(db, wdb, rtol=2e-4, atol=2e-4)
