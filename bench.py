#!/usr/bin/env python3
"""Benchmark of the LuxLib fused-operator path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C2]

A "step" is one forward + pullback pass of the workload's operator chain over one batch of
synthetic input that is already resident in HBM.  Prints ONE JSON line (see the README of the
benchmark contract): whole-job throughput in the workload's roofline unit, the roofline of
the dominant kernel (per-kernel durations measured with HIP events on the launch stream) and
a CPU baseline (the C restatement of LuxLib's CPU loops, timed on this host).
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from __graft_entry__ import load_package  # noqa: E402

PEAK_HBM_GBS = 8000.0                 # MI355X HBM3E
PEAK_MFMA_TFLOPS = {"bf16": 2500.0, "f32": 157.3}
# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs scaled by a copy of known
# size (profiles/*_hbm_traffic_pmc.md hold the commands and the raw counter values).
MEASURED_TRAFFIC = {
    ("C2", "bn_fwd_resident_kernel"): 67769957,
    ("C2", "bias_act_fwd_kernel"): 67141018,
    ("C2", "bias_act_bwd_channel_kernel"): 100903236,
    ("C2", "bn_bwd_resident_kernel"): 100990363,
    ("C3", "gn_fwd_kernel"): 134388357,
    ("C3", "gn_bwd_kernel"): 202241307,
    ("C3bf16", "gn_fwd_kernel"): 67319219,
    ("C3bf16", "gn_bwd_kernel"): 101392385,
    ("IN", "gn_fwd_kernel"): 135504475,
    ("IN", "gn_bwd_kernel"): 202878042,
    ("DROPOUT", "dropout_fwd_kernel"): 100695641,      # dropout_rng_kernel<float, 4, 2> in the trace
    ("DROPOUT", "dropout_mul_kernel"): 100691812,
    # contractions (profiles/c4_gemm_mfma_lds_pmc.md, profiles/c5_conv_bf16_mfma_lds_pmc.md): reads + writes that
    # left the per-XCD L2s, mean per launch; much of the GEMM's comes from the Infinity Cache rather than HBM
    ("C4", "dense_gemm_kernel<bf16>"): 1557583872,
    ("C5bf16", "conv_wgrad_kernel<bf16>"): 140685312,
    ("C5bf16", "conv_fprop_kernel<bf16>"): 137945088,
    ("C5bf16", "conv_dgrad_kernel<bf16>"): 137945088,
}
METRIC = "fwd+bwd TFLOP/s & HBM GB/s (% MI355X roofline) per LuxLib fused op, 1 GPU"


# ----------------------------------------------------------------------------- workloads
class Workload:
    name = ""
    dtype = "f32"
    bound = "hbm"            # "hbm" -> GB/s, "mfma" -> TFLOP/s
    description = ""

    def setup(self, lux):
        raise NotImplementedError

    def step(self):
        raise NotImplementedError

    def work_per_step(self) -> float:
        """Algorithmic bytes (hbm) or flops (mfma) of one step."""
        raise NotImplementedError

    def kernel_work(self) -> dict:
        """kernel name -> algorithmic bytes/flops of ONE launch."""
        return {}

    def cpu_baseline(self, budget_s: float):
        return None


class C2BatchnormBiasAct(Workload):
    """benchmark configuration 2: batchnorm (training, running stats updated) then bias_activation(relu),
    forward and pullback, fp32, x 32x32x64x128."""
    name = "C2"
    dtype = "f32"
    bound = "hbm"
    description = "batchnorm(train)+bias_activation(relu) fwd+bwd, x 32x32x64x128 fp32"
    shape = (32, 32, 64, 128)

    def host_inputs(self):
        rng = np.random.default_rng(1001)
        W, H, Cc, N = self.shape
        return dict(
            x=(0.5 + 2.0 * rng.standard_normal(size=self.shape, dtype=np.float32)),
            gamma=rng.uniform(0.5, 1.5, Cc).astype(np.float32),
            beta=(0.1 * rng.standard_normal(Cc)).astype(np.float32),
            rmean=np.zeros(Cc, np.float32), rvar=np.ones(Cc, np.float32),
            bias2=(0.1 * rng.standard_normal(Cc)).astype(np.float32),
            delta=rng.standard_normal(size=self.shape, dtype=np.float32),
        )

    def setup(self, lux):
        self.lux = lux
        lib = lux._lib.load()
        W, H, Cc, N = self.shape
        self.I, self.C, self.N = W * H, Cc, N
        h = self.host_inputs()
        d = lux.DeviceArray.from_numpy
        self.sm, self.si = lux.StatArray(Cc), lux.StatArray(Cc)
        # --rotate N: N sets of the six large tensors, used in turn, so that no step finds a tensor of the step
        # before it in a cache (the working set becomes N x 201 MB)
        self.sets = []
        for _ in range(max(int(getattr(self, "rotate", 1)), 1)):
            t = {k: d(v) for k, v in h.items()}
            for k in ("y1", "y2", "dy1", "dx"):
                t[k] = lux.DeviceArray(self.shape, "f32")
            for k in ("rmean_out", "rvar_out", "dgamma", "dbeta", "dbias2"):
                t[k] = lux.DeviceArray((Cc,), "f32")
            self.sets.append((t,) + self._calls(lib, lux, t))
        self.t, self.calls, self.fused_calls = self.sets[0]
        self.turn = 0

    def _calls(self, lib, lux, t):
        s = lux.current_stream()
        Cc = self.C
        vp = C.c_void_p
        p = lambda k: vp(t[k].ptr)
        I, Cc_, N_ = C.c_int64(self.I), C.c_int64(self.C), C.c_int64(self.N)
        f32, ident, relu = 0, 0, 1
        calls = [
            (lib.luxhip_batchnorm_fwd, (s, f32, ident, I, Cc_, N_, p("x"), p("gamma"), p("beta"), p("rmean"), p("rvar"), 1,
                                        C.c_double(0.1), C.c_double(1e-5), p("y1"), p("rmean_out"), p("rvar_out"),
                                        vp(self.sm.ptr), vp(self.si.ptr))),
            (lib.luxhip_bias_activation_fwd, (s, f32, relu, I, Cc_, N_, p("y1"), p("bias2"), p("y2"), None)),
            (lib.luxhip_bias_activation_bwd, (s, f32, relu, I, Cc_, N_, p("delta"), p("y2"), None, p("dy1"), p("dbias2"))),
            (lib.luxhip_batchnorm_bwd, (s, f32, ident, I, Cc_, N_, p("dy1"), p("x"), p("gamma"), p("beta"), vp(self.sm.ptr),
                                        vp(self.si.ptr), 1, p("dx"), p("dgamma"), p("dbeta"))),
        ]
        # fused variant: batchnorm(..., relu) forward + pullback
        fused_calls = [
            (lib.luxhip_batchnorm_fwd, (s, f32, relu, I, Cc_, N_, p("x"), p("gamma"), p("beta"), p("rmean"), p("rvar"), 1,
                                        C.c_double(0.1), C.c_double(1e-5), p("y2"), p("rmean_out"), p("rvar_out"),
                                        vp(self.sm.ptr), vp(self.si.ptr))),
            (lib.luxhip_batchnorm_bwd, (s, f32, relu, I, Cc_, N_, p("delta"), p("x"), p("gamma"), p("beta"), vp(self.sm.ptr),
                                        vp(self.si.ptr), 1, p("dx"), p("dgamma"), p("dbeta"))),
        ]
        return calls, fused_calls

    def step(self):
        if len(self.sets) > 1:
            self.turn = (self.turn + 1) % len(self.sets)
            self.calls = self.sets[self.turn][1]
        for fn, args in self.calls:
            rc = fn(*args)
            if rc != 0:
                raise RuntimeError(self.lux._lib.last_error())

    def rotating_step(self):
        self.step()

    def isolated_ops(self):
        """kernel name -> call that launches exactly that kernel (default library options); successive calls go
        through the sets of tensors in turn, like rotating_step()."""
        names = ["bn_fwd_resident_kernel", "bias_act_fwd_kernel", "bias_act_bwd_channel_kernel", "bn_bwd_resident_kernel"]
        turn = [0]

        def one(i):
            def call():
                turn[0] = (turn[0] + 1) % len(self.sets)
                fn, args = self.sets[turn[0]][1][i]
                if fn(*args) != 0:
                    raise RuntimeError(self.lux._lib.last_error())
            return call
        return {n: one(i) for i, n in enumerate(names)}

    def step_fused(self):
        for fn, args in self.fused_calls:
            rc = fn(*args)
            if rc != 0:
                raise RuntimeError(self.lux._lib.last_error())

    def rotating_step_fused(self):
        self.turn = (self.turn + 1) % len(self.sets)
        self.fused_calls = self.sets[self.turn][2]
        self.step_fused()

    @property
    def E(self):
        return int(np.prod(self.shape)) * 4

    def work_per_step(self):
        # bn fwd 2E + relu fwd 2E + relu bwd 3E + bn bwd 3E (each API-level tensor read/written once)
        return 10 * self.E

    def work_per_step_fused(self):
        return 5 * self.E        # fwd: x in, y out; bwd: delta, x in, dx out

    def kernel_work(self):
        E = self.E
        return {"bn_fwd_resident_kernel": 2 * E, "bn_bwd_resident_kernel": 3 * E,
                "bn_stats_kernel": 1 * E, "bn_apply_kernel": 2 * E, "bias_act_fwd_kernel": 2 * E,
                "bias_act_bwd_channel_kernel": 3 * E, "bn_bwd_reduce_kernel": 2 * E, "bn_bwd_apply_kernel": 3 * E}

    def cpu_baseline(self, budget_s: float):
        path = os.path.join(ROOT, "oracle", "libluxcpu.so")
        if not os.path.exists(path):
            return None
        cpu = C.CDLL(path)
        cpu.luxcpu_num_threads.restype = C.c_int
        h = self.host_inputs()
        W, H, Cc, N = self.shape
        I = W * H
        fa = lambda a: np.asfortranarray(a, dtype=np.float32)
        x, delta = fa(h["x"]), fa(h["delta"])
        y1, y2, dy1, dx = (np.empty(self.shape, np.float32, order="F") for _ in range(4))
        mean, var, rmo, rvo, dg, db, db2 = (np.empty(Cc, np.float32) for _ in range(7))
        ptr = lambda a: a.ctypes.data_as(C.c_void_p)
        i64 = C.c_int64

        def cpu_step():
            cpu.luxcpu_batchnorm_train_fwd(0, i64(I), i64(Cc), i64(N), ptr(x), ptr(h["gamma"]), ptr(h["beta"]), ptr(h["rmean"]),
                                           ptr(h["rvar"]), C.c_float(0.1), C.c_float(1e-5), ptr(y1), ptr(rmo), ptr(rvo),
                                           ptr(mean), ptr(var))
            cpu.luxcpu_bias_activation_fwd(1, i64(I), i64(Cc), i64(N), ptr(y1), ptr(h["bias2"]), ptr(y2))
            cpu.luxcpu_bias_activation_bwd(1, i64(I), i64(Cc), i64(N), ptr(delta), ptr(y2), None, ptr(dy1), ptr(db2))
            cpu.luxcpu_batchnorm_train_bwd(i64(I), i64(Cc), i64(N), ptr(dy1), ptr(x), ptr(h["gamma"]), ptr(mean), ptr(var),
                                           C.c_float(1e-5), ptr(dx), ptr(dg), ptr(db))

        cpu_step()                      # warm-up / page-in
        t0 = time.perf_counter()
        n = 0
        while True:
            cpu_step()
            n += 1
            if time.perf_counter() - t0 > budget_s or n >= 200:
                break
        dt = (time.perf_counter() - t0) / n
        threads = int(cpu.luxcpu_num_threads())
        return {"value": self.work_per_step() / dt / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
                "ms_per_step": dt * 1e3,
                "sample": f"{n} full-size steps of the same chain (C port of LuxLib's CPU loops; like LuxLib, only the "
                          f"normalise loop is threaded: {threads} OpenMP threads; all other passes are serial SIMD loops)"}


class _ApiWorkload(Workload):
    """Workloads driven through the host API mirror (pullback closures); outputs come from the
    library's pooled allocator, so no hipMalloc happens inside the timed region."""

    def setup(self, lux):
        self.lux = lux
        # rotate > 1: that many sets of input tensors, used in turn by rotating_step()
        self._sets = []
        for _ in range(max(int(getattr(self, "rotate", 1)), 1)):
            self.build(lux)
            self._sets.append({k: v for k, v in vars(self).items() if isinstance(v, lux.DeviceArray)})
        self._turn = 0
        self.step()               # allocate pool blocks and workspaces once

    def rotating_step(self):
        self._turn = (self._turn + 1) % len(self._sets)
        self.__dict__.update(self._sets[self._turn])
        self.step()

    def d(self, a, dtype=None):
        return self.lux.DeviceArray.from_numpy(a, dtype or self.storage)

    @property
    def storage(self):
        return "bf16" if self.dtype == "bf16" else "f32"


class C1Dense(_ApiWorkload):
    """benchmark configuration 1: fused_dense_bias_activation 128 -> 256, batch 64, tanh, fp32."""
    name, dtype, bound = "C1", "f32", "mfma"
    description = "fused_dense_bias_activation(tanh) fwd+bwd, W 256x128, x 128x64 fp32 (latency-bound)"

    def build(self, lux):
        rng = np.random.default_rng(1000)
        lim = np.sqrt(6.0 / 384.0)
        self.W = self.d(rng.uniform(-lim, lim, size=(256, 128)).astype(np.float32))
        self.x = self.d(rng.standard_normal(size=(128, 64)).astype(np.float32))
        self.b = self.d((0.01 * rng.standard_normal(256)).astype(np.float32))
        self.delta = self.d(rng.standard_normal(size=(256, 64)).astype(np.float32))

    def step(self):
        y, back = self.lux.pullback(self.lux.fused_dense_bias_activation, "tanh", self.W, self.x, self.b)
        back(self.delta)

    def work_per_step(self):
        return 3 * 2.0 * 256 * 128 * 64

    def kernel_work(self):
        return {"dense_gemm_kernel<f32>": 2.0 * 256 * 128 * 64}

    def cpu_baseline(self, budget_s: float):
        """The reference's CPU path for this op is `matmuladd` through BLAS + a fused bias/activation loop and, in
        the pullback, two BLAS products with a transposed operand (impl/dense.jl:71-113): the same calls in numpy."""
        rng = np.random.default_rng(1000)
        lim = np.sqrt(6.0 / 384.0)
        W = rng.uniform(-lim, lim, size=(256, 128)).astype(np.float32)
        x = rng.standard_normal(size=(128, 64)).astype(np.float32)
        b = (0.01 * rng.standard_normal(256)).astype(np.float32)
        delta = rng.standard_normal(size=(256, 64)).astype(np.float32)

        def cpu_step():
            y = np.tanh(W @ x + b[:, None])
            dz = delta * (1.0 - y * y)
            return dz @ x.T, W.T @ dz, dz.sum(axis=1)

        return _time_cpu(cpu_step, budget_s, self.work_per_step(), 1e12, "TFLOP/s", blas_threads(), "port",
                         "full-size steps in numpy fp32 (BLAS products + elementwise loops, the structure of LuxLib's CPU path)")


class C3Groupnorm(_ApiWorkload):
    """benchmark configuration 3: groupnorm(32 groups) + swish, x 64x64x256x16."""
    name, bound = "C3", "hbm"
    shape, groups = (64, 64, 256, 16), 32

    def __init__(self, dtype="f32"):
        self.dtype = dtype
        self.name = "C3" if dtype == "f32" else "C3bf16"
        self.description = f"groupnorm(32 groups, swish) fwd+bwd, x 64x64x256x16 {dtype}"

    def build(self, lux):
        rng = np.random.default_rng(1002)
        self.x = self.d(rng.standard_normal(size=self.shape, dtype=np.float32))
        self.g = self.d(rng.uniform(0.8, 1.2, 256).astype(np.float32))
        self.b = self.d((0.05 * rng.standard_normal(256)).astype(np.float32))
        self.delta = self.d(rng.standard_normal(size=self.shape, dtype=np.float32))

    def step(self):
        y, back = self.lux.pullback(self.lux.groupnorm, self.x, self.g, self.b, self.groups, "swish", 1e-5)
        back(self.delta)

    @property
    def E(self):
        return int(np.prod(self.shape)) * (4 if self.dtype == "f32" else 2)

    def work_per_step(self):
        return 5 * self.E        # fwd: x in, y out; bwd: delta, x in, dx out

    def kernel_work(self):
        return {"gn_fwd_kernel": 2 * self.E, "gn_bwd_kernel": 3 * self.E}

    def cpu_baseline(self, budget_s: float):
        path = os.path.join(ROOT, "oracle", "libluxcpu.so")
        if not os.path.exists(path):
            return None
        cpu = C.CDLL(path)
        rng = np.random.default_rng(1002)
        fa = lambda a: np.asfortranarray(a, dtype=np.float32)
        x = fa(rng.standard_normal(size=self.shape, dtype=np.float32))
        g = rng.uniform(0.8, 1.2, 256).astype(np.float32)
        b = (0.05 * rng.standard_normal(256)).astype(np.float32)
        delta = fa(rng.standard_normal(size=self.shape, dtype=np.float32))
        W, H, Cc, N = self.shape
        G = self.groups
        y, dx = np.empty(self.shape, np.float32, order="F"), np.empty(self.shape, np.float32, order="F")
        mean, var = np.empty(G * N, np.float32), np.empty(G * N, np.float32)
        dg, db = np.empty(Cc, np.float32), np.empty(Cc, np.float32)
        ptr = lambda a: a.ctypes.data_as(C.c_void_p)
        i64 = C.c_int64

        def cpu_step():
            cpu.luxcpu_groupnorm_fwd(4, i64(W * H), i64(Cc // G), i64(G), i64(N), ptr(x), ptr(g), ptr(b), C.c_float(1e-5), ptr(y),
                                     ptr(mean), ptr(var))
            cpu.luxcpu_groupnorm_bwd(4, i64(W * H), i64(Cc // G), i64(G), i64(N), ptr(delta), ptr(x), ptr(g), ptr(b), ptr(mean),
                                     ptr(var), C.c_float(1e-5), ptr(dx), ptr(dg), ptr(db))

        E32 = int(np.prod(self.shape)) * 4
        return _time_cpu(cpu_step, budget_s, 5 * E32, 1e9, "GB/s", 1, "port",
                         "full-size fp32 steps of the C port of LuxLib's groupnorm CPU loops (serial @simd loops in the reference, "
                         "one thread here; the bf16 workload has no CPU counterpart in LuxLib and is compared with the same fp32 figure)")


class C4TransformerMLP(_ApiWorkload):
    """benchmark configuration 4: layernorm(4096 x 8192) -> dense 4096->11008 gelu -> dense 11008->4096,
    bf16 storage, fp32 accumulation."""
    name, dtype, bound = "C4", "bf16", "mfma"
    description = "layernorm + dense(4096->11008, gelu) + dense(11008->4096) fwd+bwd, 8192 tokens, bf16/fp32-acc"
    D, F, Ntok = 4096, 11008, 8192

    def build(self, lux):
        rng = np.random.default_rng(1003)
        D, F, N = self.D, self.F, self.Ntok
        std = np.sqrt(2.0 / (D + F))
        self.x = self.d(rng.standard_normal(size=(D, N), dtype=np.float32))
        self.g = self.d(rng.uniform(0.5, 1.5, (D, 1)).astype(np.float32))
        self.b = self.d((0.1 * rng.standard_normal((D, 1))).astype(np.float32))
        self.W1 = self.d(std * rng.standard_normal(size=(F, D), dtype=np.float32))
        self.b1 = self.d(np.zeros(F, np.float32))
        self.W2 = self.d(std * rng.standard_normal(size=(D, F), dtype=np.float32))
        self.b2 = self.d(np.zeros(D, np.float32))
        self.delta = self.d(0.02 * rng.standard_normal(size=(D, N), dtype=np.float32))

    def step(self):
        lux = self.lux
        h0, back_ln = lux.pullback(lux.layernorm, self.x, self.g, self.b, "identity", (1,), 1e-5)
        h1, back_d1 = lux.pullback(lux.fused_dense_bias_activation, "gelu", self.W1, h0, self.b1)
        h2, back_d2 = lux.pullback(lux.fused_dense_bias_activation, "identity", self.W2, h1, self.b2)
        dW2, dh1, db2 = back_d2(self.delta)
        dW1, dh0, db1 = back_d1(dh1)
        back_ln(dh0)

    def work_per_step(self):
        return 6 * 2.0 * self.D * self.F * self.Ntok      # six GEMMs (the metric counts GEMM flops only)

    def kernel_work(self):
        return {"dense_gemm_kernel<bf16>": 2.0 * self.D * self.F * self.Ntok}

    def cpu_baseline(self, budget_s: float):
        """LuxLib's CPU path in fp32 (it has no bf16 code): layernorm as mean/var + broadcasts, dense layers as
        BLAS products + bias/activation loops, the pullbacks as the rrules compose them, on 1/8 of the tokens."""
        rng = np.random.default_rng(1003)
        D, F, N = self.D, self.F, self.Ntok // 8
        std = np.sqrt(2.0 / (D + F))
        x = rng.standard_normal(size=(D, N), dtype=np.float32)
        g = rng.uniform(0.5, 1.5, (D, 1)).astype(np.float32)
        b = (0.1 * rng.standard_normal((D, 1))).astype(np.float32)
        W1 = std * rng.standard_normal(size=(F, D), dtype=np.float32)
        W2 = std * rng.standard_normal(size=(D, F), dtype=np.float32)
        b1, b2 = np.zeros((F, 1), np.float32), np.zeros((D, 1), np.float32)
        delta = 0.02 * rng.standard_normal(size=(D, N), dtype=np.float32)
        c0, c1 = np.float32(0.7978845608028654), np.float32(0.044715)

        def cpu_step():
            mu = x.mean(axis=0, keepdims=True)
            var = x.var(axis=0, keepdims=True)
            inv = 1.0 / np.sqrt(var + np.float32(1e-5))
            xh = (x - mu) * inv
            h0 = xh * g + b
            z1 = W1 @ h0 + b1
            t = np.tanh(c0 * (z1 + c1 * z1 ** 3))
            h1 = 0.5 * z1 * (1.0 + t)
            h2 = W2 @ h1 + b2
            dW2, dh1, db2 = delta @ h1.T, W2.T @ delta, delta.sum(axis=1)
            dz1 = dh1 * (0.5 * (1.0 + t) + 0.5 * z1 * (1.0 - t * t) * c0 * (1.0 + 3.0 * c1 * z1 * z1))
            dW1, dh0, db1 = dz1 @ h0.T, W1.T @ dz1, dz1.sum(axis=1)
            dg, dbeta = (dh0 * xh).sum(axis=1), dh0.sum(axis=1)
            gd = dh0 * g
            dx = (gd - gd.mean(axis=0, keepdims=True) - xh * (gd * xh).mean(axis=0, keepdims=True)) * inv
            return h2, dW2, db2, dW1, db1, dg, dbeta, dx

        return _time_cpu(cpu_step, budget_s, self.work_per_step() / 8, 1e12, "TFLOP/s", blas_threads(), "port",
                         f"steps of the same block on {N} of the {self.Ntok} tokens, numpy fp32 (BLAS products + elementwise "
                         "passes, the structure of LuxLib's CPU path, which has no bf16 code); GEMM flops counted as on the GPU")

    def kernel_bytes(self):
        """HBM-bound kernels of this workload: name -> algorithmic bytes of one launch."""
        E, H = 2 * self.D * self.Ntok, 2 * self.F * self.Ntok      # bytes of a (D, tokens) / (F, tokens) bf16 tensor
        return {"ln_fwd_kernel": 2 * E, "ln_bwd_fused_kernel": 3 * E, "ln_bwd_dx_kernel": 3 * E, "ln_param_grad_kernel": 2 * E,
                "whcn_to_cwhn_kernel": None,                         # operand copies: sizes differ per launch
                "bias_act_bwd_plane_kernel": None}


class C5Conv(_ApiWorkload):
    """benchmark configuration 5: fused_conv_bias_activation 3x3, 128->128, 56x56, batch 64, pad 1, relu."""
    bound = "mfma"
    xs, ws = (56, 56, 128, 64), (3, 3, 128, 128)

    def __init__(self, dtype="f32"):
        self.dtype = dtype
        self.name = "C5" if dtype == "f32" else "C5bf16"
        self.description = f"fused_conv_bias_activation(relu) 3x3 128->128, x 56x56x128x64, pad 1, fwd+bwd {dtype}"

    def build(self, lux):
        rng = np.random.default_rng(1004)
        self.cd = lux.DenseConvDims(self.xs, self.ws, padding=1)
        self.x = self.d(rng.standard_normal(size=self.xs, dtype=np.float32))
        self.w = self.d(np.sqrt(2.0 / 1152) * rng.standard_normal(size=self.ws, dtype=np.float32))
        self.b = self.d((0.01 * rng.standard_normal(128)).astype(np.float32))
        self.delta = self.d(rng.standard_normal(size=self.cd.y_shape, dtype=np.float32))

    def step(self):
        y, back = self.lux.pullback(self.lux.fused_conv_bias_activation, "relu", self.w, self.x, self.b, self.cd)
        back(self.delta)

    def work_per_step(self):
        return 3 * 2.0 * (56 * 56 * 64) * 128 * 1152

    def kernel_work(self):
        f = 2.0 * (56 * 56 * 64) * 128 * 1152
        t = "bf16" if self.dtype == "bf16" else "f32"
        return {f"conv_fprop_kernel<{t}>": f, f"conv_dgrad_kernel<{t}>": f, f"conv_wgrad_kernel<{t}>": f}

    def cpu_baseline(self, budget_s: float):
        """NNlib's CPU convolution is im2col + GEMM per image (threaded over the batch); LuxLib adds the bias /
        activation loop and, in the pullback, the activation gradient, the bias sum and the two NNlib gradients:
        the same steps in numpy fp32 on 8 of the 64 images."""
        rng = np.random.default_rng(1004)
        N = 8
        x = rng.standard_normal(size=(N, 128, 56, 56), dtype=np.float32)                  # image-major for the host loops
        w = (np.sqrt(2.0 / 1152) * rng.standard_normal(size=(128, 128, 3, 3), dtype=np.float32))
        b = (0.01 * rng.standard_normal(128)).astype(np.float32)
        delta = rng.standard_normal(size=(N, 128, 56, 56), dtype=np.float32)
        wm = np.ascontiguousarray(w[:, :, ::-1, ::-1].reshape(128, 1152))                  # true convolution: flipped taps
        from numpy.lib.stride_tricks import sliding_window_view

        def im2col(a):                                                                     # (C, 56, 56) -> (C*9, 3136), pad 1
            p = np.pad(a, ((0, 0), (1, 1), (1, 1)))
            return np.ascontiguousarray(sliding_window_view(p, (3, 3), axis=(1, 2)).transpose(0, 3, 4, 1, 2)).reshape(1152, 3136)

        def cpu_step():
            dw = np.zeros((128, 1152), np.float32)
            db = np.zeros(128, np.float32)
            for n in range(N):
                col = im2col(x[n])
                y = np.maximum(wm @ col + b[:, None], 0.0)
                dz = delta[n].reshape(128, 3136) * (y > 0)
                db += dz.sum(axis=1)
                dw += dz @ col.T
                dcol = wm.T @ dz                                                           # (1152, 3136): col2im
                d = dcol.reshape(128, 3, 3, 56, 56)
                dx = np.zeros((128, 58, 58), np.float32)
                for p in range(3):
                    for q in range(3):
                        dx[:, p:p + 56, q:q + 56] += d[:, p, q]
            return dw, db

        return _time_cpu(cpu_step, budget_s, self.work_per_step() * N / 64, 1e12, "TFLOP/s", blas_threads(), "port",
                         f"steps on {N} of the 64 images, numpy fp32: im2col + BLAS product per image (NNlib's CPU algorithm), "
                         "bias/relu loop, pullback with col2im; the bf16 workload is compared with the same fp32 figure")


class Conv3d(_ApiWorkload):
    """fused_conv_bias_activation with three spatial dims: 3x3x3, 64->128, volumes 32x32x16, batch 8, pad 1, relu.
    Runs as the two-dimensional problem on the depth-unfolded input (192 channels, 128 samples)."""
    bound = "mfma"
    xs, ws = (32, 32, 16, 64, 8), (3, 3, 3, 64, 128)

    def __init__(self, dtype="bf16"):
        self.dtype = dtype
        self.name = "CONV3D" if dtype == "bf16" else "CONV3Df32"
        self.description = f"fused_conv_bias_activation(relu) 3x3x3 64->128, x 32x32x16x64x8, pad 1, fwd+bwd {dtype}"

    def build(self, lux):
        rng = np.random.default_rng(1013)
        self.cd = lux.DenseConvDims(self.xs, self.ws, padding=1)
        self.x = self.d(rng.standard_normal(size=self.xs, dtype=np.float32))
        self.w = self.d(np.sqrt(2.0 / 1728) * rng.standard_normal(size=self.ws, dtype=np.float32))
        self.b = self.d((0.01 * rng.standard_normal(128)).astype(np.float32))
        self.delta = self.d(rng.standard_normal(size=self.cd.y_shape, dtype=np.float32))

    def step(self):
        y, back = self.lux.pullback(self.lux.fused_conv_bias_activation, "relu", self.w, self.x, self.b, self.cd)
        back(self.delta)

    def work_per_step(self):
        return 3 * 2.0 * (32 * 32 * 16 * 8) * 128 * 1728

    def kernel_work(self):
        f = 2.0 * (32 * 32 * 16 * 8) * 128 * 1728
        t = "bf16" if self.dtype == "bf16" else "f32"
        return {f"conv_fprop_kernel<{t}>": f, f"conv_dgrad_kernel<{t}>": f, f"conv_wgrad_kernel<{t}>": f}


class InstanceNorm(_ApiWorkload):
    """instancenorm (training, running statistics updated) + relu, x 64x64x256x16 fp32: one slice per channel and sample."""
    name, bound, dtype = "IN", "hbm", "f32"
    shape = (64, 64, 256, 16)
    description = "instancenorm(train, running stats, relu) fwd+bwd, x 64x64x256x16 f32"

    def build(self, lux):
        rng = np.random.default_rng(1010)
        self.x = self.d(rng.standard_normal(size=self.shape, dtype=np.float32))
        self.g = self.d(rng.uniform(0.8, 1.2, 256).astype(np.float32))
        self.b = self.d((0.05 * rng.standard_normal(256)).astype(np.float32))
        self.rm, self.rv = self.d(np.zeros(256, np.float32)), self.d(np.ones(256, np.float32))
        self.delta = self.d(rng.standard_normal(size=self.shape, dtype=np.float32))

    def step(self):
        _, back = self.lux.pullback(self.lux.instancenorm, self.x, self.g, self.b, self.rm, self.rv, True, "relu", 0.1, 1e-5)
        back(self.delta)

    def work_per_step(self):
        return 5 * 4 * int(np.prod(self.shape))

    def kernel_work(self):
        E = 4 * int(np.prod(self.shape))
        return {"gn_fwd_kernel": 2 * E, "gn_bwd_kernel": 3 * E}


class Dropout(_ApiWorkload):
    """dropout(p = 0.5) with a full-size mask, forward (x in, y and mask out) + pullback (delta, mask in, dx out)."""
    name, bound, dtype = "DROPOUT", "hbm", "f32"
    shape = (32, 32, 64, 128)
    description = "dropout(p=0.5, dims=:) fwd+bwd, x 32x32x64x128 f32"

    def build(self, lux):
        rng = np.random.default_rng(1011)
        self.x = self.d(rng.standard_normal(size=self.shape, dtype=np.float32))
        self.delta = self.d(rng.standard_normal(size=self.shape, dtype=np.float32))
        self.rng = lux.PhiloxRNG(1, 0)

    def step(self):
        (_, _, self.rng), back = self.lux.pullback(self.lux.dropout, self.rng, self.x, 0.5, True, 2.0)
        back(self.delta)

    def work_per_step(self):
        return 6 * 4 * int(np.prod(self.shape))

    def kernel_work(self):
        E = 4 * int(np.prod(self.shape))
        return {"dropout_fwd_kernel": 3 * E, "dropout_mul_kernel": 3 * E}


class Attention(_ApiWorkload):
    """scaled_dot_product_attention, causal, 32 heads of width 128 over 2048 positions, batch 4, bf16, fwd+bwd."""
    name, bound, dtype = "SDPA", "mfma", "bf16"
    E, H, L, B = 128, 32, 2048, 4
    description = "scaled_dot_product_attention(causal) fwd+bwd, q/k/v 128x32x2048x4 bf16"

    def build(self, lux):
        rng = np.random.default_rng(1012)
        shp = (self.E, self.H, self.L, self.B)
        self.q, self.k, self.v, self.do = (self.d(rng.standard_normal(size=shp, dtype=np.float32)) for _ in range(4))

    def step(self):
        _, back = self.lux.pullback(self.lux.scaled_dot_product_attention, self.q, self.k, self.v, 1, 3, None, None, True, None)
        back(self.do)

    def work_per_step(self):
        return 6 * 2.0 * self.E * self.L * self.L * self.H * self.B     # six batched products (all positions computed)

    def kernel_work(self):
        return {"batched_gemm_kernel<bf16>": 2.0 * self.E * self.L * self.L * self.H * self.B}


WORKLOADS = {"IN": InstanceNorm, "DROPOUT": Dropout, "SDPA": Attention, "C1": C1Dense, "C2": C2BatchnormBiasAct, "C3": lambda: C3Groupnorm("f32"), "C3bf16": lambda: C3Groupnorm("bf16"),
             "C4": C4TransformerMLP, "C5": lambda: C5Conv("f32"), "C5bf16": lambda: C5Conv("bf16"),
             "CONV3D": lambda: Conv3d("bf16"), "CONV3Df32": lambda: Conv3d("f32")}


# ----------------------------------------------------------------------------- CPU baselines
def blas_threads() -> int:
    try:
        from threadpoolctl import threadpool_info
        n = [p.get("num_threads", 1) for p in threadpool_info() if p.get("user_api") == "blas"]
        return int(max(n)) if n else 1
    except Exception:
        return int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))


def _time_cpu(step, budget_s, work, scale, unit, cores, kind, sample):
    step()                                  # warm-up / page-in
    t0 = time.perf_counter()
    n = 0
    while True:
        step()
        n += 1
        if time.perf_counter() - t0 > budget_s or n >= 2000:
            break
    dt = (time.perf_counter() - t0) / n
    return {"value": work / dt / scale, "unit": unit, "cores": cores, "kind": kind, "ms_per_step": dt * 1e3,
            "sample": f"{n} {sample}"}


# ----------------------------------------------------------------------------- timing
def timed(lux, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    lux.synchronize()
    e0, e1 = lux.Event(), lux.Event()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    ms_gpu = e0.elapsed_ms(e1)          # waits for e1
    lux.synchronize()
    ms_wall = (time.perf_counter() - t0) * 1e3
    return ms_gpu / steps, ms_wall / steps


REGIONS = 3
SETTLE_S = 0.3          # untimed run-in of every workload before its timed regions (at least the warm-up steps)


def timed_regions(lux, fn, steps, warmup):
    """The warm-up, then REGIONS timed regions of `steps` steps each, back to back.  Returns the region with the
    median time (device events, host clock) and the per-step times of all regions: one sample cannot tell a slow
    box from a clock that has not settled."""
    t_warm = time.perf_counter()
    for _ in range(warmup):
        fn()
    lux.synchronize()
    # the device's clock needs a few hundred milliseconds of the workload before it settles (it is power-managed);
    # short workloads therefore keep running, untimed, until SETTLE_S have passed since the warm-up began
    while time.perf_counter() - t_warm < SETTLE_S:
        for _ in range(max(warmup, 10)):
            fn()
        lux.synchronize()
    samples = []
    for _ in range(REGIONS):
        e0, e1 = lux.Event(), lux.Event()
        t0 = time.perf_counter()
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        ms_gpu = e0.elapsed_ms(e1)          # waits for e1
        lux.synchronize()
        ms_wall = (time.perf_counter() - t0) * 1e3
        samples.append((max(ms_gpu, ms_wall) / steps, ms_gpu / steps, ms_wall / steps))
    order = sorted(samples)
    med = order[len(order) // 2]
    spread = {"regions": REGIONS, "ms_per_step_median": round(med[0], 5), "ms_per_step_min": round(order[0][0], 5),
              "ms_per_step_max": round(order[-1][0], 5), "ms_per_step_in_order": [round(x[0], 5) for x in samples]}
    return med[1], med[2], spread


def timed_graph(lux, fn, steps):
    """One step recorded into a HIP graph on the library's stream (after the eager warm-up has sized the
    workspace and filled the allocator's pool) and replayed `steps` times: the step without the host's
    per-call work.  While the stream records, batchnorm and groupnorm use their two-pass kernels."""
    hip = C.CDLL("libamdhip64.so")
    hip.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
    hip.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
    hip.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_char_p, C.c_size_t]
    hip.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
    hip.hipGraphExecDestroy.argtypes = [C.c_void_p]
    hip.hipGraphDestroy.argtypes = [C.c_void_p]
    stream = lux.current_stream()
    lux.synchronize()
    if hip.hipStreamBeginCapture(stream, 1) != 0:
        return None
    try:
        fn()
    finally:
        graph = C.c_void_p()
        rc = hip.hipStreamEndCapture(stream, C.byref(graph))
    if rc != 0 or not graph.value:
        return None
    gexec = C.c_void_p()
    if hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) != 0:
        hip.hipGraphDestroy(graph)
        return None
    for _ in range(3):
        hip.hipGraphLaunch(gexec, stream)
    lux.synchronize()
    e0, e1 = lux.Event(), lux.Event()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        hip.hipGraphLaunch(gexec, stream)
    e1.record()
    ms_gpu = e0.elapsed_ms(e1)
    lux.synchronize()
    ms_wall = (time.perf_counter() - t0) * 1e3
    hip.hipGraphExecDestroy(gexec)
    hip.hipGraphDestroy(graph)
    return max(ms_gpu, ms_wall) / steps


def kernel_profile(lux, fn, steps):
    """Per-kernel average duration from HIP events on the launch stream: the HBM-bound kernels hand two events to
    their dispatch (begin and end of the kernel itself), the others are bracketed by events recorded around the
    launch (the kernel plus the gap to its predecessor, which is negligible for kernels of hundreds of microseconds)."""
    lux._lib.call("luxhip_profile_enable", 1)
    for _ in range(steps):
        fn()
    buf = C.create_string_buffer(1 << 16)
    lux._lib.call("luxhip_profile_report", buf, len(buf))
    lux._lib.call("luxhip_profile_enable", 0)
    return json.loads(buf.value.decode())


HEAVY = ("C4", "C5", "C5bf16", "SDPA", "CONV3D", "CONV3Df32")
_CPU_DONE = {}
DEFAULT_ORDER = ["C4", "C1", "C2", "C3", "C3bf16", "C5", "C5bf16"]      # the benchmark configurations; the largest one first (headline)


def measure(lux, name, args):
    """Times one workload and returns its entry: whole-step throughput, per-kernel table, roofline of the
    dominant kernel, warm / cold figures for HBM-bound workloads, CPU baseline."""
    wl = WORKLOADS[name]()
    heavy = name in HEAVY
    steps = args.steps if args.steps is not None else (30 if heavy else 200)
    warmup = args.warmup if args.warmup is not None else (30 if heavy else 50)   # long enough for the clocks to settle
    wl.rotate = args.rotate
    wl.setup(lux)
    peak = PEAK_HBM_GBS if wl.bound == "hbm" else PEAK_MFMA_TFLOPS[wl.dtype]
    unit = "GB/s" if wl.bound == "hbm" else "TFLOP/s"
    scale = 1e9 if wl.bound == "hbm" else 1e12
    work = wl.work_per_step()

    step = wl.rotating_step if args.rotate > 1 and hasattr(wl, "rotating_step") else wl.step
    ms_gpu, ms_wall, spread = timed_regions(lux, step, steps, warmup)
    ms = max(ms_gpu, ms_wall)           # whole-job time: the slower of the device and host clocks
    ms_graph = timed_graph(lux, wl.step, steps) if args.graph else None
    warm = {"ms_per_step": round(ms, 5), "value": round(work / (ms * 1e-3) / scale, 2), "unit": unit,
            "frac_of_peak": round(work / (ms * 1e-3) / scale / peak, 4),
            "note": "every step on the same buffers (inputs may come from the 256 MB Infinity Cache)"}

    # HBM-bound workloads: the headline figure is taken on several sets of tensors used in turn, so that no step
    # finds its inputs in the Infinity Cache from the step before
    cold_wl = None
    cold = None
    if wl.bound == "hbm" and args.rotate == 1 and not args.option and args.cold_sets > 1:
        cold_wl = WORKLOADS[name]()
        cold_wl.rotate = args.cold_sets
        cold_wl.setup(lux)
        cg, cw_, spread = timed_regions(lux, cold_wl.rotating_step, steps, warmup)
        cms = max(cg, cw_)
        cold = {"sets_of_tensors": args.cold_sets, "ms_per_step": round(cms, 5), "value": round(work / (cms * 1e-3) / scale, 2),
                "unit": unit, "frac_of_peak": round(work / (cms * 1e-3) / scale / peak, 4)}
        ms_head, ms_gpu_head, ms_wall_head = cms, cg, cw_
    else:
        ms_head, ms_gpu_head, ms_wall_head = ms, ms_gpu, ms_wall
    value = work / (ms_head * 1e-3) / scale

    prof_wl = cold_wl if cold_wl is not None else wl
    prof_step = prof_wl.rotating_step if cold_wl is not None else step
    prof = kernel_profile(lux, prof_step, min(steps, 100))
    kw = wl.kernel_work()
    kernels = []
    # "<name>+tail" is a second launch that finishes the rows of <name>: one kernel's work, so its
    # time is added to <name>'s
    tails = {k["kernel"][:-5]: k for k in prof if k["kernel"].endswith("+tail")}
    prof = [dict(k) for k in prof if not k["kernel"].endswith("+tail")]
    for k in prof:
        if k["kernel"] in tails:
            k["total_ms"] += tails[k["kernel"]]["total_ms"]
            k["tail_launches"] = tails[k["kernel"]]["count"]
        avg_ms = k["total_ms"] / max(k["count"], 1)
        w = kw.get(k["kernel"])
        ent = {"kernel": k["kernel"], "avg_us": round(avg_ms * 1e3, 3), "launches": k["count"]}
        if "tail_launches" in k:
            ent["tail_launches"] = k["tail_launches"]
        if w:
            ach = w / (avg_ms * 1e-3) / scale
            ent.update({"algorithmic": w, "achieved": round(ach, 1), "frac": round(ach / peak, 4)})
        elif hasattr(wl, "kernel_bytes") and wl.kernel_bytes().get(k["kernel"]):
            # an HBM-bound kernel inside a contraction-bound workload: reported against the HBM peak
            b = wl.kernel_bytes()[k["kernel"]]
            gbs = b / (avg_ms * 1e-3) / 1e9
            ent.update({"algorithmic_bytes": b, "achieved_GBps": round(gbs, 1), "frac_of_hbm_peak": round(gbs / PEAK_HBM_GBS, 4)})
        kernels.append(ent)
    # Kernels that an API call launches alone are also timed back to back (two events around a run of identical
    # launches, on the rotating sets when those are the headline): that average is the kernel plus the gap between
    # dependent launches, reported beside avg_us.  avg_us of these kernels comes from two events that the dispatch
    # itself signals at its begin and end, which is the duration that rocprofv3 --kernel-trace reports.
    iso = prof_wl.isolated_ops() if hasattr(prof_wl, "isolated_ops") and not args.option else {}
    seen = {e["kernel"] for e in kernels}
    for kname, call in iso.items():
        if kname not in seen:
            continue
        ms_iso, _ = timed(lux, call, 64, 8)
        for e in kernels:
            if e["kernel"] == kname:
                e["avg_us_back_to_back"] = round(ms_iso * 1e3, 3)
    kernels.sort(key=lambda e: -e["avg_us"])
    dom = next((e for e in kernels if "achieved" in e), None)
    roofline = None
    if dom is not None:
        roofline = {"bound": "hbm" if wl.bound == "hbm" else "mfma", "kernel": dom["kernel"], "achieved": dom["achieved"], "peak": peak,
                    "unit": unit, "frac": dom["frac"], "traffic": MEASURED_TRAFFIC.get((wl.name, dom["kernel"])),
                    "avg_us": dom["avg_us"], "algorithmic_per_launch": dom["algorithmic"]}

    out = {
        "workload": wl.name, "description": wl.description, "dtype": wl.dtype, "bound": wl.bound, "value": round(value, 2), "unit": unit,
        "steps": steps, "warmup": warmup, "ms_per_step": round(ms_head, 5), "frac_of_peak": round(value / peak, 4),
        "ms_per_step_gpu_events": round(ms_gpu_head, 5), "ms_per_step_host_clock": round(ms_wall_head, 5),
        "timing": f"median of {REGIONS} timed regions of {steps} steps each, after {warmup} warm-up steps and an untimed run-in "
                  f"that lasts until {SETTLE_S} s have passed since the warm-up began", "spread": spread,
        "roofline": roofline, "kernels": kernels,
    }
    if cold is not None:
        out["cold_inputs"] = cold
        out["warm_inputs"] = warm
        out["inputs"] = f"{args.cold_sets} sets of tensors used in turn (value, ms_per_step, kernels); warm_inputs: one set"
    if ms_graph is not None:
        out["graph_replay"] = {"ms_per_step": round(ms_graph, 5), "speedup_over_eager": round(ms / ms_graph, 3),
                               "note": "one step recorded into a HIP graph, replayed; batchnorm/groupnorm record their two-pass kernels"}
    if hasattr(wl, "step_fused"):
        fw_ = cold_wl if cold_wl is not None else wl
        fstep = fw_.rotating_step_fused if cold_wl is not None and hasattr(fw_, "rotating_step_fused") else fw_.step_fused
        fg, fw = timed(lux, fstep, steps, warmup)
        fms = max(fg, fw)
        out["fused_variant"] = {"workload": "batchnorm(..., relu) fwd+bwd (activation fused into batchnorm)",
                                "ms_per_step": round(fms, 5), "value": round(wl.work_per_step_fused() / (fms * 1e-3) / 1e9, 2),
                                "unit": "GB/s", "algorithmic_bytes": wl.work_per_step_fused()}
    del cold_wl
    if args.cpu_seconds > 0:
        key = type(wl).__name__         # the bf16 variant of a workload has the fp32 CPU figure beside it: timed once
        if key not in _CPU_DONE:
            cb = wl.cpu_baseline(args.cpu_seconds)
            if cb is not None:
                cb["value"] = round(cb["value"], 4)
                cb["ms_per_step"] = round(cb["ms_per_step"], 3)
            _CPU_DONE[key] = cb
        if _CPU_DONE[key] is not None:
            out["cpu_baseline"] = _CPU_DONE[key]
    del wl
    lux._lib.call("luxhip_trim")            # the next workload starts from an empty pool
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps per workload (default 200, heavy workloads 30)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps per workload (default 50, heavy workloads 30)")
    ap.add_argument("--workload", default="ALL", choices=["ALL"] + sorted(WORKLOADS),
                    help="ALL (default): the benchmark configurations C1, C2, C3, C3bf16, C4, C5, C5bf16 in one run; "
                         "the headline (top-level fields) is C4, the largest one")
    ap.add_argument("--cpu-seconds", type=float, default=8.0, help="budget of each CPU baseline (0 disables them)")
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="library tuning switch (luxhip_set_option), e.g. bn_resident=0; may be repeated")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run three device-to-device copies of 256 MiB: a kernel of known traffic that "
                         "scales the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run")
    ap.add_argument("--rotate", type=int, default=1,
                    help="number of separate sets of the large tensors that the timed steps use in turn "
                         "(1 = every step on the same buffers)")
    ap.add_argument("--cold-sets", type=int, default=8,
                    help="HBM-bound workloads: the headline is timed on this many sets of tensors used in turn "
                         "(0 = one set only, e.g. under a profiler)")
    ap.add_argument("--graph", action="store_true",
                    help="also record one step into a HIP graph and time its replays (reported as graph_replay; "
                         "value stays the eager figure)")
    ap.add_argument("--no-peaks", action="store_true", help="skip the measured copy / MFMA peaks")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path is single-GPU; no collective is part of it); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    lux = load_package()
    lux.init(0)
    for opt in args.option:
        name, _, val = opt.partition("=")
        lux.set_option(name, int(val))
    def peaks():
        cp, mb, mf = C.c_double(), C.c_double(), C.c_double()
        lux._lib.call("luxhip_measure_peaks", lux.current_stream(), C.byref(cp), C.byref(mb), C.byref(mf))
        return {"copy_GBps": round(cp.value, 1), "mfma_bf16_TFLOPs": round(mb.value, 1), "mfma_f32_TFLOPs": round(mf.value, 1)}

    peaks_before = None if args.no_peaks else peaks()
    names = DEFAULT_ORDER if args.workload == "ALL" else [args.workload]
    entries = [measure(lux, n, args) for n in names]
    head = entries[0]

    out = {
        "metric": METRIC, "value": head["value"], "unit": head["unit"], "n_gpus": 1, "steps": head["steps"], "warmup": head["warmup"],
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": head["dtype"],
        "data": "synthetic", "config": {"workload": f"{head['workload']}: {head['description']}"},
        "options": args.option + ([f"rotate={args.rotate}"] if args.rotate > 1 else []), "frac_of_peak": head["frac_of_peak"],
        "ms_per_step_gpu_events": head["ms_per_step_gpu_events"], "ms_per_step_host_clock": head["ms_per_step_host_clock"],
        "timing": head["timing"], "spread": head["spread"],
        "roofline": head["roofline"], "kernels": head["kernels"],
    }
    for k in ("cold_inputs", "warm_inputs", "inputs", "graph_replay", "fused_variant", "cpu_baseline"):
        if k in head:
            out[k] = head[k]
    out["configs"] = entries
    if not args.no_peaks:
        after = peaks()
        out["measured_peaks"] = dict(after, before_the_workloads=peaks_before, after_the_workloads=after,
                                     published={"hbm_GBps": PEAK_HBM_GBS, "mfma_bf16_TFLOPs": PEAK_MFMA_TFLOPS["bf16"],
                                                "mfma_f32_TFLOPs": PEAK_MFMA_TFLOPS["f32"]},
                                     note="streaming copy of 512 MiB (read + written bytes); register-only MFMA loops on pseudo-random "
                                          "operands, 8 waves per compute unit, after the clocks have settled; measured once before and "
                                          "once after the workloads (the top-level figures are the later ones)")
    if args.calibrate_copy:
        nbytes = 256 << 20
        a, b = lux.DeviceArray((nbytes // 4,), "f32"), lux.DeviceArray((nbytes // 4,), "f32")
        for _ in range(3):
            lux._lib.call("luxhip_memcpy_d2d", C.c_void_p(b.ptr), C.c_void_p(a.ptr), C.c_size_t(nbytes), lux.current_stream())
        lux.synchronize()
        out["calibration_copy_bytes"] = nbytes
    print(json.dumps(out))


if __name__ == "__main__":
    main()
