"""layernorm forward + pullback on the GPU against the oracle
(mirrors lib/LuxLib/test/normalization/layernorm_tests.jl:22-113 of the reference)."""
import numpy as np
import pytest

from oracle import luxlib_oracle as O
from tests.util import stable_seed, assert_close, dev, f64, host_inputs, rms

pytestmark = pytest.mark.gpu

# (shape, number of leading normalised dims)
CASES = [((4, 4, 6, 2), 3), ((6, 3), 1), ((16, 5), 1), ((3, 4, 5), 1), ((3, 4, 5), 2), ((512, 9), 1), ((1000, 7), 1),
         ((4096, 6), 1), ((20000, 3), 1), ((24, 24, 8, 5), 3),
         # 64 columns or more of at most 512 vectors: the pullback that reads delta and x once (an odd
         # number of columns, more columns than wavefront pairs in the grid, a ragged last round)
         ((256, 67), 1), ((4096, 70), 1), ((520, 1601), 1), ((24, 8, 200), 2)]


def test_invariants_without_affine(gpu):
    # layernorm_tests.jl:54-57: mean(y) ~ 0, std(y) ~ 1
    x = O.generate_fixed_array(np.float32, (4, 4, 6, 2))
    y = gpu.layernorm(gpu.DeviceArray.from_numpy(x), None, None, "identity", (1, 2, 3)).to_numpy()
    assert abs(y.mean(axis=(0, 1, 2))).max() < 1e-5
    np.testing.assert_allclose(y.std(axis=(0, 1, 2)), 1, atol=1e-3)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("act", ["identity", "relu", "gelu", "tanh"])
@pytest.mark.parametrize("affine", [True, False])
def test_forward_and_pullback(gpu, dtype, act, affine):
    rng = np.random.default_rng(stable_seed(dtype, act, affine))
    for shape, nd in CASES:
        pshape = shape[:nd] + (1,) * (len(shape) - nd)
        eps = 1e-5 if dtype == "f32" else 1e-3
        dims_np, dims_jl = tuple(range(nd)), tuple(range(1, nd + 1))
        for _ in range(50):
            x, g, b, delta = host_inputs(dtype, rng.normal(size=shape), rng.uniform(0.5, 1.5, pshape) if affine else None,
                                         rng.normal(size=pshape) if affine else None, rng.normal(size=shape))
            # keep the pre-activation away from relu's kink (a sign flip is a discontinuity)
            if act != "relu" or shape[0] > 4000 or np.abs(O.layernorm(f64(x), f64(g), f64(b), "identity", dims_np, eps)).min() > 1e-4:
                break
        tag = f"{dtype} {act} {shape} nd={nd} affine={affine}"
        y, back = gpu.pullback(gpu.layernorm, dev(gpu, x, dtype), dev(gpu, g, dtype), dev(gpu, b, dtype), act, dims_jl, eps)
        wy = O.layernorm(f64(x), f64(g), f64(b), act, dims_np, eps)
        assert_close(y.to_numpy(), wy, dtype, tag + " y", want32=O.layernorm(x, g, b, act, dims_np, np.float32(eps)))
        gx, gg, gb = back(dev(gpu, delta, dtype))
        wdx, wdg, wdb = O.layernorm_pullback(f64(x), f64(g), f64(b), act, dims_np, eps, f64(delta))
        w32 = O.layernorm_pullback(x, g, b, act, dims_np, np.float32(eps), delta)
        rel = None
        var = f64(x).var(axis=dims_np)
        scale = rms(delta) * (1.5 if affine else 1.0) / float(np.sqrt(var.min() + eps))
        assert_close(gx.to_numpy(), wdx, dtype, tag + " dx", rel=rel, scale=scale, want32=w32[0])
        if affine:
            assert gg.shape == pshape and gb.shape == pshape
            assert_close(gg.to_numpy(), wdg, dtype, tag + " dgamma", rel=rel, scale=rms(delta), want32=w32[1])
            assert_close(gb.to_numpy(), wdb, dtype, tag + " dbeta", rel=rel, scale=rms(delta), want32=w32[2])
        else:
            assert gg is None and gb is None


def test_default_dims_and_errors(gpu):
    rng = np.random.default_rng(2)
    x = rng.normal(size=(6, 5, 4)).astype(np.float32)
    g = rng.normal(size=(6, 5, 1)).astype(np.float32)
    b = rng.normal(size=(6, 5, 1)).astype(np.float32)
    d = gpu.DeviceArray.from_numpy
    y = gpu.layernorm(d(x), d(g), d(b))                      # dims default 1:(N-1)
    assert_close(y.to_numpy(), O.layernorm(f64(x), f64(g), f64(b), "identity", (0, 1), O.default_epsilon(np.float32)),
                 "f32", "default dims")
    with pytest.raises(gpu.ArgumentError):                   # layernorm_tests.jl:100-113
        gpu.layernorm(d(x), None, None, "identity", None)
    with pytest.raises(gpu.Unsupported):                     # non-leading dims: generic host path
        gpu.layernorm(d(x), None, None, "identity", (2,))


def test_config4_layernorm_full_size(gpu):
    """benchmark configuration 4's layernorm: 4096 features x 8192 tokens, bf16, affine.  Oracle on a
    token subset; invariants on all tokens (normalised rows have zero mean / unit variance;
    dx rows sum to zero and are orthogonal to xhat)."""
    rng = np.random.default_rng(1003)
    L, R = 4096, 8192
    x = rng.standard_normal(size=(L, R), dtype=np.float32)
    g = rng.uniform(0.5, 1.5, (L, 1)).astype(np.float32)
    b = (0.1 * rng.standard_normal((L, 1))).astype(np.float32)
    delta = (0.02 * rng.standard_normal(size=(L, R), dtype=np.float32))
    x, g, b, delta = host_inputs("bf16", x, g, b, delta)
    eps = 1e-5
    y, back = gpu.pullback(gpu.layernorm, dev(gpu, x, "bf16"), dev(gpu, g, "bf16"), dev(gpu, b, "bf16"), "identity", (1,), eps)
    gx, gg, gb = back(dev(gpu, delta, "bf16"))
    yh, gxh = y.to_numpy(), gx.to_numpy().astype(np.float64)
    sub = slice(0, R, 257)
    assert_close(yh[:, sub], O.layernorm(f64(x[:, sub]), f64(g), f64(b), "identity", (0,), eps), "bf16", "config4 LN y")
    wdx, _, _ = O.layernorm_pullback(f64(x[:, sub]), f64(g), f64(b), "identity", (0,), eps, f64(delta[:, sub]))
    assert_close(gxh[:, sub], wdx, "bf16", "config4 LN dx")
    xh = (yh.astype(np.float64) - f64(b)) / f64(g)
    assert np.abs(xh.mean(axis=0)).max() < 1e-2
    assert np.abs(xh.var(axis=0) - 1).max() < 1e-2
    assert np.abs(gxh.sum(axis=0)).max() < 0.5            # 4096 bf16-rounded terms of size ~0.02
    _, wdg, wdb = O.layernorm_pullback(f64(x), f64(g), f64(b), "identity", (0,), eps, f64(delta))
    assert_close(gg.to_numpy(), wdg, "bf16", "config4 LN dgamma", scale=rms(delta) * 90)
    assert_close(gb.to_numpy(), wdb, "bf16", "config4 LN dbeta", scale=rms(delta) * 90)


REFERENCE_CONFIGS = [(xs, aff, act) for xs in ((3, 3, 2, 1), (2, 2, 2, 1)) for aff in (None, "channel")
                     for act in ("identity", "sigmoid_fast", "tanh")]


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("xs,aff,act", REFERENCE_CONFIGS)
def test_reference_test_configurations(gpu, dtype, xs, aff, act):
    """The configurations of lib/LuxLib/test/normalization/layernorm_tests.jl:80-86 on its own input
    generator: dims = Colon() with parameters (1, 1, C, 1), and dims = nothing with parameters
    (1, 1, C) (statistics over 1:(N - 3), :22-32).  (Its cube activation is not in the table; tanh
    stands in.)"""
    eps = gpu.default_epsilon(dtype)
    x = O.generate_fixed_array(np.float32, xs)
    cases = [(gpu.COLON, (1, 1, xs[2], 1), tuple(range(len(xs))))]
    if aff is not None:
        cases.append((None, (1, 1, xs[2]), (0,)))
    for dims, pshape, axes in cases:
        if aff is None:
            g = b = gfull = bfull = None
        else:
            g, b = O.generate_fixed_array(np.float32, pshape), O.generate_fixed_array(np.float32, pshape)
            gfull, bfull = g.reshape(pshape + (1,) * (len(xs) - len(pshape))), b.reshape(pshape + (1,) * (len(xs) - len(pshape)))
        xq, gq, bq = host_inputs(dtype, x, g, b)
        gfq = None if gq is None else gq.reshape(gfull.shape)
        bfq = None if bq is None else bq.reshape(bfull.shape)
        delta = host_inputs(dtype, np.random.default_rng(5).normal(size=xs))[0]
        y, back = gpu.pullback(gpu.layernorm, dev(gpu, xq, dtype), dev(gpu, gq, dtype), dev(gpu, bq, dtype), act, dims, eps)
        tag = f"{dtype} {xs} {pshape if aff else None} {act} dims={dims}"
        want = O.layernorm(f64(xq), f64(gfq), f64(bfq), act, axes, eps)
        assert y.shape == tuple(xs)
        assert_close(y.to_numpy(), want, dtype, tag + " y", rel=None)
        if aff is None and act == "identity":        # :56-59
            np.testing.assert_allclose(y.to_numpy().mean(axis=axes), 0, atol=1e-3 if dtype == "f32" else 1e-2)
        gx, gg, gb = back(dev(gpu, delta, dtype))
        wdx, wdg, wdb = O.layernorm_pullback(f64(xq), f64(gfq), f64(bfq), act, axes, eps, f64(delta))
        w32 = O.layernorm_pullback(xq, gfq, bfq, act, axes, np.float32(eps), delta)
        rel = None
        assert_close(gx.to_numpy(), wdx, dtype, tag + " dx", rel=rel, scale=rms(delta), want32=w32[0])
        if aff is not None:
            assert gg.shape == tuple(pshape) and gb.shape == tuple(pshape)
            assert_close(gg.to_numpy().reshape(gfull.shape), wdg, dtype, tag + " dgamma", rel=rel, scale=rms(delta), want32=w32[1])
            assert_close(gb.to_numpy().reshape(bfull.shape), wdb, dtype, tag + " dbeta", rel=rel, scale=rms(delta), want32=w32[2])
        else:
            assert gg is None and gb is None


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_channel_parameters_on_larger_shapes(gpu, dtype):
    """Statistics over a prefix of the dims with parameters that vary along one other run of dims."""
    rng = np.random.default_rng(8)
    eps = 1e-5 if dtype == "f32" else 1e-3
    for xs, dims, pshape, axes in [((16, 12, 24, 5), gpu.COLON, (1, 1, 24, 1), (0, 1, 2, 3)),
                                   ((16, 12, 24, 5), (1, 2, 3), (1, 1, 24, 1), (0, 1, 2)),
                                   ((16, 12, 24, 5), (1, 2), (1, 1, 24, 1), (0, 1)),
                                   ((64, 8, 6), (1,), (1, 8, 6), (0,)),
                                   ((32, 10, 7), None, (32, 10), (0,)),
                                   ((8, 4, 6, 3), (1, 2), (1, 1, 1, 1), (0, 1)),
                                   # test/core_layers/normalize_tests.jl:279-283: LayerNorm((3, 3, 3)), ((1, 3, 1)), ((3, 1, 3)) on
                                   # x 3x3x3x2 with the layer's dims = Colon()
                                   ((3, 3, 3, 2), gpu.COLON, (3, 3, 3, 1), (0, 1, 2, 3)),
                                   ((3, 3, 3, 2), gpu.COLON, (1, 3, 1, 1), (0, 1, 2, 3)),
                                   ((3, 3, 3, 2), gpu.COLON, (3, 1, 3, 1), (0, 1, 2, 3)),
                                   ((16, 5, 12, 4), (1, 2, 3), (16, 1, 12, 1), (0, 1, 2)),
                                   ((6, 4, 5, 3, 2), (1, 2), (6, 1, 5, 1, 2), (0, 1))]:
        full = pshape + (1,) * (len(xs) - len(pshape))
        x, g, b, delta = host_inputs(dtype, rng.normal(size=xs) * 2 + 0.5, rng.uniform(0.5, 1.5, size=pshape), rng.normal(size=pshape),
                                     rng.normal(size=xs))
        for act in ("identity", "gelu"):
            y, back = gpu.pullback(gpu.layernorm, dev(gpu, x, dtype), dev(gpu, g, dtype), dev(gpu, b, dtype), act, dims, eps)
            tag = f"{dtype} {xs} dims={dims} params={pshape} {act}"
            assert_close(y.to_numpy(), O.layernorm(f64(x), f64(g).reshape(full), f64(b).reshape(full), act, axes, eps), dtype, tag + " y",
                         rel=None)
            gx, gg, gb = back(dev(gpu, delta, dtype))
            wdx, wdg, wdb = O.layernorm_pullback(f64(x), f64(g).reshape(full), f64(b).reshape(full), act, axes, eps, f64(delta))
            w32 = O.layernorm_pullback(x, g.reshape(full), b.reshape(full), act, axes, np.float32(eps), delta)
            rel = None
            assert_close(gx.to_numpy(), wdx, dtype, tag + " dx", rel=rel, scale=rms(delta) * 1.5, want32=w32[0])
            assert_close(gg.to_numpy().reshape(full), wdg, dtype, tag + " dgamma", rel=rel, scale=rms(delta) * np.sqrt(x.size / g.size), want32=w32[1])
            assert_close(gb.to_numpy().reshape(full), wdb, dtype, tag + " dbeta", rel=rel, scale=rms(delta) * np.sqrt(x.size / g.size), want32=w32[2])


def test_dims_nothing_assertion(gpu):
    d = gpu.DeviceArray.from_numpy
    x = np.random.default_rng(1).random((2, 3)).astype(np.float32)
    sc = np.random.default_rng(2).random((2, 1)).astype(np.float32)
    with pytest.raises(AssertionError):                      # layernorm_tests.jl:108-111
        gpu.layernorm(d(x), d(sc), d(sc), "identity", None, 1e-5)
