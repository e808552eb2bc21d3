"""dropout / alpha_dropout on the GPU against the oracle (mirrors
lib/LuxLib/test/common_ops/dropout_tests.jl): the noise stream bit for bit, masks and products
exactly, every training / mask / update_mask combination."""
import numpy as np
import pytest

from oracle import luxlib_oracle as O
from tests.util import stable_seed, assert_close, dev, f64, host_inputs

pytestmark = pytest.mark.gpu

# the last four are the shapes of lib/LuxLib/test/common_ops/dropout_tests.jl:10
SHAPES = [(7,), (4, 4), (5, 3, 2), (16, 16, 8, 3), (33, 65, 2), (1000, 37), (0, 3), (2, 3), (2, 2, 3), (2, 2, 3, 1), (2, 2, 1, 3, 1)]


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_rand_uniform_bit_exact(gpu, dtype):
    rng = gpu.PhiloxRNG(seed=0x1234_5678_9abc_def0, offset=(1 << 32) - 3)       # crosses the 32-bit counter word
    for shape in SHAPES + [(1 << 20,)]:
        n = int(np.prod(shape))
        out, rng2 = gpu.rand_uniform(rng, shape, dtype)
        assert rng2 == gpu.PhiloxRNG(rng.seed, rng.offset + (n + 3) // 4)
        want = O.rand_uniform(n, rng.seed, rng.offset, bf16=dtype == "bf16").reshape(shape, order="F")
        np.testing.assert_array_equal(out.to_numpy(), want)
        rng = rng2


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("p", [0.0, 0.3, 0.5, 0.9])
def test_dropout(gpu, dtype, p):
    nprng = np.random.default_rng(stable_seed(dtype, p))
    invp = 1.0 / (1.0 - p)
    T = np.float32
    rd = (lambda a: O.round_to_bf16(np.asarray(a, np.float32))) if dtype == "bf16" else (lambda a: np.asarray(a, np.float32))
    rng = gpu.PhiloxRNG(seed=77, offset=5)
    for shape in SHAPES:
        nd = len(shape)
        for dims in [None, (1,), (nd,), tuple(range(1, nd)), (1, nd), (1, 2)][: (6 if nd > 2 else 5) if nd > 1 else 1]:
            if dims is not None and (len(dims) == 0 or len(set(dims)) != len(dims)):
                continue
            x, delta = host_inputs(dtype, nprng.normal(size=shape), nprng.normal(size=shape))
            tag = f"{dtype} p={p} {shape} dims={dims}"
            ms = O.dropout_shape(shape, dims)
            n = int(np.prod(ms))
            (y, mask, rng2), back = gpu.pullback(gpu.dropout, rng, dev(gpu, x, dtype), p, True, invp, dims)
            noise = O.rand_uniform(n, rng.seed, rng.offset, bf16=dtype == "bf16").reshape(ms, order="F")
            wm = (noise > rd(p)).astype(T) * rd(invp)                 # T(p), T(invp) act in the storage type
            assert rng2 == rng.advanced(n)
            np.testing.assert_array_equal(mask.to_numpy(), wm, err_msg=tag)
            np.testing.assert_array_equal(y.to_numpy(), rd(x * wm), err_msg=tag)
            (dx,) = back(dev(gpu, delta, dtype))
            np.testing.assert_array_equal(dx.to_numpy(), rd(delta * wm), err_msg=tag)
            # the stored-noise route gives the same mask
            nz, _ = gpu.rand_uniform(rng, ms, dtype)
            gpu._lib.call("luxhip_dropout_mask", gpu.current_stream(), nz.code, nz.size, float(p), float(invp), nz.ptr)
            np.testing.assert_array_equal(nz.to_numpy(), wm, err_msg=tag)
            # a given mask: used as it is (update_mask false), replaced (update_mask true)
            xm = dev(gpu, x, dtype)
            y3, m3, r3 = gpu.dropout(rng, xm, p, True, invp, dims, mask=mask, update_mask=False)
            assert m3 is mask and r3 == rng
            np.testing.assert_array_equal(y3.to_numpy(), y.to_numpy())
            y4, m4, r4 = gpu.dropout(rng, xm, p, True, invp, dims, mask=mask, update_mask=True)
            assert r4 == rng2
            np.testing.assert_array_equal(m4.to_numpy(), wm)
            # not training: x comes back untouched
            y5, m5, r5 = gpu.dropout(rng, xm, p, False, invp, dims)
            assert y5 is xm and m5 is xm and r5 == rng
            y6, m6, r6 = gpu.dropout(rng, xm, p, False, invp, dims, mask=mask, update_mask=False)
            assert y6 is xm and m6 is mask and r6 == rng
            rng = rng2
    with pytest.raises(AssertionError):
        d = lambda *s: gpu.DeviceArray.from_numpy(np.ones(s, np.float32))
        gpu.dropout(rng, d(4, 3), p, True, invp, None, mask=d(4, 2), update_mask=False)


def test_dropout_keeps_the_expected_fraction(gpu):
    x = gpu.DeviceArray.from_numpy(np.ones((1 << 20,), np.float32))
    for p in (0.1, 0.5, 0.8):
        y, mask, _ = gpu.dropout(gpu.PhiloxRNG(3, 0), x, p, True, 1 / (1 - p))
        kept = (mask.to_numpy() != 0).mean()
        assert abs(kept - (1 - p)) < 5 * np.sqrt(p * (1 - p) / (1 << 20))
        assert abs(y.to_numpy().mean() - 1.0) < 0.01             # dropout_tests.jl: the mean is preserved


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("p", [0.2, 0.5])
def test_alpha_dropout(gpu, dtype, p):
    nprng = np.random.default_rng(stable_seed(dtype, p, "alpha"))
    rng = gpu.PhiloxRNG(seed=11, offset=0)
    for shape in SHAPES:
        x, delta = host_inputs(dtype, nprng.normal(size=shape), nprng.normal(size=shape))
        n = int(np.prod(shape))
        (y, rng2), back = gpu.pullback(gpu.alpha_dropout, rng, dev(gpu, x, dtype), p, True)
        assert rng2 == rng.advanced(n)
        noise = O.rand_uniform(n, rng.seed, rng.offset, bf16=dtype == "bf16").reshape(shape, order="F")
        alpha, A, B = O.alpha_dropout_coefficients(p)
        if dtype == "bf16":
            alpha, A, B = (float(O.round_to_bf16(np.float32(v))) for v in (alpha, A, B))
        assert_close(y.to_numpy(), O.alpha_dropout(f64(noise), p, f64(x), alpha, A, B), dtype, f"alpha {shape} y")
        (dx,) = back(dev(gpu, delta, dtype))
        assert_close(dx.to_numpy(), O.alpha_dropout_pullback(f64(noise), p, f64(delta), A), dtype, f"alpha {shape} dx")
        # explicit coefficients and the inference path
        y2, _ = gpu.alpha_dropout(rng, dev(gpu, x, dtype), p, True, *O.alpha_dropout_coefficients(p))
        np.testing.assert_array_equal(y2.to_numpy(), y.to_numpy())
        xd = dev(gpu, x, dtype)
        y3, r3 = gpu.alpha_dropout(rng, xd, p, False)
        assert y3 is xd and r3 == rng
        rng = rng2
    # standardised input keeps mean 0 / variance 1 (dropout_tests.jl checks the same)
    big = gpu.DeviceArray.from_numpy(nprng.normal(size=(1 << 20,)).astype(np.float32), dtype)
    yb, _ = gpu.alpha_dropout(gpu.PhiloxRNG(5, 0), big, p, True)
    yb = yb.to_numpy()
    assert abs(yb.mean()) < 0.02 and abs(yb.var() - 1) < 0.05
