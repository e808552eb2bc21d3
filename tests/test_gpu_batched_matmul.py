"""batched_matmul forward + pullback on the GPU against the oracle
(mirrors lib/LuxLib/test/common_ops/bmm_tests.jl: shared operands, transposed operands, sizes that
are no multiple of a tile)."""
import numpy as np
import pytest

from oracle import luxlib_oracle as O
from tests.util import stable_seed, assert_close, dev, f64, host_inputs, rms

pytestmark = pytest.mark.gpu

CASES = [
    # x shape, y shape, lhs contracting dim, rhs contracting dim
    ((4, 5, 3), (5, 6, 3), 2, 1), ((4, 5, 1), (5, 6, 3), 2, 1), ((4, 5, 3), (5, 6, 1), 2, 1),
    ((5, 4, 3), (5, 6, 3), 1, 1), ((4, 5, 3), (6, 5, 3), 2, 2), ((5, 4, 2, 3), (6, 5, 2, 3), 1, 2),
    ((4, 5), (5, 6, 3), 2, 1), ((4, 5, 3), (5, 6), 2, 1),
    ((37, 65, 7), (65, 29, 7), 2, 1), ((130, 70, 5), (70, 129, 5), 2, 1), ((70, 130, 5), (129, 70, 1), 1, 2),
    # whole 128 x 128 tiles (the kernels without bounds checks), every operand layout
    ((128, 64, 6), (64, 256, 6), 2, 1), ((64, 128, 6), (64, 256, 6), 1, 1), ((128, 64, 6), (256, 64, 6), 2, 2),
    ((64, 256, 4), (128, 64, 4), 1, 2), ((256, 32, 1), (32, 128, 9), 2, 1),
]


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("case", range(len(CASES)))
def test_forward_and_pullback(gpu, dtype, case):
    xs, ys, lc, rc = CASES[case]
    rng = np.random.default_rng(stable_seed(dtype, case))
    x, y = host_inputs(dtype, rng.normal(size=xs), rng.normal(size=ys))
    z, back = gpu.pullback(gpu.batched_matmul, dev(gpu, x, dtype), dev(gpu, y, dtype), lc, rc)
    wz = O.batched_matmul(f64(x), f64(y), lc, rc)
    K = xs[lc - 1]
    tag = f"{dtype} case {case}"
    assert z.shape == wz.shape
    assert_close(z.to_numpy(), wz, dtype, tag + " z", scale=np.sqrt(K))
    np.testing.assert_array_equal(gpu.batched_matmul(dev(gpu, x, dtype), dev(gpu, y, dtype), lc, rc).to_numpy(), z.to_numpy())
    (delta,) = host_inputs(dtype, rng.normal(size=wz.shape))
    dx, dy = back(dev(gpu, delta, dtype))
    wdx, wdy = O.batched_matmul_pullback(f64(x), f64(y), f64(delta), lc, rc)
    assert dx.shape == tuple(xs) and dy.shape == tuple(ys)
    batch = int(np.prod(wz.shape[2:]))
    shared_x = int(np.prod(xs[2:])) == 1 and batch > 1
    shared_y = int(np.prod(ys[2:])) == 1 and batch > 1
    # a shared operand's gradient is a sum of per-product results that are stored (bf16: rounded) first
    rel = None
    assert_close(dx.to_numpy(), wdx, dtype, tag + " dx", rel=rel, scale=np.sqrt(wz.shape[1] * (batch if shared_x else 1)))
    assert_close(dy.to_numpy(), wdy, dtype, tag + " dy", rel=rel, scale=np.sqrt(wz.shape[0] * (batch if shared_y else 1)))


def test_errors(gpu):
    d = lambda *s: gpu.DeviceArray.from_numpy(np.ones(s, np.float32))
    with pytest.raises(gpu.DimensionMismatch):
        gpu.batched_matmul(d(4, 5, 3), d(5, 6, 2))
    with pytest.raises(gpu.DimensionMismatch):
        gpu.batched_matmul(d(4, 5, 3), d(4, 6, 3))
    with pytest.raises(gpu.ArgumentError):
        gpu.batched_matmul(d(4, 5), d(5, 6))
    z = gpu.batched_matmul(d(4, 0, 3), d(0, 6, 3))                 # an empty contraction gives zeros
    np.testing.assert_array_equal(z.to_numpy(), np.zeros((4, 6, 3), np.float32))
    assert gpu.batched_matmul(d(4, 5, 0), d(5, 6, 0)).shape == (4, 6, 0)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_attention_shaped_products(gpu, dtype):
    """scores = K' Q and values = V P for 64 heads of width 64 over 512 positions (the products of
    scaled_dot_product_attention, impl/attention.jl:70-117): oracle on three heads, the rest
    through linearity (the sum over heads of z equals the product with summed operands only for a
    shared operand, which the shared-operand case covers)."""
    rng = np.random.default_rng(7)
    E, L, H = 64, 512, 64
    k, q = host_inputs(dtype, rng.normal(size=(E, L, H)) / np.sqrt(E), rng.normal(size=(E, L, H)))
    s = gpu.batched_matmul(dev(gpu, k, dtype), dev(gpu, q, dtype), 1, 1)            # (L, L, H)
    sub = [0, 31, 63]
    assert_close(s.to_numpy()[..., sub], O.batched_matmul(f64(k[..., sub]), f64(q[..., sub]), 1, 1), dtype, "scores",
                 scale=1.0)
    shared = gpu.batched_matmul(dev(gpu, k[..., :1], dtype), dev(gpu, q, dtype), 1, 1).to_numpy()
    assert_close(shared[..., sub], O.batched_matmul(f64(k[..., :1]), f64(q[..., sub]), 1, 1), dtype, "shared scores", scale=1.0)


GENERAL = [
    # x shape, y shape, lhs contracting, rhs contracting, lhs batching dims, rhs batching dims
    ((3, 4, 5, 2), (5, 4, 5, 1), 2, 2, None, None),            # generalized_bmm_tests.jl:8-22: a partly repeated operand
    ((3, 5, 2, 4), (4, 5, 1, 5), 4, 1, (2, 3), (4, 3)),        # generalized_bmm_tests.jl:36-58: batch dims in the middle
    ((6, 3, 4, 7), (6, 3, 5, 7), 1, 1, (2, 4), (2, 4)),        # contraction along the first dim of both
    ((4, 2, 3, 5, 6), (1, 6, 3, 7, 5), 5, 2, (2, 3, 4), (1, 3, 5)),
    ((33, 2, 3, 70), (70, 3, 1, 40), 4, 1, (2, 3), (3, 2)),
    ((5, 4, 1, 1), (4, 6, 3, 2), 2, 1, None, None),
    ((5, 2, 3, 4, 1), (4, 2, 3, 6, 2), 4, 1, (2, 3, 5), (2, 3, 5)),
]


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("case", range(len(GENERAL)))
def test_general_batching_dims(gpu, dtype, case):
    xs, ys, cx, cy, bx, by = GENERAL[case]
    rng = np.random.default_rng(stable_seed("bmm-general", case))
    x, y = host_inputs(dtype, rng.normal(size=xs), rng.normal(size=ys))
    want = O.batched_matmul_general(f64(x), f64(y), cx, cy, bx, by)
    (delta,) = host_inputs(dtype, rng.normal(size=want.shape))
    z, back = gpu.pullback(gpu.batched_matmul, dev(gpu, x, dtype), dev(gpu, y, dtype), cx, cy, bx, by)
    assert z.shape == want.shape
    assert_close(z.to_numpy(), want, dtype, f"case {case} z")
    dx, dy = back(dev(gpu, delta, dtype))
    wdx, wdy = O.batched_matmul_general_pullback(f64(x), f64(y), f64(delta), cx, cy, bx, by)
    assert dx.shape == tuple(xs) and dy.shape == tuple(ys)
    rel = None
    assert_close(dx.to_numpy(), wdx, dtype, f"case {case} dx", rel=rel)
    assert_close(dy.to_numpy(), wdy, dtype, f"case {case} dy", rel=rel)


def test_operand_without_a_contiguous_matrix_dim_is_refused(gpu):
    d = lambda *shape: gpu.DeviceArray.from_numpy(np.ones(shape, np.float32))
    with pytest.raises(gpu.Unsupported):          # y: contracting dim 3 (stride 6), free dim 4 (stride 36)
        gpu.batched_matmul(d(4, 2, 3, 5, 6), d(2, 3, 6, 7, 5), 5, 3, (2, 3, 4), (1, 2, 5))
