"""Pins the oracle's operators against the reference's own known-answer tests, independent
library routines (torch CPU + autograd), closed forms and fp64 finite differences."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import luxlib_oracle as O

RNG = np.random.default_rng(20240)


def fd_grad(f, x, h=1e-6):
    """Central finite differences of scalar f at x (fp64), as LuxTestUtils.test_gradients does
    (lib/LuxTestUtils/src/autodiff.jl:147-294)."""
    g = np.zeros_like(x)
    it = np.nditer(x, flags=["multi_index"])
    for _ in it:
        i = it.multi_index
        xp, xm = x.copy(), x.copy()
        xp[i] += h
        xm[i] -= h
        g[i] = (f(xp) - f(xm)) / (2 * h)
    return g


# ----------------------------------------------------------------------------- bias_activation
@pytest.mark.parametrize("act", ["identity", "relu", "sigmoid", "softplus", "logsigmoid", "gelu",
                                 "swish", "lisht", "tanh"])
@pytest.mark.parametrize("shape", [(2, 2, 3, 4), (4, 5)])
def test_bias_activation_closed_form_and_grad(act, shape):
    # lib/LuxLib/test/common_ops/bias_act_tests.jl:6,16-99
    x = RNG.random(shape)
    b = RNG.random(shape[-2])
    bshape = [1] * len(shape)
    bshape[-2] = shape[-2]
    want = O.act_value(act, x + b.reshape(bshape))
    np.testing.assert_allclose(O.bias_activation(act, x, b), want, rtol=0, atol=0)
    delta = RNG.normal(size=shape)
    y, dx, db = O.bias_activation_pullback(act, x, b, delta)
    np.testing.assert_allclose(dx, fd_grad(lambda v: (O.bias_activation(act, v, b) * delta).sum(), x),
                               rtol=1e-6, atol=1e-8)
    np.testing.assert_allclose(db, fd_grad(lambda v: (O.bias_activation(act, x, v) * delta).sum(), b),
                               rtol=1e-6, atol=1e-8)


def test_bias_activation_edge_cases():
    # zero-sized arrays (bias_act_tests.jl:119-131), vectors, missing bias, wrong bias length
    x = np.zeros((4, 3, 2, 0))
    assert O.bias_activation("relu", x, np.ones(2)).shape == (4, 3, 2, 0)
    v = np.array([1.0, -2.0, 3.0])
    np.testing.assert_array_equal(O.bias_activation("relu", v, np.array([0.5, 0.5, 0.5])), [1.5, 0, 3.5])
    np.testing.assert_array_equal(O.bias_activation("relu", v, None), [1, 0, 3])
    with pytest.raises(AssertionError):
        O.bias_activation("relu", np.ones((3, 4)), np.ones(4))


# ----------------------------------------------------------------------------- dense
def test_dense_reference_known_answers():
    # test/core_layers/basic_tests.jl:151-194: Dense(10 => 1/2) with ones -> 10, [10 20; 10 20]
    y = O.fused_dense_bias_activation("identity", np.ones((1, 10)), np.ones((10, 1)), None)
    assert y.tolist() == [[10.0]]
    y = O.fused_dense_bias_activation("identity", np.ones((2, 10)), np.ones((10, 1)), np.ones(2))
    assert y.tolist() == [[11.0], [11.0]]
    y = O.fused_dense_bias_activation("identity", np.ones((2, 10)), np.array([np.ones(10), 2 * np.ones(10)]).T, None)
    assert y.tolist() == [[10.0, 20.0], [10.0, 20.0]]
    y = O.fused_dense_bias_activation("relu", -np.ones((1, 10)), np.ones((10, 1)), None)
    assert y.tolist() == [[0.0]]


@pytest.mark.parametrize("act", ["identity", "tanh", "sigmoid_fast", "relu", "gelu", "swish"])
@pytest.mark.parametrize("M,N,bias", [(4, 32, True), (32, 4, False)])
def test_dense_vs_torch_autograd(act, M, N, bias):
    # lib/LuxLib/test/common_ops/dense_tests.jl:13-76: sizes 4/32, batch 3, bias on/off
    W = RNG.normal(size=(M, N))
    x = RNG.normal(size=(N, 3))
    b = RNG.normal(size=M) if bias else None
    delta = RNG.normal(size=(M, 3))
    y, dW, dx, db = O.fused_dense_pullback(act, W, x, b, delta)
    from tests.test_oracle_activations import TORCH
    tW, tx = torch.tensor(W, requires_grad=True), torch.tensor(x, requires_grad=True)
    tb = torch.tensor(b, requires_grad=True) if bias else None
    ty = TORCH[act](F.linear(tx.T, tW, tb)).T          # torch: rows = batch
    ty.backward(torch.tensor(delta))
    np.testing.assert_allclose(y, ty.detach().numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dW, tW.grad.numpy(), rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(dx, tx.grad.numpy(), rtol=1e-10, atol=1e-12)
    if bias:
        np.testing.assert_allclose(db, tb.grad.numpy(), rtol=1e-10, atol=1e-12)
    else:
        assert db is None


def test_dense_dimension_mismatch():
    # impl/matmul.jl:21-34
    with pytest.raises(O.DimensionMismatch):
        O.fused_dense_bias_activation("relu", np.ones((3, 4)), np.ones((5, 2)), None)
    with pytest.raises(O.DimensionMismatch):
        O.fused_dense_bias_activation("relu", np.ones((3, 4)), np.ones((4, 2)), np.ones(4))


# ----------------------------------------------------------------------------- batchnorm
def test_batchnorm_reference_known_answer():
    # test/core_layers/normalize_tests.jl:10-49: x = [1 3 5; 2 4 6] (2 channels x 3 samples)
    x = np.array([[1.0, 3.0, 5.0], [2.0, 4.0, 6.0]], dtype=np.float32)
    y, rm, rv = O.batchnorm(x, np.ones(2, np.float32), np.zeros(2, np.float32),
                            np.zeros(2, np.float32), np.ones(2, np.float32), True, "identity",
                            0.1, 1e-5)
    np.testing.assert_allclose(y, [[-1.22474, 0, 1.22474], [-1.22474, 0, 1.22474]], atol=1e-5)
    np.testing.assert_allclose(rm, [0.3, 0.4], rtol=1e-6)
    # 0.1 * var(corrected) + 0.9 = 0.1 * (8/3 * 3/2) + 0.9 = 1.3
    np.testing.assert_allclose(rv, [1.3, 1.3], rtol=1e-6)
    yi, rm2, rv2 = O.batchnorm(x, np.ones(2, np.float32), np.zeros(2, np.float32), rm, rv, False,
                               "identity", 0.1, 1e-5)
    np.testing.assert_allclose(yi[0, 0], (1 - 0.3) / np.sqrt(1.3 + 1e-5), rtol=1e-6)
    assert rm2 is rm and rv2 is rv


@pytest.mark.parametrize("shape", [(4, 4, 6, 2), (8, 2), (3, 5, 4)])
@pytest.mark.parametrize("act", ["identity", "sigmoid_fast", "relu", "swish"])
@pytest.mark.parametrize("affine", [True, False])
def test_batchnorm_vs_torch(shape, act, affine):
    # lib/LuxLib/test/normalization/batchnorm_tests.jl:58-145 shapes; inputs from generate_fixed_array
    from tests.test_oracle_activations import TORCH
    x = O.generate_fixed_array(np.float64, shape) + 0.1 * RNG.normal(size=shape)
    C = shape[-2]
    g = RNG.uniform(0.5, 1.5, C) if affine else None
    b = RNG.normal(size=C) if affine else None
    rm, rv = RNG.normal(size=C), RNG.uniform(0.5, 2, C)
    delta = RNG.normal(size=shape)
    eps = 1e-5
    y, rm_n, rv_n = O.batchnorm(x, g, b, rm, rv, True, act, 0.1, eps)
    dx, dg, db = O.batchnorm_pullback(x, g, b, act, eps, delta)
    perm = (len(shape) - 1, len(shape) - 2) + tuple(range(len(shape) - 2))   # -> N, C, spatial...
    inv = np.argsort(perm)
    tx = torch.tensor(np.transpose(x, perm).copy(), requires_grad=True)
    tg = torch.tensor(g, requires_grad=True) if affine else None
    tb = torch.tensor(b, requires_grad=True) if affine else None
    trm, trv = torch.tensor(rm), torch.tensor(rv)
    ty = TORCH[act](F.batch_norm(tx, trm, trv, tg, tb, True, 0.1, eps))
    ty.backward(torch.tensor(np.transpose(delta, perm).copy()))
    np.testing.assert_allclose(y, np.transpose(ty.detach().numpy(), inv), rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(rm_n, trm.numpy(), rtol=1e-12)
    np.testing.assert_allclose(rv_n, trv.numpy(), rtol=1e-12)
    np.testing.assert_allclose(dx, np.transpose(tx.grad.numpy(), inv), rtol=1e-8, atol=1e-10)
    if affine:
        np.testing.assert_allclose(dg, tg.grad.numpy(), rtol=1e-9, atol=1e-11)
        np.testing.assert_allclose(db, tb.grad.numpy(), rtol=1e-9, atol=1e-11)
    # inference mode
    yi, _, _ = O.batchnorm(x, g, b, rm, rv, False, act, 0.1, eps)
    tyi = TORCH[act](F.batch_norm(tx.detach(), torch.tensor(rm), torch.tensor(rv), None if not affine else tg.detach(),
                                  None if not affine else tb.detach(), False, 0.1, eps))
    np.testing.assert_allclose(yi, np.transpose(tyi.numpy(), inv), rtol=1e-10, atol=1e-11)


def test_batchnorm_pullback_finite_differences():
    shape = (3, 2, 4, 3)
    x = RNG.normal(size=shape)
    g, b = RNG.uniform(0.5, 1.5, 4), RNG.normal(size=4)
    delta = RNG.normal(size=shape)
    dx, dg, db = O.batchnorm_pullback(x, g, b, "gelu", 1e-5, delta)
    loss = lambda xx, gg, bb: (O.batchnorm(xx, gg, bb, None, None, True, "gelu", 0.1, 1e-5)[0] * delta).sum()
    np.testing.assert_allclose(dx, fd_grad(lambda v: loss(v, g, b), x), rtol=2e-6, atol=1e-8)
    np.testing.assert_allclose(dg, fd_grad(lambda v: loss(x, v, b), g), rtol=2e-6, atol=1e-8)
    np.testing.assert_allclose(db, fd_grad(lambda v: loss(x, g, v), b), rtol=2e-6, atol=1e-8)
    # inference-mode pullback: statistics are constants
    rm, rv = RNG.normal(size=4), RNG.uniform(0.5, 2, 4)
    dxi, _, _ = O.batchnorm_pullback(x, g, b, "gelu", 1e-5, delta, training=False, rmean=rm, rvar=rv)
    lossi = lambda xx: (O.batchnorm(xx, g, b, rm, rv, False, "gelu", 0.1, 1e-5)[0] * delta).sum()
    np.testing.assert_allclose(dxi, fd_grad(lossi, x), rtol=2e-6, atol=1e-8)


# ----------------------------------------------------------------------------- groupnorm
@pytest.mark.parametrize("shape,groups", [((6, 2), 2), ((4, 4, 6, 2), 3), ((2, 2, 6, 2), 2), ((5, 12, 3), 4)])
@pytest.mark.parametrize("act", ["identity", "swish", "relu"])
@pytest.mark.parametrize("affine", [True, False])
def test_groupnorm_vs_torch(shape, groups, act, affine):
    # lib/LuxLib/test/normalization/groupnorm_tests.jl:48-115 shapes and groups
    from tests.test_oracle_activations import TORCH
    x = RNG.normal(size=shape)
    C = shape[-2]
    g = RNG.uniform(0.8, 1.2, C) if affine else None
    b = RNG.normal(size=C) if affine else None
    delta = RNG.normal(size=shape)
    eps = 1e-5
    y = O.groupnorm(x, g, b, groups, act, eps)
    dx, dg, db = O.groupnorm_pullback(x, g, b, groups, act, eps, delta)
    perm = (len(shape) - 1, len(shape) - 2) + tuple(range(len(shape) - 2))
    inv = np.argsort(perm)
    tx = torch.tensor(np.transpose(x, perm).copy(), requires_grad=True)
    tg = torch.tensor(g, requires_grad=True) if affine else None
    tb = torch.tensor(b, requires_grad=True) if affine else None
    ty = TORCH[act](F.group_norm(tx, groups, tg, tb, eps))
    ty.backward(torch.tensor(np.transpose(delta, perm).copy()))
    np.testing.assert_allclose(y, np.transpose(ty.detach().numpy(), inv), rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(dx, np.transpose(tx.grad.numpy(), inv), rtol=1e-8, atol=1e-10)
    if affine:
        np.testing.assert_allclose(dg, tg.grad.numpy(), rtol=1e-9, atol=1e-11)
        np.testing.assert_allclose(db, tb.grad.numpy(), rtol=1e-9, atol=1e-11)


def test_groupnorm_argument_errors():
    # api/groupnorm.jl:40-64
    with pytest.raises(O.ArgumentError):
        O.groupnorm(np.ones((4, 6, 2)), np.ones(6), np.ones(6), 4)
    with pytest.raises(O.ArgumentError):
        O.groupnorm(np.ones((4, 6, 2)), np.ones(5), np.ones(5), 2)


def test_groupnorm_equals_instance_stats_when_groups_eq_channels():
    # G == C  =>  per-(channel, sample) statistics (instancenorm, impl/normalization.jl:191-208)
    x = RNG.normal(size=(5, 4, 3))
    y = O.groupnorm(x, None, None, 4, "identity", 0.0)
    np.testing.assert_allclose(y.mean(axis=0), 0, atol=1e-14)
    np.testing.assert_allclose(y.std(axis=0), 1, rtol=1e-12)


# ----------------------------------------------------------------------------- instancenorm
@pytest.mark.parametrize("shape", [(4, 4, 6, 2), (7, 3, 4), (3, 2, 2, 5, 3)])
@pytest.mark.parametrize("act", ["identity", "relu", "swish"])
@pytest.mark.parametrize("affine", [True, False])
def test_instancenorm_vs_torch(shape, act, affine):
    # shapes of lib/LuxLib/test/normalization/instancenorm_tests.jl; torch.nn.functional.instance_norm
    # is the library routine (values, running statistics averaged over the batch, autograd)
    from tests.test_oracle_activations import TORCH
    x = RNG.normal(size=shape) * 1.5 + 0.3
    C = shape[-2]
    g = RNG.uniform(0.5, 1.5, C) if affine else None
    b = RNG.normal(size=C) if affine else None
    rm, rv = RNG.normal(size=C), RNG.uniform(0.5, 2, C)
    delta = RNG.normal(size=shape)
    eps = 1e-5
    perm = (len(shape) - 1, len(shape) - 2) + tuple(range(len(shape) - 2))
    inv = np.argsort(perm)
    tx = torch.tensor(np.transpose(x, perm).copy(), requires_grad=True)
    tg = torch.tensor(g, requires_grad=True) if affine else None
    tb = torch.tensor(b, requires_grad=True) if affine else None
    trm, trv = torch.tensor(rm), torch.tensor(rv)
    ty = TORCH[act](F.instance_norm(tx, trm, trv, tg, tb, True, 0.1, eps))
    ty.backward(torch.tensor(np.transpose(delta, perm).copy()))
    y, rm_n, rv_n = O.instancenorm(x, g, b, rm, rv, True, act, 0.1, eps)
    dx, dg, db = O.instancenorm_pullback(x, g, b, act, eps, delta)
    np.testing.assert_allclose(y, np.transpose(ty.detach().numpy(), inv), rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(rm_n, trm.numpy(), rtol=1e-12)
    np.testing.assert_allclose(rv_n, trv.numpy(), rtol=1e-12)
    np.testing.assert_allclose(dx, np.transpose(tx.grad.numpy(), inv), rtol=1e-8, atol=1e-10)
    if affine:
        np.testing.assert_allclose(dg, tg.grad.numpy(), rtol=1e-9, atol=1e-11)
        np.testing.assert_allclose(db, tb.grad.numpy(), rtol=1e-9, atol=1e-11)
    # the same statistics as groupnorm with one channel per group
    np.testing.assert_allclose(y, O.groupnorm(x, g, b, C, act, eps), rtol=1e-12, atol=1e-13)
    gdx, gdg, gdb = O.groupnorm_pullback(x, g, b, C, act, eps, delta)
    np.testing.assert_allclose(dx, gdx, rtol=1e-10, atol=1e-12)
    # without running statistics nothing is updated; in inference they replace the sample statistics
    y0, r0, v0 = O.instancenorm(x, g, b, None, None, True, act, 0.1, eps)
    assert r0 is None and v0 is None
    np.testing.assert_array_equal(y0, y)
    yi, ri, vi = O.instancenorm(x, g, b, rm, rv, False, act, 0.1, eps)
    assert ri is rm and vi is rv
    tyi = TORCH[act](F.instance_norm(tx.detach(), torch.tensor(rm), torch.tensor(rv), None if not affine else tg.detach(),
                                     None if not affine else tb.detach(), False, 0.1, eps))
    np.testing.assert_allclose(yi, np.transpose(tyi.numpy(), inv), rtol=1e-10, atol=1e-11)


def test_instancenorm_inference_pullback_finite_differences():
    x = RNG.normal(size=(3, 4, 2))
    g, b = RNG.uniform(0.5, 1.5, 4), RNG.normal(size=4)
    rm, rv = RNG.normal(size=4), RNG.uniform(0.5, 2, 4)
    delta = RNG.normal(size=x.shape)
    for training, stats in ((False, (rm, rv)), (False, (None, None)), (True, (rm, rv))):
        loss = lambda xx: float((O.instancenorm(xx, g, b, stats[0], stats[1], training, "swish", 0.1, 1e-5)[0] * delta).sum())
        dx, dg, db = O.instancenorm_pullback(x, g, b, "swish", 1e-5, delta, training=training, rmean=stats[0], rvar=stats[1])
        np.testing.assert_allclose(dx, fd_grad(loss, x), rtol=1e-5, atol=1e-7)
        lg = lambda gg: float((O.instancenorm(x, gg, b, stats[0], stats[1], training, "swish", 0.1, 1e-5)[0] * delta).sum())
        np.testing.assert_allclose(dg, fd_grad(lg, g), rtol=1e-5, atol=1e-7)


def test_instancenorm_needs_three_dims():
    with pytest.raises(AssertionError):
        O.instancenorm(np.ones((4, 3)), None, None, None, None, True)


# ----------------------------------------------------------------------------- layernorm
def test_layernorm_invariants():
    # lib/LuxLib/test/normalization/layernorm_tests.jl:54-57: mean ~ 0, std ~ 1 without affine
    x = O.generate_fixed_array(np.float32, (4, 4, 6, 2))
    y = O.layernorm(x, None, None, "identity", (0, 1, 2), None)
    assert abs(y.mean(axis=(0, 1, 2))).max() < 1e-5
    # epsilon in the denominator biases the std slightly below 1
    np.testing.assert_allclose(y.std(axis=(0, 1, 2)), 1, atol=1e-3)


@pytest.mark.parametrize("shape,nd", [((4, 4, 6, 2), 3), ((6, 3), 1), ((16, 5), 1), ((3, 4, 5), 1)])
@pytest.mark.parametrize("act", ["identity", "relu", "gelu"])
@pytest.mark.parametrize("affine", [True, False])
def test_layernorm_vs_torch(shape, nd, act, affine):
    from tests.test_oracle_activations import TORCH
    x = RNG.normal(size=shape)
    dims = tuple(range(nd))
    pshape = shape[:nd] + (1,) * (len(shape) - nd)
    g = RNG.uniform(0.5, 1.5, pshape) if affine else None
    b = RNG.normal(size=pshape) if affine else None
    delta = RNG.normal(size=shape)
    eps = 1e-5
    y = O.layernorm(x, g, b, act, dims, eps)
    dx, dg, db = O.layernorm_pullback(x, g, b, act, dims, eps, delta)
    # torch normalises trailing dims: reverse the axes
    rev = tuple(reversed(range(len(shape))))
    tx = torch.tensor(np.transpose(x, rev).copy(), requires_grad=True)
    nshape = tuple(reversed(shape[:nd]))
    tg = torch.tensor(np.transpose(g, rev).reshape(nshape).copy(), requires_grad=True) if affine else None
    tb = torch.tensor(np.transpose(b, rev).reshape(nshape).copy(), requires_grad=True) if affine else None
    ty = TORCH[act](F.layer_norm(tx, nshape, tg, tb, eps))
    ty.backward(torch.tensor(np.transpose(delta, rev).copy()))
    np.testing.assert_allclose(y, np.transpose(ty.detach().numpy(), rev), rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(dx, np.transpose(tx.grad.numpy(), rev), rtol=1e-8, atol=1e-10)
    if affine:
        np.testing.assert_allclose(dg, np.transpose(tg.grad.numpy().reshape(tuple(reversed(pshape))), rev), rtol=1e-9, atol=1e-11)
        np.testing.assert_allclose(db, np.transpose(tb.grad.numpy().reshape(tuple(reversed(pshape))), rev), rtol=1e-9, atol=1e-11)


@pytest.mark.parametrize("shape,nd,pshape", [((3, 3, 2, 1), 4, (1, 1, 2, 1)), ((5, 4, 6, 3), 2, (1, 1, 6, 1)), ((5, 4, 6, 3), 1, (1, 4, 6, 1))])
@pytest.mark.parametrize("act", ["identity", "gelu"])
def test_layernorm_with_parameters_along_other_dims_vs_torch(shape, nd, pshape, act):
    """Statistics over the leading `nd` dims, parameters broadcast along others (the reference's own test
    configurations: dims = Colon() with (1, 1, C, 1) parameters): torch layer_norm without affine
    parameters, then the broadcast affine transform, differentiated by autograd."""
    from tests.test_oracle_activations import TORCH
    x, delta = RNG.normal(size=shape), RNG.normal(size=shape)
    g, b = RNG.uniform(0.5, 1.5, pshape), RNG.normal(size=pshape)
    eps = 1e-5
    dims = tuple(range(nd))
    y = O.layernorm(x, g, b, act, dims, eps)
    dx, dg, db = O.layernorm_pullback(x, g, b, act, dims, eps, delta)
    rev = tuple(reversed(range(len(shape))))
    tx = torch.tensor(np.transpose(x, rev).copy(), requires_grad=True)
    tg = torch.tensor(np.transpose(g, rev).copy(), requires_grad=True)
    tb = torch.tensor(np.transpose(b, rev).copy(), requires_grad=True)
    ty = TORCH[act](F.layer_norm(tx, tuple(reversed(shape[:nd])), None, None, eps) * tg + tb)
    ty.backward(torch.tensor(np.transpose(delta, rev).copy()))
    np.testing.assert_allclose(y, np.transpose(ty.detach().numpy(), rev), rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(dx, np.transpose(tx.grad.numpy(), rev), rtol=1e-8, atol=1e-10)
    np.testing.assert_allclose(dg, np.transpose(tg.grad.numpy(), rev), rtol=1e-9, atol=1e-11)
    np.testing.assert_allclose(db, np.transpose(tb.grad.numpy(), rev), rtol=1e-9, atol=1e-11)


# ----------------------------------------------------------------------------- conv
def brute_conv(x, w, cd):
    """7-loop direct convolution straight from the index formula
    y[o] = sum_k w[k] x[(o)*s + (K-1-k)*d - pad_lo] (0-based), grouped."""
    W, H, Cin, N = x.shape
    kW, kH, Cg, Cout = w.shape
    OW, OH = cd.out_spatial
    G = cd.groups
    y = np.zeros((OW, OH, Cout, N))
    for n in range(N):
        for co in range(Cout):
            g = co // (Cout // G)
            for oh in range(OH):
                for ow in range(OW):
                    acc = 0.0
                    for b in range(kH):
                        for a in range(kW):
                            ka = a if cd.flipkernel else kW - 1 - a
                            kb = b if cd.flipkernel else kH - 1 - b
                            iw = ow * cd.stride[0] + ka * cd.dilation[0] - cd.padding[0]
                            ih = oh * cd.stride[1] + kb * cd.dilation[1] - cd.padding[2]
                            if 0 <= iw < W and 0 <= ih < H:
                                for c in range(Cg):
                                    acc += w[a, b, c, co] * x[iw, ih, g * Cg + c, n]
                    y[ow, oh, co, n] = acc
    return y


def test_conv_reference_impulse_known_answer():
    # test/core_layers/conv_tests.jl:145-190: delta at the centre of 7x7, 3x3 kernel
    #   => y[2:4, 2:4] == w  (true convolution orientation)
    x = np.zeros((7, 7, 1, 1))
    x[3, 3, 0, 0] = 1
    w = RNG.normal(size=(3, 3, 1, 1))
    y = O.conv(x, w, O.ConvDims(x.shape, w.shape))
    assert y.shape == (5, 5, 1, 1)
    np.testing.assert_array_equal(y[1:4, 1:4, 0, 0], w[:, :, 0, 0])
    # cross-correlation flips it
    yc = O.conv(x, w, O.ConvDims(x.shape, w.shape, flipkernel=True))
    np.testing.assert_array_equal(yc[1:4, 1:4, 0, 0], w[::-1, ::-1, 0, 0])


def test_conv_reference_asymmetric_padding_known_answer():
    # test/core_layers/conv_tests.jl:54-69: ones(28,28,1,1), 3x3 ones kernel, pad=(0, 1, 1, 2):
    # the reference checks size (27, 29) and the counts 6, 9, 4, 3, 6, 2 at fixed positions.
    x = np.ones((28, 28, 1, 1))
    w = np.ones((3, 3, 1, 1))
    y = O.conv(x, w, O.ConvDims(x.shape, w.shape, padding=(0, 1, 1, 2)))
    assert y.shape == (27, 29, 1, 1)
    y = y[:, :, 0, 0]
    assert y[0, 0] == 6.0            # (1, 1)
    assert y[1, 1] == 9.0            # (2, 2)
    assert y[26, 0] == 4.0           # (end, 1)
    assert y[0, 28] == 3.0           # (1, end)
    assert y[0, 27] == 6.0           # (1, end-1)
    assert y[26, 28] == 2.0          # (end, end)


CONV_CASES = [
    # (x shape, w shape, stride, pad, dilation, groups, flip)
    ((6, 5, 4, 2), (2, 2, 4, 6), 1, 0, 1, 1, False),
    ((6, 5, 4, 2), (2, 2, 4, 6), 2, 1, 1, 1, False),
    ((6, 5, 4, 2), (2, 2, 2, 6), 1, 1, 1, 2, False),      # groups=2 (conv_tests.jl:87-92)
    ((7, 8, 3, 2), (3, 3, 3, 5), (2, 1), (0, 1, 2, 1), (1, 2), 1, False),
    ((7, 8, 3, 2), (3, 2, 3, 5), 1, 1, 1, 1, True),
]


@pytest.mark.parametrize("xs,ws,stride,pad,dil,groups,flip", CONV_CASES)
def test_conv_vs_bruteforce_and_torch(xs, ws, stride, pad, dil, groups, flip):
    x, w = RNG.normal(size=xs), RNG.normal(size=ws)
    cd = O.ConvDims(xs, ws, stride=stride, padding=pad, dilation=dil, groups=groups, flipkernel=flip)
    y = O.conv(x, w, cd)
    np.testing.assert_allclose(y, brute_conv(x, w, cd), rtol=1e-12, atol=1e-12)
    # torch conv2d is cross-correlation over NCHW; flip the kernel spatially unless flipkernel
    tx = torch.tensor(np.transpose(x, (3, 2, 1, 0)).copy(), requires_grad=True)      # N C H W
    wk = w if flip else w[::-1, ::-1]
    tw = torch.tensor(np.transpose(wk, (3, 2, 1, 0)).copy(), requires_grad=True)     # Cout Cin kH kW
    p = cd.padding
    txp = F.pad(tx, (p[0], p[1], p[2], p[3]))
    ty = F.conv2d(txp, tw, None, stride=(cd.stride[1], cd.stride[0]), dilation=(cd.dilation[1], cd.dilation[0]),
                  groups=groups)
    np.testing.assert_allclose(y, np.transpose(ty.detach().numpy(), (3, 2, 1, 0)), rtol=1e-11, atol=1e-11)
    delta = RNG.normal(size=y.shape)
    ty.backward(torch.tensor(np.transpose(delta, (3, 2, 1, 0)).copy()))
    dx = O.conv_data_grad(delta, w, cd)
    dw = O.conv_filter_grad(x, delta, cd)
    np.testing.assert_allclose(dx, np.transpose(tx.grad.numpy(), (3, 2, 1, 0)), rtol=1e-10, atol=1e-11)
    twg = np.transpose(tw.grad.numpy(), (3, 2, 1, 0))
    np.testing.assert_allclose(dw, twg if flip else twg[::-1, ::-1], rtol=1e-10, atol=1e-11)


@pytest.mark.parametrize("xs,ws,stride,pad,dil,groups,flip", [
    ((12, 4, 2), (3, 4, 6), 1, (1, 1), 1, 1, False), ((13, 6, 3), (4, 3, 4), 2, (0, 2), 2, 2, False),
    ((9, 2, 2), (2, 2, 3), 1, (1, 0), 1, 1, True)])
def test_conv_one_spatial_dim_vs_torch(xs, ws, stride, pad, dil, groups, flip):
    """(W, C, N) inputs as a height-1 problem against torch conv1d (cross-correlation over NCW)."""
    x, w = RNG.normal(size=xs), RNG.normal(size=ws)
    cd = O.ConvDims.one_spatial_dim(xs, ws, stride, pad, dil, groups, flip)
    x4, w4 = x.reshape(cd.x_shape), w.reshape(cd.w_shape)
    y = O.conv(x4, w4, cd)
    tx = torch.tensor(np.transpose(x, (2, 1, 0)).copy(), requires_grad=True)
    tw = torch.tensor(np.transpose(w if flip else w[::-1], (2, 1, 0)).copy(), requires_grad=True)
    ty = F.conv1d(F.pad(tx, pad), tw, None, stride=stride, dilation=dil, groups=groups)
    assert y.shape[1] == 1
    np.testing.assert_allclose(y[:, 0], np.transpose(ty.detach().numpy(), (2, 1, 0)), rtol=1e-11, atol=1e-11)
    delta = RNG.normal(size=y.shape)
    ty.backward(torch.tensor(np.transpose(delta[:, 0], (2, 1, 0)).copy()))
    np.testing.assert_allclose(O.conv_data_grad(delta, w4, cd)[:, 0], np.transpose(tx.grad.numpy(), (2, 1, 0)),
                               rtol=1e-10, atol=1e-11)
    twg = np.transpose(tw.grad.numpy(), (2, 1, 0))
    np.testing.assert_allclose(O.conv_filter_grad(x4, delta, cd)[:, 0], twg if flip else twg[::-1], rtol=1e-10, atol=1e-11)


def test_fused_conv_pullback_finite_differences():
    xs, ws = (5, 4, 2, 2), (3, 3, 2, 3)
    x, w, b = RNG.normal(size=xs), RNG.normal(size=ws), RNG.normal(size=3)
    cd = O.ConvDims(xs, ws, padding=1)
    delta = RNG.normal(size=cd.y_shape())
    y, dw, dx, db = O.fused_conv_pullback("gelu", w, x, b, cd, delta)
    loss = lambda ww, xx, bb: (O.fused_conv_bias_activation("gelu", ww, xx, bb, cd) * delta).sum()
    np.testing.assert_allclose(dw, fd_grad(lambda v: loss(v, x, b), w), rtol=2e-6, atol=1e-8)
    np.testing.assert_allclose(dx, fd_grad(lambda v: loss(w, v, b), x), rtol=2e-6, atol=1e-8)
    np.testing.assert_allclose(db, fd_grad(lambda v: loss(w, x, v), b), rtol=2e-6, atol=1e-8)


# ----------------------------------------------------------------------------- helpers
def test_generate_fixed_array_is_column_major():
    a = O.generate_fixed_array(np.float32, (2, 3))
    np.testing.assert_allclose(a, np.array([[1, 3, 5], [2, 4, 6]], np.float32) / 6)


def test_bf16_round_trip_is_rne():
    a = np.array([1.0, 1.00390625, 1.005859375, 3.140625, -2.5], np.float32)
    r = O.round_to_bf16(a)
    # 1 + 2^-8 is a tie between 1.0 and 1+2^-7 -> rounds to even (1.0)
    assert r[0] == 1.0 and r[1] == 1.0 and r[2] == 1.0078125
    t = torch.tensor(a).to(torch.bfloat16).to(torch.float32).numpy()
    np.testing.assert_array_equal(r, t)
    big = RNG.normal(size=1000).astype(np.float32)
    np.testing.assert_array_equal(O.round_to_bf16(big), torch.tensor(big).to(torch.bfloat16).float().numpy())


def test_default_epsilon():
    # utils.jl:130: eps(T)^(5/7)
    assert abs(O.default_epsilon(np.float32) - (2.0 ** -23) ** (5 / 7)) < 1e-12


# ----------------------------------------------------------------------------- batched_matmul
@pytest.mark.parametrize("xs,ys,lc,rc", [
    ((4, 5, 3), (5, 6, 3), 2, 1), ((4, 5, 1), (5, 6, 3), 2, 1), ((4, 5, 3), (5, 6, 1), 2, 1),
    ((5, 4, 3), (5, 6, 3), 1, 1), ((4, 5, 3), (6, 5, 3), 2, 2), ((5, 4, 2, 3), (6, 5, 2, 3), 1, 2),
    ((4, 5), (5, 6, 3), 2, 1), ((4, 5, 3), (5, 6), 2, 1)])
def test_batched_matmul_vs_torch(xs, ys, lc, rc):
    # lib/LuxLib/test/common_ops/bmm_tests.jl compares with a loop of `*`; here torch.matmul + autograd
    x, y = RNG.normal(size=xs), RNG.normal(size=ys)
    z = O.batched_matmul(x, y, lc, rc)
    tx, ty = torch.tensor(x, requires_grad=True), torch.tensor(y, requires_grad=True)
    bx = tx if tx.ndim > 2 else tx.reshape(tx.shape + (1,) * (ty.ndim - 2))
    by = ty if ty.ndim > 2 else ty.reshape(ty.shape + (1,) * (tx.ndim - 2))
    nd = bx.ndim
    to_batch_first = tuple(range(nd - 1, 1, -1)) + (0, 1)
    ax = bx.permute(to_batch_first)
    ay = by.permute(to_batch_first)
    if lc == 1:
        ax = ax.transpose(-1, -2)
    if rc == 2:
        ay = ay.transpose(-1, -2)
    tz = torch.matmul(ax, ay)
    back_perm = (nd - 2, nd - 1) + tuple(range(nd - 3, -1, -1))
    np.testing.assert_allclose(z, tz.permute(back_perm).detach().numpy(), rtol=1e-12, atol=1e-12)
    delta = RNG.normal(size=z.shape)
    tz.backward(torch.tensor(delta).permute(to_batch_first).contiguous())
    dx, dy = O.batched_matmul_pullback(x, y, delta, lc, rc)
    np.testing.assert_allclose(dx, tx.grad.numpy(), rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(dy, ty.grad.numpy(), rtol=1e-11, atol=1e-12)


def test_batched_matmul_errors():
    with pytest.raises(O.DimensionMismatch):
        O.batched_matmul(np.ones((4, 5, 3)), np.ones((5, 6, 2)))
    with pytest.raises(O.DimensionMismatch):
        O.batched_matmul(np.ones((4, 5, 3)), np.ones((4, 6, 3)))
    with pytest.raises(O.ArgumentError):
        O.batched_matmul(np.ones((4, 5)), np.ones((5, 6)))


# ----------------------------------------------------------------------------- attention
@pytest.mark.parametrize("E,Ev,H,G,L,S,B,token_dim,kind", [
    (8, 8, 4, 4, 5, 5, 2, 3, "plain"), (8, 6, 4, 2, 5, 7, 2, 3, "plain"), (4, 4, 2, 2, 6, 6, 3, 3, "causal"),
    (4, 4, 2, 1, 6, 6, 1, 2, "causal"), (8, 8, 2, 2, 4, 6, 2, 3, "mask"), (8, 8, 2, 2, 4, 6, 2, 2, "bias"),
    (8, 8, 3, 3, 4, 6, 2, 3, "mask+bias")])
def test_attention_vs_torch(E, Ev, H, G, L, S, B, token_dim, kind):
    # lib/LuxLib/test/common_ops/attention_tests.jl compares with NNlib.dot_product_attention; here the
    # torch library routine on [B, H, L, E] tensors
    shape = (lambda e, h, t: (e, h, t, B) if token_dim == 3 else (e, t, h, B))
    q, k, v = RNG.normal(size=shape(E, H, L)), RNG.normal(size=shape(E, G, S)), RNG.normal(size=shape(Ev, G, S))
    mask = (RNG.uniform(size=(S, L, 1, B)) > 0.3) if "mask" in kind else None
    if mask is not None:
        mask[0] = True                                              # no fully masked query
    bias = RNG.normal(size=(S, L, H, 1)) if "bias" in kind else None
    causal = True if kind == "causal" else None
    out, w = O.scaled_dot_product_attention(q, k, v, token_dim, None, mask, causal, bias)
    canon = lambda a: torch.tensor(np.transpose(a if token_dim == 3 else np.swapaxes(a, 1, 2), (3, 1, 2, 0)).copy(),
                                   requires_grad=True)           # [B, H, T, E]
    tq, tk, tv = canon(q), canon(k), canon(v)
    tkr, tvr = tk.repeat_interleave(H // G, dim=1), tv.repeat_interleave(H // G, dim=1)
    am = None
    if bias is not None or mask is not None:
        am = torch.zeros(B, H, L, S, dtype=torch.float64)
        if bias is not None:
            am = am + torch.tensor(np.transpose(np.broadcast_to(bias, (S, L, H, B)), (3, 2, 1, 0)).copy())
        if mask is not None:
            am = am.masked_fill(~torch.tensor(np.transpose(np.broadcast_to(mask, (S, L, H, B)), (3, 2, 1, 0)).copy()), -np.inf)
    if causal:
        # the reference keeps key s for query l where s <= l, for any S and L (triu! of an S x L matrix)
        am = torch.zeros(L, S, dtype=torch.float64).masked_fill(~torch.tensor(np.triu(np.ones((S, L), bool)).T.copy()), -np.inf)
    to = F.scaled_dot_product_attention(tq, tkr, tvr, attn_mask=am)
    assert out.shape == (Ev, H, L, B) and w.shape == (S, L, H, B)
    np.testing.assert_allclose(out, np.transpose(to.detach().numpy(), (3, 1, 2, 0)), rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(w.sum(axis=0), 1.0, rtol=1e-12)
    d_out = RNG.normal(size=out.shape)
    to.backward(torch.tensor(np.transpose(d_out, (3, 1, 2, 0)).copy()))
    dq, dk, dv = O.scaled_dot_product_attention_pullback(q, k, v, d_out, token_dim, None, mask, causal, bias)
    uncanon = lambda t: (lambda a: a if token_dim == 3 else np.swapaxes(a, 1, 2))(np.transpose(t.grad.numpy(), (3, 1, 2, 0)))
    np.testing.assert_allclose(dq, uncanon(tq), rtol=1e-9, atol=1e-11)
    np.testing.assert_allclose(dk, uncanon(tk), rtol=1e-9, atol=1e-11)
    np.testing.assert_allclose(dv, uncanon(tv), rtol=1e-9, atol=1e-11)


def test_attention_scale_and_trailing_batch_dims():
    q, k, v = RNG.normal(size=(4, 2, 3, 2, 2)), RNG.normal(size=(4, 2, 5, 2, 2)), RNG.normal(size=(6, 2, 5, 2, 2))
    out, w = O.scaled_dot_product_attention(q, k, v, scale=2.0)
    assert out.shape == (6, 2, 3, 2, 2) and w.shape == (5, 3, 2, 2, 2)
    logits = np.einsum("dhsab,dhlab->slhab", k, q) / 2.0
    e = np.exp(logits)
    np.testing.assert_allclose(w, e / e.sum(axis=0), rtol=1e-12)
    np.testing.assert_allclose(out, np.einsum("ehsab,slhab->ehlab", v, w), rtol=1e-12)


# ------------------------------------------------------------------ convolutions with k spatial dims
def _conv_nd_brute(x, w, cd):
    """Element-by-element definition: y[o, co, n] = sum_{t, c} w[t, c, co] x[o*s + koff(t)*d - p, c, n]."""
    k = cd.k
    Cg, Cout = cd.w_shape[k], cd.w_shape[k + 1]
    Cout_g = Cout // cd.groups
    y = np.zeros(cd.out_spatial + (Cout, x.shape[-1]))
    for o in np.ndindex(*cd.out_spatial):
        for t in np.ndindex(*cd.w_shape[:k]):
            pos = []
            for d in range(k):
                koff = t[d] if cd.flipkernel else cd.w_shape[d] - 1 - t[d]
                pos.append(o[d] * cd.stride[d] + koff * cd.dilation[d] - cd.padding[2 * d])
            if any(p < 0 or p >= cd.x_shape[d] for d, p in enumerate(pos)):
                continue
            for co in range(Cout):
                g = co // Cout_g
                for c in range(Cg):
                    y[o + (co,)] += w[t + (c, co)] * x[tuple(pos) + (g * Cg + c,)]
    return y


def test_conv_nd_equals_the_two_dimensional_oracle():
    rng = np.random.default_rng(60)
    for stride, pad, dil, groups, flip in [((1, 1), (0, 0, 0, 0), (1, 1), 1, False), ((2, 1), (1, 2, 0, 1), (1, 2), 2, False),
                                           ((1, 2), (2, 2, 1, 1), (2, 1), 1, True)]:
        x = rng.normal(size=(9, 8, 4, 3))
        w = rng.normal(size=(3, 2, 4 // groups, 6))
        cd2 = O.ConvDims(x.shape, w.shape, stride, pad, dil, groups, flip)
        cdn = O.ConvDimsND(x.shape, w.shape, stride, pad, dil, groups, flip)
        y = O.conv(x, w, cd2)
        np.testing.assert_allclose(O.conv_nd(x, w, cdn), y, rtol=1e-12, atol=1e-12)
        dy = rng.normal(size=y.shape)
        np.testing.assert_allclose(O.conv_nd_data_grad(dy, w, cdn), O.conv_data_grad(dy, w, cd2), rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(O.conv_nd_filter_grad(x, dy, cdn), O.conv_filter_grad(x, dy, cd2), rtol=1e-12, atol=1e-12)


def test_conv_3d_against_scipy_and_brute_force():
    from scipy import signal
    rng = np.random.default_rng(61)
    # one channel, stride 1, no padding: true convolution is scipy's N-d 'valid' convolution and
    # flipkernel is its correlation
    x = rng.normal(size=(7, 6, 5, 1, 1))
    w = rng.normal(size=(3, 2, 3, 1, 1))
    got = O.conv_nd(x, w, O.ConvDimsND(x.shape, w.shape))
    np.testing.assert_allclose(got[..., 0, 0], signal.convolve(x[..., 0, 0], w[..., 0, 0], mode="valid"), rtol=1e-12, atol=1e-12)
    got = O.conv_nd(x, w, O.ConvDimsND(x.shape, w.shape, flipkernel=True))
    np.testing.assert_allclose(got[..., 0, 0], signal.correlate(x[..., 0, 0], w[..., 0, 0], mode="valid"), rtol=1e-12, atol=1e-12)
    # strides, asymmetric padding, dilation and groups against the element-by-element definition
    for flip in (False, True):
        x = rng.normal(size=(5, 4, 6, 4, 2))
        w = rng.normal(size=(2, 3, 2, 2, 4))
        cd = O.ConvDimsND(x.shape, w.shape, (1, 2, 2), (1, 0, 2, 1, 1, 2), (2, 1, 2), 2, flip)
        np.testing.assert_allclose(O.conv_nd(x, w, cd), _conv_nd_brute(x, w, cd), rtol=1e-12, atol=1e-12)


def test_conv_3d_gradients_are_the_adjoints():
    rng = np.random.default_rng(62)
    x = rng.normal(size=(5, 4, 6, 4, 2))
    w = rng.normal(size=(2, 3, 2, 2, 4))
    cd = O.ConvDimsND(x.shape, w.shape, (1, 2, 2), (1, 0, 2, 1, 1, 2), (2, 1, 2), 2)
    y = O.conv_nd(x, w, cd)
    dy = rng.normal(size=y.shape)
    x2, w2 = rng.normal(size=x.shape), rng.normal(size=w.shape)
    # <dy, conv(x2, w)> = <conv_data_grad(dy, w), x2>;  <dy, conv(x, w2)> = <conv_filter_grad(x, dy), w2>
    np.testing.assert_allclose(np.vdot(dy, O.conv_nd(x2, w, cd)), np.vdot(O.conv_nd_data_grad(dy, w, cd), x2), rtol=1e-10)
    np.testing.assert_allclose(np.vdot(dy, O.conv_nd(x, w2, cd)), np.vdot(O.conv_nd_filter_grad(x, dy, cd), w2), rtol=1e-10)


def test_attention_reference_specific_results():
    """test/common_ops/attention_tests.jl:115-170: q = k = v = reshape(1:12, 2, 2, 3, 1) ./ 12 and the
    output and weights the reference's test holds for it."""
    q = (np.arange(1, 13, dtype=np.float64) / 12).reshape((2, 2, 3, 1), order="F")
    y, w = O.scaled_dot_product_attention(q, q, q)
    ytrue = [0.429754, 0.513087, 0.613791, 0.697125, 0.46431, 0.547644, 0.647876, 0.73121, 0.49773, 0.581064, 0.680455,
             0.763788]
    wtrue = [0.313896, 0.332948, 0.353157, 0.264431, 0.328206, 0.407362, 0.219215, 0.31838, 0.462405, 0.288691, 0.331243,
             0.380066, 0.241239, 0.323893, 0.434868, 0.198438, 0.311761, 0.489801]
    np.testing.assert_allclose(y, np.reshape(ytrue, (2, 2, 3, 1), order="F"), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(w, np.reshape(wtrue, (3, 3, 2, 1), order="F"), rtol=1e-5, atol=1e-5)


def _nnlib_batched_mul(a, b):
    """NNlib.batched_mul on (M, K, B...) and (K, N, B...) arrays of equal batch dims, slice by slice."""
    out = np.zeros((a.shape[0], b.shape[1]) + a.shape[2:])
    for idx in np.ndindex(*a.shape[2:]):
        out[(slice(None), slice(None)) + idx] = a[(slice(None), slice(None)) + idx] @ b[(slice(None), slice(None)) + idx]
    return out


def test_generalized_batched_matmul_as_the_reference_tests_it():
    """test/others/bmm/generalized_bmm_tests.jl:8-22 and :36-58: the result equals NNlib.batched_mul on the
    operands after permutedims + repeat."""
    rng = np.random.default_rng(70)
    x, y = rng.normal(size=(3, 4, 5, 2)), rng.normal(size=(5, 4, 5, 1))
    want = _nnlib_batched_mul(x, np.tile(np.transpose(y, (1, 0, 2, 3)), (1, 1, 1, 2)))
    np.testing.assert_allclose(O.batched_matmul_general(x, y, 2, 2), want, rtol=1e-12, atol=1e-12)
    x, y = rng.normal(size=(3, 5, 2, 4)), rng.normal(size=(4, 5, 1, 5))
    want = _nnlib_batched_mul(np.transpose(x, (0, 3, 1, 2)), np.tile(np.transpose(y, (0, 1, 3, 2)), (1, 1, 1, 2)))
    got = O.batched_matmul_general(x, y, 4, 1, (2, 3), (4, 3))
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)
    # gradients: finite differences of sum(z .* delta)
    delta = rng.normal(size=got.shape)
    dx, dy = O.batched_matmul_general_pullback(x, y, delta, 4, 1, (2, 3), (4, 3))
    f = lambda xx, yy: float(np.sum(O.batched_matmul_general(xx, yy, 4, 1, (2, 3), (4, 3)) * delta))
    for arr, grad, which in ((x, dx, 0), (y, dy, 1)):
        assert grad.shape == arr.shape
        for idx in [tuple(rng.integers(0, n) for n in arr.shape) for _ in range(6)]:
            e = np.zeros_like(arr)
            e[idx] = 1e-5
            num = (f(x + e, y) - f(x - e, y)) / 2e-5 if which == 0 else (f(x, y + e) - f(x, y - e)) / 2e-5
            np.testing.assert_allclose(grad[idx], num, rtol=1e-6, atol=1e-8)
    # the default dims agree with the plain function
    a, b = rng.normal(size=(4, 3, 2, 5)), rng.normal(size=(3, 6, 1, 5))
    np.testing.assert_allclose(O.batched_matmul_general(a, b), O.batched_matmul(a, b), rtol=1e-12)
