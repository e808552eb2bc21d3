"""The two benchmark configurations that chain several fused operators, at full size, end to end on the GPU:
every stage's input is the device's own output of the stage before (nothing is re-uploaded in between), and every
output of every stage is compared with the oracle evaluated from the test inputs, with the device's storage
roundings (bf16 between stages) applied where the device stores a tensor.  Two comparisons take a device tensor as
oracle input, and say so where they do: relu's kink in configuration 2, and the layernorm parameter gradients of
configuration 4.  All errors measured stay below half a bf16 unit in the last place (3.9e-3) resp. 3e-7 in fp32, so
the allowances are the plain 1e-2 / 1e-5.

configuration 4: layernorm(4096 x 8192) -> dense 4096->11008 gelu -> dense 11008->4096, bf16 storage / fp32
accumulation (impl/layernorm.jl:1-36, impl/dense.jl:1-113 of the reference's LuxLib), pullback in reverse order.
configuration 2: batchnorm (training) -> bias_activation(relu), fp32 (impl/batchnorm.jl:1-120,
impl/bias_activation.jl:1-120), pullback in reverse order."""
import numpy as np
import pytest

from oracle import luxlib_oracle as O
from tests.util import assert_close, dev, f64, host_inputs, rms

pytestmark = pytest.mark.gpu


def q(a):
    """What the device keeps of a tensor it stores as bf16."""
    return f64(O.round_to_bf16(np.asarray(a, dtype=np.float32)))


def one_per_block(rng, n, block=256):
    """One random index out of every `block` consecutive ones: every tile row / column of a product is visited."""
    starts = np.arange(0, n, block)
    return np.array([s + rng.integers(0, min(block, n - s)) for s in starts])


@pytest.mark.parametrize("pretranspose", [1, 0])
def test_config4_block_full_size(gpu, pretranspose):
    rng = np.random.default_rng(1003)
    D, F, N = 4096, 11008, 8192
    std = np.sqrt(2.0 / (D + F))
    x = rng.standard_normal(size=(D, N), dtype=np.float32)
    g = rng.uniform(0.5, 1.5, (D, 1)).astype(np.float32)
    b = (0.1 * rng.standard_normal((D, 1))).astype(np.float32)
    W1 = std * rng.standard_normal(size=(F, D), dtype=np.float32)
    b1 = (0.02 * rng.standard_normal(F)).astype(np.float32)
    W2 = std * rng.standard_normal(size=(D, F), dtype=np.float32)
    b2 = (0.02 * rng.standard_normal(D)).astype(np.float32)
    delta = 0.02 * rng.standard_normal(size=(D, N), dtype=np.float32)
    x, g, b, W1, b1, W2, b2, delta = host_inputs("bf16", x, g, b, W1, b1, W2, b2, delta)
    eps = 1e-5
    dv = lambda a: dev(gpu, a, "bf16")
    gpu.set_option("gemm_pretranspose", pretranspose)
    try:
        dW1, dW2 = dv(W1), dv(W2)
        h0, back_ln = gpu.pullback(gpu.layernorm, dv(x), dv(g), dv(b), "identity", (1,), eps)
        h1, back_d1 = gpu.pullback(gpu.fused_dense_bias_activation, "gelu", dW1, h0, dv(b1))
        h2, back_d2 = gpu.pullback(gpu.fused_dense_bias_activation, "identity", dW2, h1, dv(b2))
        gW2, gh1, gb2 = back_d2(dv(delta))
        gW1, gh0, gb1 = back_d1(gh1)
        gx, gg, gb = back_ln(gh0)
        gpu.synchronize()
    finally:
        gpu.set_option("gemm_pretranspose", 1)
    tag = f"config4 block (pretranspose={pretranspose}) "

    # ---- stage 1, whole tensor: layernorm over the features of every token
    w_h0 = O.layernorm(f64(x), f64(g), f64(b), "identity", (0,), eps)
    assert_close(h0.to_numpy(), w_h0, "bf16", tag + "h0 = layernorm(x)")
    h0q = q(w_h0)

    # ---- everything that belongs to one token: a token out of every 256, all features
    tok = one_per_block(rng, N)
    z1_t = f64(W1) @ h0q[:, tok] + f64(b1)[:, None]
    h1_t = q(O.act_value("gelu", z1_t))
    assert_close(h1.to_numpy()[:, tok], O.act_value("gelu", z1_t), "bf16", tag + "h1 tokens")
    w_h2_t = f64(W2) @ h1_t + f64(b2)[:, None]
    assert_close(h2.to_numpy()[:, tok], w_h2_t, "bf16", tag + "h2 tokens")
    w_dh1_t = f64(W2).T @ f64(delta[:, tok])
    assert_close(gh1.to_numpy()[:, tok], w_dh1_t, "bf16", tag + "dh1 tokens")
    z1q_t = q(z1_t)                                          # the pullback reads the stored pre-activation
    dz1_t = q(q(w_dh1_t) * O.act_derivative("gelu", O.act_value("gelu", z1q_t), z1q_t))
    w_dh0_t = f64(W1).T @ dz1_t
    assert_close(gh0.to_numpy()[:, tok], w_dh0_t, "bf16", tag + "dh0 tokens")
    w_dx_t, _, _ = O.layernorm_pullback(f64(x[:, tok]), f64(g), f64(b), "identity", (0,), eps, q(w_dh0_t))
    var_t = f64(x[:, tok]).var(axis=0)
    assert_close(gx.to_numpy()[:, tok], w_dx_t, "bf16", tag + "dx tokens",
                 scale=rms(w_dh0_t) * 1.5 / float(np.sqrt(var_t.min() + eps)))

    # ---- everything that sums over all tokens: one hidden feature out of every 256
    hid = one_per_block(rng, F)
    z1_h = f64(W1[hid]) @ h0q + f64(b1[hid])[:, None]
    assert_close(h1.to_numpy()[hid], O.act_value("gelu", z1_h), "bf16", tag + "h1 hidden rows")
    h1q_h = q(O.act_value("gelu", z1_h))
    assert_close(gW2.to_numpy()[:, hid], f64(delta) @ h1q_h.T, "bf16", tag + "dW2 columns")
    w_dh1_h = f64(W2[:, hid]).T @ f64(delta)
    assert_close(gh1.to_numpy()[hid], w_dh1_h, "bf16", tag + "dh1 hidden rows")
    z1q_h = q(z1_h)
    dz1_exact_h = q(w_dh1_h) * O.act_derivative("gelu", O.act_value("gelu", z1q_h), z1q_h)
    assert_close(gW1.to_numpy()[hid], q(dz1_exact_h) @ h0q.T, "bf16", tag + "dW1 rows")
    assert_close(gb1.to_numpy()[hid], dz1_exact_h.sum(axis=1), "bf16", tag + "db1", scale=rms(dz1_exact_h) * 90)
    assert_close(gb2.to_numpy(), f64(delta).sum(axis=1), "bf16", tag + "db2", scale=rms(delta) * 90)

    # ---- the layernorm parameter gradients sum over all tokens of dh0, whose exact value needs the whole of dz1
    # (a product of 7.4e11 multiply-adds in fp64): the device's own dh0, checked above on a token out of every 256,
    # stands in for it here
    gh0h = f64(gh0.to_numpy())
    w_dx, w_dg, w_db = O.layernorm_pullback(f64(x), f64(g), f64(b), "identity", (0,), eps, gh0h)
    assert_close(gg.to_numpy(), w_dg, "bf16", tag + "dgamma", scale=rms(gh0h) * 90)
    assert_close(gb.to_numpy(), w_db, "bf16", tag + "dbeta", scale=rms(gh0h) * 90)
    assert_close(gx.to_numpy(), w_dx, "bf16", tag + "dx (all tokens, from the device's dh0)",
                 scale=rms(gh0h) * 1.5 / float(np.sqrt(f64(x).var(axis=0).min() + eps)))


def test_config2_chain_full_size(gpu, bn_path):
    """batchnorm (training) -> bias_activation(relu) and the pullback in reverse, every element of every output
    against the fp64 oracle."""
    rng = np.random.default_rng(1001)
    shape = (32, 32, 64, 128)
    Cn = shape[2]
    x = 0.5 + 2.0 * rng.standard_normal(size=shape, dtype=np.float32)
    g = rng.uniform(0.5, 1.5, Cn).astype(np.float32)
    b = (0.1 * rng.standard_normal(Cn)).astype(np.float32)
    bias2 = (0.1 * rng.standard_normal(Cn)).astype(np.float32)
    delta = rng.standard_normal(size=shape, dtype=np.float32)
    d = gpu.DeviceArray.from_numpy
    rm, rv = d(np.zeros(Cn, np.float32)), d(np.ones(Cn, np.float32))
    (y1, st), back_bn = gpu.pullback(gpu.batchnorm, d(x), d(g), d(b), rm, rv, True, "identity", 0.1, 1e-5)
    y2, back_ba = gpu.pullback(gpu.bias_activation, "relu", y1, d(bias2))
    gy1, gbias2 = back_ba(d(delta))
    gx, gg, gb = back_bn(gy1)
    gpu.synchronize()

    w_y1, w_rm, w_rv = O.batchnorm(f64(x), f64(g), f64(b), np.zeros(Cn), np.ones(Cn), True, "identity", 0.1, 1e-5)
    w32_y1 = O.batchnorm(x, g, b, np.zeros(Cn, np.float32), np.ones(Cn, np.float32), True, "identity", np.float32(0.1), np.float32(1e-5))[0]
    assert_close(y1.to_numpy(), w_y1, "f32", "config2 chain y1", want32=w32_y1)
    assert_close(st["running_mean"].to_numpy(), w_rm, "f32", "config2 chain running_mean")
    assert_close(st["running_var"].to_numpy(), w_rv, "f32", "config2 chain running_var")
    # relu of the float32 values the device holds: a pre-activation within rounding of zero may land on either side
    y1h = f64(y1.to_numpy())
    w_y2 = O.bias_activation("relu", y1h, f64(bias2))
    assert_close(y2.to_numpy(), w_y2, "f32", "config2 chain y2")
    _, w_dy1, w_dbias2 = O.bias_activation_pullback("relu", y1h, f64(bias2), f64(delta))
    assert_close(gy1.to_numpy(), w_dy1, "f32", "config2 chain dy1")
    assert_close(gbias2.to_numpy(), w_dbias2, "f32", "config2 chain dbias2", scale=rms(delta) * np.sqrt(delta.size / Cn))
    w_dx, w_dg, w_db = O.batchnorm_pullback(f64(x), f64(g), f64(b), "identity", 1e-5, w_dy1)
    m = np.sqrt(delta.size / Cn)
    assert_close(gx.to_numpy(), w_dx, "f32", "config2 chain dx", scale=rms(w_dy1))
    assert_close(gg.to_numpy(), w_dg, "f32", "config2 chain dgamma", scale=rms(w_dy1) * m)
    assert_close(gb.to_numpy(), w_db, "f32", "config2 chain dbeta", scale=rms(w_dy1) * m)
