"""Golden vectors (tests/golden/luxlib_golden.npz, written by tests/golden/make_golden.py):
the oracle must keep reproducing them (CPU), and the HIP path must match them (GPU)."""
import os

import numpy as np
import pytest

from oracle import luxlib_oracle as O
from tests.util import assert_close

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "luxlib_golden.npz"))


def test_oracle_reproduces_golden_vectors():
    y, dW, dx, db = O.fused_dense_pullback("tanh", G["dense_W"], G["dense_x"], G["dense_b"], G["dense_delta"])
    for got, k in ((y, "dense_y"), (dW, "dense_dW"), (dx, "dense_dx"), (db, "dense_db")):
        np.testing.assert_allclose(got, G[k], rtol=1e-13, atol=1e-14)
    y, rm, rv = O.batchnorm(G["bn_x"], G["bn_gamma"], G["bn_beta"], G["bn_rmean"], G["bn_rvar"], True, "relu", 0.1, 1e-5)
    np.testing.assert_allclose(y, G["bn_y"], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(rv, G["bn_rvar_out"], rtol=1e-13)
    y, *_ = O.batchnorm(G["kat_bn_x"], np.ones(2), np.zeros(2), np.zeros(2), np.ones(2), True, "identity", 0.1, 1e-5)
    np.testing.assert_allclose(y, G["kat_bn_y"], atol=1e-5)
    np.testing.assert_allclose(O.groupnorm(G["bn_x"], G["bn_gamma"], G["bn_beta"], 3, "swish", 1e-5), G["gn_y"], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(O.layernorm(G["bn_x"], G["ln_gamma"], G["ln_beta"], "identity", (0, 1, 2), 1e-5), G["ln_y"],
                               rtol=1e-12, atol=1e-13)
    cd = O.ConvDims(G["conv_x"].shape, G["conv_w"].shape, stride=2, padding=1, groups=2)
    y, dw, dx, db = O.fused_conv_pullback("sigmoid", G["conv_w"], G["conv_x"], G["conv_b"], cd, G["conv_delta"])
    for got, k in ((y, "conv_y"), (dw, "conv_dw"), (dx, "conv_dx"), (db, "conv_db")):
        np.testing.assert_allclose(got, G[k], rtol=1e-12, atol=1e-13)
    y, rm, rv = O.instancenorm(G["bn_x"], G["bn_gamma"], G["bn_beta"], G["bn_rmean"], G["bn_rvar"], True, "relu", 0.1, 1e-5)
    for got, k in ((y, "in_y"), (rm, "in_rmean_out"), (rv, "in_rvar_out")):
        np.testing.assert_allclose(got, G[k], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(O.batched_matmul(G["bmm_x"], G["bmm_y"], 2, 2), G["bmm_z"], rtol=1e-13, atol=1e-14)
    out, w = O.scaled_dot_product_attention(G["attn_q"], G["attn_k"], G["attn_v"], 3, None, None, True, None)
    np.testing.assert_allclose(out, G["attn_out"], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(w, G["attn_weights"], rtol=1e-12, atol=1e-14)
    np.testing.assert_array_equal(O.rand_uniform(24, 7, 2).reshape((4, 3, 2), order="F"), G["drop_noise"].astype(np.float32))
    y, w = O.scaled_dot_product_attention(G["kat_attn_q"], G["kat_attn_q"], G["kat_attn_q"])
    np.testing.assert_allclose(y, G["kat_attn_y"], rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(w, G["kat_attn_w"], rtol=1e-5, atol=1e-5)
    cd3 = O.ConvDimsND(G["conv3_x"].shape, G["conv3_w"].shape, (1, 2, 1), (1, 0, 0, 1, 1, 1), 1, 2)
    for got, k in zip(O.fused_conv_nd_pullback("gelu", G["conv3_w"], G["conv3_x"], G["conv3_b"], cd3, G["conv3_delta"]),
                      ("conv3_y", "conv3_dw", "conv3_dx", "conv3_db")):
        np.testing.assert_allclose(got, G[k], rtol=1e-12, atol=1e-13)
    eps = float(G["lnc_eps"])
    np.testing.assert_allclose(O.layernorm(G["lnc_x"], G["lnc_gamma"], G["lnc_beta"], "sigmoid_fast", (0, 1, 2, 3), eps), G["lnc_y"],
                               rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(O.batched_matmul_general(G["gbmm_x"], G["gbmm_y"], 4, 1, (2, 3), (4, 3)), G["gbmm_z"], rtol=1e-13,
                               atol=1e-14)


@pytest.mark.gpu
def test_hip_path_matches_golden_vectors(gpu):
    d = lambda k: gpu.DeviceArray.from_numpy(G[k].astype(np.float32))
    chk = lambda got, k, **kw: assert_close(got.to_numpy(), G[k], "f32", k, **kw)
    y, back = gpu.pullback(gpu.fused_dense_bias_activation, "tanh", d("dense_W"), d("dense_x"), d("dense_b"))
    dW, dx, db = back(d("dense_delta"))
    chk(y, "dense_y"); chk(dW, "dense_dW"); chk(dx, "dense_dx"); chk(db, "dense_db")
    y, back = gpu.pullback(gpu.bias_activation, "gelu", d("ba_x"), d("ba_b"))
    dx, db = back(d("ba_delta"))
    chk(y, "ba_y"); chk(dx, "ba_dx"); chk(db, "ba_db")
    (y, st), back = gpu.pullback(gpu.batchnorm, d("bn_x"), d("bn_gamma"), d("bn_beta"), d("bn_rmean"), d("bn_rvar"), True,
                                 "relu", 0.1, 1e-5)
    dx, dg, dbt = back(d("bn_delta"))
    chk(y, "bn_y"); chk(st["running_mean"], "bn_rmean_out"); chk(st["running_var"], "bn_rvar_out")
    chk(dx, "bn_dx", scale=2.0); chk(dg, "bn_dgamma", scale=1.0); chk(dbt, "bn_dbeta", scale=1.0)
    y, back = gpu.pullback(gpu.groupnorm, d("bn_x"), d("bn_gamma"), d("bn_beta"), 3, "swish", 1e-5)
    dx, dg, dbt = back(d("bn_delta"))
    chk(y, "gn_y"); chk(dx, "gn_dx", scale=2.0); chk(dg, "gn_dgamma", scale=1.0); chk(dbt, "gn_dbeta", scale=1.0)
    y, back = gpu.pullback(gpu.layernorm, d("bn_x"), d("ln_gamma"), d("ln_beta"), "identity", (1, 2, 3), 1e-5)
    dx, dg, dbt = back(d("bn_delta"))
    chk(y, "ln_y"); chk(dx, "ln_dx", scale=2.0); chk(dg, "ln_dgamma", scale=1.0); chk(dbt, "ln_dbeta", scale=1.0)
    cd = gpu.DenseConvDims(G["conv_x"].shape, G["conv_w"].shape, stride=2, padding=1, groups=2)
    y, back = gpu.pullback(gpu.fused_conv_bias_activation, "sigmoid", d("conv_w"), d("conv_x"), d("conv_b"), cd)
    dw, dx, db = back(d("conv_delta"))
    chk(y, "conv_y"); chk(dw, "conv_dw"); chk(dx, "conv_dx"); chk(db, "conv_db")
    # reference known answers straight through the device
    yk, stk = gpu.batchnorm(d("kat_bn_x"), gpu.DeviceArray.from_numpy(np.ones(2, np.float32)),
                            gpu.DeviceArray.from_numpy(np.zeros(2, np.float32)), gpu.DeviceArray.from_numpy(np.zeros(2, np.float32)),
                            gpu.DeviceArray.from_numpy(np.ones(2, np.float32)), True, "identity", 0.1, 1e-5)
    np.testing.assert_allclose(yk.to_numpy(), G["kat_bn_y"], atol=1e-5)
    np.testing.assert_allclose(stk["running_mean"].to_numpy(), G["kat_bn_running_mean"], rtol=1e-6)
    np.testing.assert_allclose(stk["running_var"].to_numpy(), G["kat_bn_running_var"], rtol=1e-6)
    # the widened operators
    (y, st), back = gpu.pullback(gpu.instancenorm, d("bn_x"), d("bn_gamma"), d("bn_beta"), d("bn_rmean"), d("bn_rvar"), True,
                                 "relu", 0.1, 1e-5)
    dx, dg, dbt = back(d("bn_delta"))
    chk(y, "in_y"); chk(st["running_mean"], "in_rmean_out"); chk(st["running_var"], "in_rvar_out")
    chk(dx, "in_dx", scale=2.0); chk(dg, "in_dgamma", scale=1.0); chk(dbt, "in_dbeta", scale=1.0)
    z, back = gpu.pullback(gpu.batched_matmul, d("bmm_x"), d("bmm_y"), 2, 2)
    dx, dy = back(d("bmm_delta"))
    chk(z, "bmm_z", scale=1.0); chk(dx, "bmm_dx", scale=2.0); chk(dy, "bmm_dy", scale=1.0)
    (out, w), back = gpu.pullback(gpu.scaled_dot_product_attention, d("attn_q"), d("attn_k"), d("attn_v"), 1, 3, None, None, True,
                                  None)
    dq, dk, dv = back(d("attn_delta"))
    chk(out, "attn_out"); chk(w, "attn_weights"); chk(dq, "attn_dq", scale=0.5); chk(dk, "attn_dk", scale=0.5)
    chk(dv, "attn_dv", scale=0.5)
    rng = gpu.PhiloxRNG(7, 2)
    noise, _ = gpu.rand_uniform(rng, (4, 3, 2))
    np.testing.assert_array_equal(noise.to_numpy(), G["drop_noise"].astype(np.float32))
    y, mask, _ = gpu.dropout(rng, d("drop_x"), 0.25, True, 1.0 / 0.75)
    np.testing.assert_array_equal(mask.to_numpy(), G["drop_mask"].astype(np.float32))
    np.testing.assert_array_equal(y.to_numpy(), G["drop_y"].astype(np.float32))
    # the reference's attention known answer, three spatial dims, layernorm over every dim, batching dims in the middle
    q = d("kat_attn_q")
    y, w = gpu.scaled_dot_product_attention(q, q, q)
    np.testing.assert_allclose(y.to_numpy(), G["kat_attn_y"], rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(w.to_numpy(), G["kat_attn_w"], rtol=1e-5, atol=1e-5)
    cd3 = gpu.DenseConvDims(G["conv3_x"].shape, G["conv3_w"].shape, stride=(1, 2, 1), padding=(1, 0, 0, 1, 1, 1), groups=2)
    y, back = gpu.pullback(gpu.fused_conv_bias_activation, "gelu", d("conv3_w"), d("conv3_x"), d("conv3_b"), cd3)
    dw, dx, db = back(d("conv3_delta"))
    chk(y, "conv3_y"); chk(dw, "conv3_dw", scale=1.0); chk(dx, "conv3_dx", scale=1.0); chk(db, "conv3_db", scale=1.0)
    y, back = gpu.pullback(gpu.layernorm, d("lnc_x"), d("lnc_gamma"), d("lnc_beta"), "sigmoid_fast", gpu.COLON, float(G["lnc_eps"]))
    dx, dg, dbt = back(d("lnc_delta"))
    chk(y, "lnc_y"); chk(dx, "lnc_dx", scale=0.5); chk(dg, "lnc_dgamma", scale=0.5); chk(dbt, "lnc_dbeta", scale=0.5)
    z, back = gpu.pullback(gpu.batched_matmul, d("gbmm_x"), d("gbmm_y"), 4, 1, (2, 3), (4, 3))
    dx, dy = back(d("gbmm_delta"))
    chk(z, "gbmm_z", scale=1.0); chk(dx, "gbmm_dx", scale=1.0); chk(dy, "gbmm_dy", scale=1.0)
