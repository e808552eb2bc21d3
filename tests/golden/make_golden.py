#!/usr/bin/env python3
"""Writes tests/golden/luxlib_golden.npz: small input/output vectors of every operator on the
path, on the deterministic inputs the reference's own tests use
(`generate_fixed_array`, lib/LuxLib/test/shared_testsetup.jl:69-73), with outputs from the
fp64 oracle, plus the reference's known-answer vectors as plain data.

The reference is Julia and cannot run here, so nothing is imported from it: the oracle that
produces these outputs is pinned independently (tests/test_oracle_*.py).  Run from the repo
root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import luxlib_oracle as O  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "luxlib_golden.npz")


def fixed(shape, shift=0.0, scale=1.0):
    return (O.generate_fixed_array(np.float64, shape) - shift) * scale


def main():
    g = {}
    # --- reference known answers (test/core_layers/normalize_tests.jl:10-49, basic_tests.jl:151-194,
    #     conv_tests.jl:54-69) stored as data
    g["kat_bn_x"] = np.array([[1.0, 3.0, 5.0], [2.0, 4.0, 6.0]])
    g["kat_bn_y"] = np.array([[-1.22474, 0.0, 1.22474], [-1.22474, 0.0, 1.22474]])
    g["kat_bn_running_mean"] = np.array([0.3, 0.4])
    g["kat_bn_running_var"] = np.array([1.3, 1.3])
    g["kat_conv_pad_counts"] = np.array([6.0, 9.0, 4.0, 3.0, 6.0, 2.0])

    # --- dense (dense_tests.jl sizes): W 4x32, x 32x3, tanh, inputs scaled like the reference (1e-3 offsets)
    W, x, b = fixed((4, 32), 0.5), fixed((32, 3), 0.5, 2.0), fixed((4,), 0.5)
    delta = fixed((4, 3), 0.3)
    y, dW, dx, db = O.fused_dense_pullback("tanh", W, x, b, delta)
    g.update(dense_W=W, dense_x=x, dense_b=b, dense_delta=delta, dense_y=y, dense_dW=dW, dense_dx=dx, dense_db=db)

    # --- bias_activation (bias_act_tests.jl shape (2,2,3,4)), gelu
    x, b, delta = fixed((2, 2, 3, 4), 0.5, 3.0), fixed((3,), 0.5), fixed((2, 2, 3, 4), 0.4)
    y, dx, db = O.bias_activation_pullback("gelu", x, b, delta)
    g.update(ba_x=x, ba_b=b, ba_delta=delta, ba_y=y, ba_dx=dx, ba_db=db)

    # --- batchnorm (batchnorm_tests.jl shape (4,4,6,2)), training, relu
    x = fixed((4, 4, 6, 2), 0.5, 2.0) + 0.05 * np.sin(np.arange(192)).reshape((4, 4, 6, 2), order="F")
    gm, bt, rm, rv = fixed((6,), -0.5), fixed((6,), 0.5), fixed((6,), 0.5), fixed((6,), -0.5)
    delta = np.cos(np.arange(192)).reshape((4, 4, 6, 2), order="F")
    y, rm2, rv2 = O.batchnorm(x, gm, bt, rm, rv, True, "relu", 0.1, 1e-5)
    dx, dg, dbt = O.batchnorm_pullback(x, gm, bt, "relu", 1e-5, delta)
    g.update(bn_x=x, bn_gamma=gm, bn_beta=bt, bn_rmean=rm, bn_rvar=rv, bn_delta=delta, bn_y=y, bn_rmean_out=rm2,
             bn_rvar_out=rv2, bn_dx=dx, bn_dgamma=dg, bn_dbeta=dbt)

    # --- groupnorm (groupnorm_tests.jl shape (4,4,6,2), 3 groups), swish
    y = O.groupnorm(x, gm, bt, 3, "swish", 1e-5)
    dx, dg, dbt = O.groupnorm_pullback(x, gm, bt, 3, "swish", 1e-5, delta)
    g.update(gn_y=y, gn_dx=dx, gn_dgamma=dg, gn_dbeta=dbt)

    # --- layernorm (layernorm_tests.jl shape (4,4,6,2), dims 1:3, affine (4,4,6,1))
    lg, lb = fixed((4, 4, 6, 1), -0.5), fixed((4, 4, 6, 1), 0.5)
    y = O.layernorm(x, lg, lb, "identity", (0, 1, 2), 1e-5)
    dx, dg, dbt = O.layernorm_pullback(x, lg, lb, "identity", (0, 1, 2), 1e-5, delta)
    g.update(ln_gamma=lg, ln_beta=lb, ln_y=y, ln_dx=dx, ln_dgamma=dg, ln_dbeta=dbt)

    # --- conv (conv_tests.jl: kernel (2,2), stride 2, pad 1, groups 2), sigmoid
    xs, ws = (6, 5, 4, 2), (2, 2, 2, 6)
    cx, cw, cb = fixed(xs, 0.5, 2.0), fixed(ws, 0.5), fixed((6,), 0.5)
    cd = O.ConvDims(xs, ws, stride=2, padding=1, groups=2)
    cdelta = np.cos(np.arange(int(np.prod(cd.y_shape())))).reshape(cd.y_shape(), order="F")
    y, dw, dx, db = O.fused_conv_pullback("sigmoid", cw, cx, cb, cd, cdelta)
    g.update(conv_x=cx, conv_w=cw, conv_b=cb, conv_delta=cdelta, conv_y=y, conv_dw=dw, conv_dx=dx, conv_db=db)

    # --- instancenorm (instancenorm_tests.jl shape (4,4,6,2)), training with running statistics, relu
    y, rm2, rv2 = O.instancenorm(x, gm, bt, rm, rv, True, "relu", 0.1, 1e-5)
    dx, dg, dbt = O.instancenorm_pullback(x, gm, bt, "relu", 1e-5, delta)
    g.update(in_y=y, in_rmean_out=rm2, in_rvar_out=rv2, in_dx=dx, in_dgamma=dg, in_dbeta=dbt)

    # --- batched_matmul (bmm_tests.jl: a shared left operand, the right one contracted along its second dim)
    bx, by = fixed((4, 5, 1), 0.5), fixed((6, 5, 3), 0.5, 2.0)
    bz = O.batched_matmul(bx, by, 2, 2)
    bdelta = np.cos(np.arange(bz.size)).reshape(bz.shape, order="F")
    bdx, bdy = O.batched_matmul_pullback(bx, by, bdelta, 2, 2)
    g.update(bmm_x=bx, bmm_y=by, bmm_z=bz, bmm_delta=bdelta, bmm_dx=bdx, bmm_dy=bdy)

    # --- scaled_dot_product_attention (attention_tests.jl): 4 query heads on 2 key/value heads, causal
    aq, ak, av = fixed((8, 4, 5, 2), 0.5, 2.0), fixed((8, 2, 5, 2), 0.5, 2.0), fixed((6, 2, 5, 2), 0.5)
    ao, aw = O.scaled_dot_product_attention(aq, ak, av, 3, None, None, True, None)
    adelta = np.sin(np.arange(ao.size)).reshape(ao.shape, order="F")
    adq, adk, adv = O.scaled_dot_product_attention_pullback(aq, ak, av, adelta, 3, None, None, True, None)
    g.update(attn_q=aq, attn_k=ak, attn_v=av, attn_out=ao, attn_weights=aw, attn_delta=adelta, attn_dq=adq, attn_dk=adk,
             attn_dv=adv)

    # --- dropout: the first 24 values of the noise stream (seed 7, offset 2; the Philox4x32-10 known-answer
    #     vectors themselves are checked in tests/test_oracle_dropout.py), the mask and the product for p = 0.25
    dnoise = O.rand_uniform(24, 7, 2).astype(np.float64).reshape((4, 3, 2), order="F")
    dxin = fixed((4, 3, 2), 0.5, 2.0)
    dy_, dmask = O.dropout(dnoise.astype(np.float32), dxin.astype(np.float32), 0.25, True, 1.0 / 0.75)
    g.update(drop_noise=dnoise, drop_x=dxin, drop_mask=dmask, drop_y=dy_)

    # --- the attention known answer of the reference (attention_tests.jl:115-170): q = k = v = reshape(1:12, 2, 2, 3, 1) ./ 12
    g["kat_attn_q"] = (np.arange(1, 13, dtype=np.float64) / 12).reshape((2, 2, 3, 1), order="F")
    g["kat_attn_y"] = np.reshape([0.429754, 0.513087, 0.613791, 0.697125, 0.46431, 0.547644, 0.647876, 0.73121, 0.49773,
                                  0.581064, 0.680455, 0.763788], (2, 2, 3, 1), order="F")
    g["kat_attn_w"] = np.reshape([0.313896, 0.332948, 0.353157, 0.264431, 0.328206, 0.407362, 0.219215, 0.31838, 0.462405,
                                  0.288691, 0.331243, 0.380066, 0.241239, 0.323893, 0.434868, 0.198438, 0.311761, 0.489801],
                                 (3, 3, 2, 1), order="F")

    # --- convolution with three spatial dims: kernel (2, 3, 2), stride (1, 2, 1), pad (1, 0, 0, 1, 1, 1), groups 2, gelu
    x, w, b = fixed((5, 6, 4, 4, 2), 0.5, 2.0), fixed((2, 3, 2, 2, 6), 0.5), fixed((6,), 0.5)
    cd3 = O.ConvDimsND(x.shape, w.shape, (1, 2, 1), (1, 0, 0, 1, 1, 1), 1, 2)
    delta = fixed(cd3.out_spatial + (6, 2), 0.4)
    y, dw, dx, db = O.fused_conv_nd_pullback("gelu", w, x, b, cd3, delta)
    g.update(conv3_x=x, conv3_w=w, conv3_b=b, conv3_delta=delta, conv3_y=y, conv3_dw=dw, conv3_dx=dx, conv3_db=db)

    # --- layernorm as the reference's own test calls it (layernorm_tests.jl:22-32,80-86): dims = Colon() with
    #     parameters (1, 1, C, 1), on its input generator
    x = O.generate_fixed_array(np.float64, (3, 3, 2, 1))
    gam, bet = O.generate_fixed_array(np.float64, (1, 1, 2, 1)), O.generate_fixed_array(np.float64, (1, 1, 2, 1))
    delta = fixed((3, 3, 2, 1), 0.45)
    eps = O.default_epsilon(np.float32)
    y = O.layernorm(x, gam, bet, "sigmoid_fast", (0, 1, 2, 3), eps)
    dx, dg, dbt = O.layernorm_pullback(x, gam, bet, "sigmoid_fast", (0, 1, 2, 3), eps, delta)
    g.update(lnc_x=x, lnc_gamma=gam, lnc_beta=bet, lnc_delta=delta, lnc_eps=np.array(eps), lnc_y=y, lnc_dx=dx, lnc_dgamma=dg,
             lnc_dbeta=dbt)

    # --- batched_matmul with batching dims in the middle (generalized_bmm_tests.jl:36-58)
    x, y_ = fixed((3, 5, 2, 4), 0.5), fixed((4, 5, 1, 5), 0.4)
    z = O.batched_matmul_general(x, y_, 4, 1, (2, 3), (4, 3))
    delta = fixed(z.shape, 0.3)
    dx, dy = O.batched_matmul_general_pullback(x, y_, delta, 4, 1, (2, 3), (4, 3))
    g.update(gbmm_x=x, gbmm_y=y_, gbmm_z=z, gbmm_delta=delta, gbmm_dx=dx, gbmm_dy=dy)

    np.savez_compressed(OUT, **{k: np.asarray(v, dtype=np.float64) for k, v in g.items()})
    print("wrote", OUT, os.path.getsize(OUT), "bytes,", len(g), "arrays")


if __name__ == "__main__":
    main()
