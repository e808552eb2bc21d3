"""scaled_dot_product_attention forward + pullback on the GPU against the oracle
(mirrors lib/LuxLib/test/common_ops/attention_tests.jl: causal / boolean masks, bias, grouped
key/value heads, both token placements, extra batch dims)."""
import numpy as np
import pytest

from oracle import luxlib_oracle as O
from tests.util import stable_seed, assert_close, dev, f64, host_inputs

pytestmark = pytest.mark.gpu


def stored_as(dtype):
    """What storing an array of the pullback does to its values: the reference's rules pass arrays of the storage
    type from one rule to the next (bf16: rounded), and they read the forward pass's stored weights."""
    if dtype == "bf16":
        return lambda a: f64(O.round_to_bf16(np.asarray(a, np.float32)))
    return lambda a: a

CASES = [
    # E, Ev, H, G, L, S, batch dims, token_dim, kind
    (8, 8, 4, 4, 5, 5, (2,), 3, "plain"), (8, 6, 4, 2, 5, 7, (2,), 3, "plain"), (4, 4, 2, 2, 6, 6, (3,), 3, "causal"),
    (4, 4, 2, 1, 6, 6, (1,), 2, "causal"), (8, 8, 2, 2, 4, 6, (2,), 3, "mask"), (8, 8, 2, 2, 4, 6, (2,), 2, "bias"),
    (8, 8, 3, 3, 4, 6, (2,), 3, "mask+bias"), (16, 24, 2, 2, 9, 11, (2, 3), 3, "plain"),
    (64, 64, 8, 2, 128, 128, (2,), 3, "causal"), (64, 64, 4, 4, 130, 257, (1,), 3, "plain"),
    (32, 32, 2, 2, 40, 1100, (1,), 3, "bias"), (64, 128, 4, 4, 256, 256, (2,), 2, "plain"),
    # causal masks over several tiles: the products skip tiles and parts of the contraction
    (64, 64, 2, 2, 512, 512, (2,), 3, "causal"), (64, 32, 4, 2, 300, 520, (1,), 3, "causal"),
    (32, 64, 2, 1, 520, 300, (1,), 2, "causal"),
]


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("case", range(len(CASES)))
def test_forward_and_pullback(gpu, dtype, case):
    E, Ev, H, G, L, S, bdims, token_dim, kind = CASES[case]
    rng = np.random.default_rng(stable_seed("attn", case))
    shape = (lambda e, h, t: ((e, h, t) if token_dim == 3 else (e, t, h)) + bdims)
    B = int(np.prod(bdims))
    q, k, v = host_inputs(dtype, rng.normal(size=shape(E, H, L)), rng.normal(size=shape(E, G, S)), rng.normal(size=shape(Ev, G, S)))
    mask = (rng.uniform(size=(S, L, 1, B)) > 0.3) if "mask" in kind else None
    if mask is not None:
        mask[0] = True
    bias = host_inputs(dtype, rng.normal(size=(S, L, H, 1)))[0] if "bias" in kind else None
    causal = True if kind == "causal" else None
    (out, w), back = gpu.pullback(gpu.scaled_dot_product_attention, dev(gpu, q, dtype), dev(gpu, k, dtype), dev(gpu, v, dtype),
                                  1, token_dim, None, mask, causal, bias)
    wout, ww = O.scaled_dot_product_attention(f64(q), f64(k), f64(v), token_dim, None, mask, causal, f64(bias))
    tag = f"{dtype} case {case}"
    assert out.shape == wout.shape and w.shape == ww.shape
    # bf16: logits and weights are stored (rounded to 8 bits) between the three passes, as they are in the
    # reference's chain of array operations; sums of a few hundred such terms stray up to ~5 sigma somewhere
    rel = None
    assert_close(w.to_numpy(), ww, dtype, tag + " weights", rel=rel)
    if dtype == "bf16":     # the output is the product of v with the weights as stored (rounded to bf16), as in the reference
        wout, _ = O.scaled_dot_product_attention(f64(q), f64(k), f64(v), token_dim, None, mask, causal, f64(bias), weights=f64(w.to_numpy()))
    assert_close(out.to_numpy(), wout, dtype, tag + " out", rel=rel)
    (d_out,) = host_inputs(dtype, rng.normal(size=wout.shape))
    dq, dk, dv = back(dev(gpu, d_out, dtype))
    # the pullback starts from the weights as the forward pass stored them (checked above) and stores the logits' cotangent
    wdq, wdk, wdv = O.scaled_dot_product_attention_pullback(f64(q), f64(k), f64(v), f64(d_out), token_dim, None, mask, causal,
                                                            f64(bias), weights=f64(w.to_numpy()) if dtype == "bf16" else None,
                                                            stored=stored_as(dtype))
    rel = None
    assert_close(dq.to_numpy(), wdq, dtype, tag + " dq", rel=rel)
    assert_close(dk.to_numpy(), wdk, dtype, tag + " dk", rel=rel)
    assert_close(dv.to_numpy(), wdv, dtype, tag + " dv", rel=rel)


def test_argument_checks(gpu):
    d = lambda *s: gpu.DeviceArray.from_numpy(np.ones(s, np.float32))
    with pytest.raises(AssertionError):
        gpu.scaled_dot_product_attention(d(4, 2, 3), d(4, 2, 3), d(4, 2, 3))
    with pytest.raises(AssertionError):
        gpu.scaled_dot_product_attention(d(4, 2, 3, 1), d(4, 2, 3, 1), d(4, 2, 3, 1), mask=np.ones((3, 3), bool), is_causal=True)
    with pytest.raises(gpu.DimensionMismatch):
        gpu.scaled_dot_product_attention(d(4, 2, 3, 2), d(4, 2, 3, 1), d(4, 2, 3, 1))
    with pytest.raises(AssertionError):
        gpu.scaled_dot_product_attention(d(4, 3, 3, 1), d(4, 2, 3, 1), d(4, 2, 3, 1))      # 3 heads, 2 key/value groups
    with pytest.raises(AssertionError):                                                     # head_dim == token_dim
        gpu.scaled_dot_product_attention(d(2, 4, 3, 1), d(2, 4, 3, 1), d(2, 4, 3, 1), head_dim=3)


# test/common_ops/attention_tests.jl:115-170 ("Specific Results Check"): q = k = v = reshape(1:12, 2, 2, 3, 1) / 12
REFERENCE_Y = [0.429754, 0.513087, 0.613791, 0.697125, 0.46431, 0.547644, 0.647876, 0.73121, 0.49773, 0.581064, 0.680455,
               0.763788]
REFERENCE_W = [0.313896, 0.332948, 0.353157, 0.264431, 0.328206, 0.407362, 0.219215, 0.31838, 0.462405, 0.288691, 0.331243,
               0.380066, 0.241239, 0.323893, 0.434868, 0.198438, 0.311761, 0.489801]


def test_reference_specific_results(gpu):
    q = (np.arange(1, 13, dtype=np.float32) / 12).reshape((2, 2, 3, 1), order="F")
    d = gpu.DeviceArray.from_numpy(q)
    y, w = gpu.scaled_dot_product_attention(d, d, d)
    np.testing.assert_allclose(y.to_numpy(), np.reshape(REFERENCE_Y, (2, 2, 3, 1), order="F"), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(w.to_numpy(), np.reshape(REFERENCE_W, (3, 3, 2, 1), order="F"), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("bdims", [(1,), (2,), (2, 1, 3)])
@pytest.mark.parametrize("nheads", [1, 3, 5])
def test_reference_batch_sizes_and_token_first_layout(gpu, dtype, bdims, nheads):
    """attention_tests.jl:7-112: n = 15 features over 1, 3 or 5 heads, 3 queries, 4 keys, batch dims 1, 2 and
    (2, 1, 3), in the default layout and with the operands permuted to (tokens, heads, features)
    (token_dim = 1, head_dim = 3); both must give the same results, and the gradients of the permuted
    call are the permuted gradients."""
    n, lenq, lenkv = 15, 3, 4
    rng = np.random.default_rng(stable_seed("attn-layout", nheads, bdims))
    e = n // nheads
    q, k, v, dout = host_inputs(dtype, rng.normal(size=(e, nheads, lenq) + bdims), rng.normal(size=(e, nheads, lenkv) + bdims),
                                rng.normal(size=(e, nheads, lenkv) + bdims), rng.normal(size=(e, nheads, lenq) + bdims))
    wy, ww = O.scaled_dot_product_attention(f64(q), f64(k), f64(v))
    rel = None
    (y1, w1), back1 = gpu.pullback(gpu.scaled_dot_product_attention, dev(gpu, q, dtype), dev(gpu, k, dtype), dev(gpu, v, dtype))
    assert y1.shape == (e, nheads, lenq) + bdims and w1.shape == (lenkv, lenq, nheads) + bdims
    np.testing.assert_allclose(w1.to_numpy().sum(axis=0), 1.0, rtol=1e-2 if dtype == "bf16" else 1e-5)
    assert_close(y1.to_numpy(), wy, dtype, "y", rel=rel)
    perm = (2, 1, 0) + tuple(range(3, 3 + len(bdims)))
    q2, k2, v2 = (np.ascontiguousarray(np.transpose(a, perm)) for a in (q, k, v))
    (y2, w2), back2 = gpu.pullback(gpu.scaled_dot_product_attention, dev(gpu, q2, dtype), dev(gpu, k2, dtype), dev(gpu, v2, dtype),
                                   3, 1)
    assert y2.shape == y1.shape and w2.shape == w1.shape
    np.testing.assert_array_equal(y2.to_numpy(), y1.to_numpy())        # the same kernels on the same canonical operands
    np.testing.assert_array_equal(w2.to_numpy(), w1.to_numpy())
    assert_close(w2.to_numpy(), ww, dtype, "weights", rel=rel)
    wdq, wdk, wdv = O.scaled_dot_product_attention_pullback(f64(q), f64(k), f64(v), f64(dout),
                                                            weights=f64(w1.to_numpy()) if dtype == "bf16" else None,
                                                            stored=stored_as(dtype))
    g1 = back1(dev(gpu, dout, dtype))
    g2 = back2(dev(gpu, dout, dtype))
    for got1, got2, want, like, name in zip(g1, g2, (wdq, wdk, wdv), (q, k, v), "qkv"):
        assert got1.shape == like.shape and got2.shape == np.transpose(like, perm).shape
        assert_close(got1.to_numpy(), want, dtype, "d" + name, rel=None)
        np.testing.assert_array_equal(got2.to_numpy(), np.transpose(got1.to_numpy(), perm))


@pytest.mark.parametrize("head_dim,token_dim", [(2, 1), (2, 3), (3, 2), (3, 1)])
def test_every_placement_of_the_embedding_dim(gpu, head_dim, token_dim):
    rng = np.random.default_rng(stable_seed("attn-perm", head_dim, token_dim))
    E, H, G, L, S, B = 8, 4, 2, 5, 7, 3
    q, k, v, dout = (rng.normal(size=s).astype(np.float32) for s in ((E, H, L, B), (E, G, S, B), (E, G, S, B), (E, H, L, B)))
    heads_dim = ({1, 2, 3} - {head_dim, token_dim}).pop()
    # canonical axes (E, H, L) sit at positions head_dim, heads_dim, token_dim of the permuted operands
    axes = [0, 0, 0]
    axes[head_dim - 1], axes[heads_dim - 1], axes[token_dim - 1] = 0, 1, 2
    perm = tuple(axes) + (3,)
    qp, kp, vp = (np.ascontiguousarray(np.transpose(a, perm)) for a in (q, k, v))
    (y, w), back = gpu.pullback(gpu.scaled_dot_product_attention, dev(gpu, qp, "f32"), dev(gpu, kp, "f32"), dev(gpu, vp, "f32"),
                                head_dim, token_dim, None, None, True)
    wy, ww = O.scaled_dot_product_attention(f64(q), f64(k), f64(v), 3, None, None, True)
    assert_close(y.to_numpy(), wy, "f32", "y")
    assert_close(w.to_numpy(), ww, "f32", "weights")
    wd = O.scaled_dot_product_attention_pullback(f64(q), f64(k), f64(v), f64(dout), 3, None, None, True)
    for got, want, name in zip(back(dev(gpu, dout, "f32")), wd, "qkv"):
        assert_close(got.to_numpy(), np.transpose(want, perm), "f32", "d" + name)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_dropout_of_the_attention_weights(gpu, dtype):
    """attention_tests.jl:291-299: fdrop = dropout with p = 0.5 on q = k = v of size (5, 2, 10, 10): about half
    of the returned weights are positive.  Beyond that: the output is v times the dropped weights, and
    the pullback takes the cotangent through the same mask."""
    rng = np.random.default_rng(12)
    (q,) = host_inputs(dtype, rng.uniform(size=(5, 2, 10, 10)))
    d = dev(gpu, q, dtype)
    fdrop = gpu.attention_dropout(gpu.PhiloxRNG(77, 0), 0.5)
    (y, w), back = gpu.pullback(gpu.scaled_dot_product_attention, d, d, d, fdrop=fdrop)
    wn = w.to_numpy().astype(np.float64)
    assert 0.4 < np.mean(wn > 0) < 0.6
    _, w_plain = gpu.scaled_dot_product_attention(d, d, d)
    wp = w_plain.to_numpy().astype(np.float64)
    noise = O.rand_uniform(wp.size, 77, 0, bf16=(dtype == "bf16")).reshape(wp.shape, order="F")
    keep = noise > 0.5
    assert_close(wn, np.where(keep, 2.0 * wp, 0.0), dtype, "dropped weights")
    assert_close(y.to_numpy(), np.einsum("ehsb,slhb->ehlb", f64(q), wn), dtype, "output", rel=None)
    # pullback against the oracle's chain with the mask applied to the weights' cotangent
    (dout,) = host_inputs(dtype, rng.normal(size=q.shape))
    dq, dk, dv = back(dev(gpu, dout, dtype))
    qf, do = f64(q), f64(dout)
    inv = 1.0 / np.sqrt(5.0)
    st = stored_as(dtype)
    dw = st(st(np.einsum("ehsb,ehlb->slhb", qf, do)) * np.where(keep, 2.0, 0.0))     # product, then fdrop's pullback: two stored arrays
    ds = st(wp * (dw - (dw * wp).sum(axis=0, keepdims=True)) * inv)
    want_dq = np.einsum("dhsb,slhb->dhlb", qf, ds)
    want_dk = np.einsum("dhlb,slhb->dhsb", qf, ds)
    want_dv = np.einsum("ehlb,slhb->ehsb", do, wn)
    rel = None
    assert_close(dq.to_numpy(), want_dq, dtype, "dq", rel=rel, scale=0.05)
    assert_close(dk.to_numpy(), want_dk, dtype, "dk", rel=rel, scale=0.05)
    assert_close(dv.to_numpy(), want_dv, dtype, "dv", rel=rel)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_causal_mask_with_dropout_of_the_weights(gpu, dtype):
    """is_causal together with an fdrop over several tiles (S = L = 512): the products of the pullback run in
    full, so every element of the logits' cotangent must have been written.  The allocator's pool is filled
    with NaN first, so that memory a kernel skipped shows up in dq / dk."""
    E, H, L, B = 64, 2, 512, 2
    rng = np.random.default_rng(stable_seed("attn-causal-fdrop", dtype))
    q, k, v = host_inputs(dtype, *(rng.normal(size=(E, H, L, B)) for _ in range(3)))
    (dout,) = host_inputs(dtype, rng.normal(size=(E, H, L, B)))
    poison = [dev(gpu, np.full((L, L, H, B), np.nan, np.float32), dtype) for _ in range(4)]
    del poison                                           # back to the pool: the next tensors of this size reuse it
    p = 0.25
    fdrop = gpu.attention_dropout(gpu.PhiloxRNG(5, 0), p)
    (y, w), back = gpu.pullback(gpu.scaled_dot_product_attention, dev(gpu, q, dtype), dev(gpu, k, dtype), dev(gpu, v, dtype),
                                1, 3, None, None, True, None, fdrop)
    dq, dk, dv = back(dev(gpu, dout, dtype))
    _, wp = O.scaled_dot_product_attention(f64(q), f64(k), f64(v), 3, None, None, True, None)
    noise = O.rand_uniform(wp.size, 5, 0, bf16=(dtype == "bf16")).reshape(wp.shape, order="F")
    # p = 0.25 is exact in both storage types; the mask holds 1 / (1 - p) in the storage type (bf16: 1.3359375)
    keep = np.where(noise > np.float32(p), float(stored_as(dtype)(np.array(1.0 / (1.0 - p)))), 0.0)
    wd = wp * keep
    rel = None
    assert_close(w.to_numpy(), wd, dtype, "dropped causal weights", rel=rel)
    if dtype == "bf16":                                   # the products read the weights as the forward pass stored them
        wd = f64(w.to_numpy())
    assert_close(y.to_numpy(), np.einsum("ehsb,slhb->ehlb", f64(v), wd), dtype, "output", rel=rel)
    do, inv = f64(dout), 1.0 / np.sqrt(float(E))
    st = stored_as(dtype)
    if dtype == "bf16":                                   # the pullback reads the softmax result as stored
        wp = st(wp)
    dw = st(st(np.einsum("ehsb,ehlb->slhb", f64(v), do)) * keep)
    ds = st(wp * (dw - (dw * wp).sum(axis=0, keepdims=True)) * inv)
    rel = None
    for got, want, name in ((dq, np.einsum("dhsb,slhb->dhlb", f64(k), ds), "dq"), (dk, np.einsum("dhlb,slhb->dhsb", f64(q), ds), "dk"),
                            (dv, np.einsum("ehlb,slhb->ehsb", do, wd), "dv")):
        g = got.to_numpy()
        assert np.isfinite(g.astype(np.float64)).all(), name + " holds values from memory that no kernel wrote"
        assert_close(g, want, dtype, name, rel=rel)
