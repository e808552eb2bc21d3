"""scaled_dot_product_attention forward + pullback on the GPU against the oracle
(mirrors lib/LuxLib/test/common_ops/attention_tests.jl: causal / boolean masks, bias, grouped
key/value heads, both token placements, extra batch dims)."""
import numpy as np
import pytest

from oracle import luxlib_oracle as O
from tests.util import stable_seed, assert_close, dev, f64, host_inputs

pytestmark = pytest.mark.gpu

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
    rel = None if dtype == "f32" else 4e-2
    assert_close(w.to_numpy(), ww, dtype, tag + " weights", rel=rel)
    assert_close(out.to_numpy(), wout, dtype, tag + " out", rel=rel)
    (d_out,) = host_inputs(dtype, rng.normal(size=wout.shape))
    dq, dk, dv = back(dev(gpu, d_out, dtype))
    wdq, wdk, wdv = O.scaled_dot_product_attention_pullback(f64(q), f64(k), f64(v), f64(d_out), token_dim, None, mask, causal,
                                                            f64(bias))
    rel = None if dtype == "f32" else 6e-2
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
    with pytest.raises(gpu.Unsupported):
        gpu.scaled_dot_product_attention(d(2, 4, 3, 1), d(2, 4, 3, 1), d(2, 4, 3, 1), head_dim=2)
