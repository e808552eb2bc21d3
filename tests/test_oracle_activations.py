"""Pins the oracle's activation table: closed forms / library routines / finite differences.

Mirrors lib/LuxLib/test/common_ops/activation_tests.jl:9-67 (11 activations, values and
gradients, finite-difference ground truth) of the reference."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import luxlib_oracle as O

ACTS = ["identity", "relu", "sigmoid", "sigmoid_fast", "softplus", "logsigmoid", "gelu", "swish",
        "lisht", "tanh", "tanh_fast"]

TORCH = {
    "identity": lambda t: t,
    "relu": F.relu,
    "sigmoid": torch.sigmoid,
    "sigmoid_fast": torch.sigmoid,
    "softplus": F.softplus,
    "logsigmoid": F.logsigmoid,
    "gelu": lambda t: F.gelu(t, approximate="tanh"),
    "swish": F.silu,
    "lisht": lambda t: t * torch.tanh(t),
    "tanh": torch.tanh,
    "tanh_fast": torch.tanh,
}


@pytest.mark.parametrize("act", ACTS)
def test_values_match_library_routines(act):
    x = np.linspace(-6, 6, 241).astype(np.float64)
    want = TORCH[act](torch.from_numpy(x)).numpy()
    np.testing.assert_allclose(O.act_value(act, x), want, rtol=1e-12, atol=1e-13)
    x32 = x.astype(np.float32)
    got32 = O.act_value(act, x32)
    assert got32.dtype == np.float32
    np.testing.assert_allclose(got32, want, rtol=2e-6, atol=2e-7)


@pytest.mark.parametrize("act", ACTS)
def test_derivative_matches_finite_differences_and_autograd(act):
    rng = np.random.default_rng(7)
    x = rng.normal(size=400) * 2.5
    x = x[np.abs(x) > 1e-3]          # relu kink
    h = 1e-6
    fd = (O.act_value(act, x + h) - O.act_value(act, x - h)) / (2 * h)
    out = O.act_value(act, x)
    got = O.act_derivative(act, out, x)
    np.testing.assert_allclose(got, fd, rtol=1e-7, atol=1e-8)
    t = torch.from_numpy(x).requires_grad_(True)
    TORCH[act](t).sum().backward()
    if act != "identity":
        np.testing.assert_allclose(got, t.grad.numpy(), rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("act", ["identity", "relu", "tanh", "sigmoid"])
def test_output_only_derivative(act):
    """Branch 1 of the rrule (impl/dense.jl:83-92): derivative from Ω alone."""
    x = np.linspace(-3, 3, 61)
    out = O.act_value(act, x)
    np.testing.assert_array_equal(O.act_derivative(act, out, None), O.act_derivative(act, out, x))
    assert O.ACT_NEEDS[O.canonical_act(act)] in ("none", "out")


def test_relu_derivative_at_zero_is_zero():
    assert O.act_derivative("relu", np.zeros(3), None).tolist() == [0, 0, 0]


def test_known_special_values():
    z = np.zeros(1)
    assert O.act_value("sigmoid", z)[0] == 0.5
    assert O.act_value("gelu", z)[0] == 0.0
    assert O.act_value("swish", z)[0] == 0.0
    assert abs(O.act_value("softplus", z)[0] - np.log(2)) < 1e-15
    assert abs(O.act_value("logsigmoid", z)[0] + np.log(2)) < 1e-15
    # gelu tanh-approximation constant check: differs from erf-gelu by ~1e-4 at x=1
    erf_gelu = 0.5 * (1 + torch.erf(torch.tensor(1.0, dtype=torch.float64) / 2 ** 0.5)).item()
    assert 1e-5 < abs(O.act_value("gelu", np.ones(1))[0] - erf_gelu) < 1e-3


def test_unknown_activation_rejected():
    with pytest.raises(ValueError):
        O.act_value("cube", np.ones(2))
