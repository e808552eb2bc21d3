"""CPU restatement (numpy) of LuxLib's fused-operator forward + pullback path.

TEST INFRASTRUCTURE ONLY.  This module is the checker that the HIP path is compared
against; it is never the thing measured or shipped.  Only tests, the smoke check and the
`cpu_baseline` leg of the benchmark may import it.

Arrays carry Julia's *logical* shapes (e.g. WHCN for images, features x batch for
matrices); numpy memory order is irrelevant here.  Every function computes in the dtype
it is handed (pass float64 inputs for the fp64 arbiter, float32 for the fp32 restatement).

Each function cites the reference file:line it follows (paths relative to
lib/LuxLib/src/ of the reference unless stated otherwise).

Pinning status (what independent evidence each function is checked against, see
tests/test_oracle_*.py):
  * activations / derivatives ......... textbook closed forms, torch library routines,
                                        fp64 central finite differences
  * bias_activation (+pullback) ....... closed form, torch autograd, finite differences
  * fused_dense (+pullback) ........... reference known answers (Dense 10->1/2 with ones),
                                        torch F.linear autograd, finite differences
  * batchnorm (+running stats, bwd) ... reference known-answer test (x=[1 3 5;2 4 6]),
                                        torch F.batch_norm autograd, finite differences
  * groupnorm (+bwd) .................. torch F.group_norm autograd, finite differences
  * layernorm (+bwd) .................. mean~0/std~1 invariant, torch F.layer_norm autograd
  * scaled_dot_product_attention ...... torch F.scaled_dot_product_attention (values, causal and
                                        boolean masks, additive bias, grouped heads) + autograd
  * batched_matmul (+pullback) ........ torch.matmul over a batch + autograd
  * dropout / alpha_dropout ........... closed forms; the Philox4x32-10 noise stream against
                                        the Random123 known-answer vectors and uniformity
                                        statistics (Julia's own rng streams are out of reach)
  * instancenorm (+running stats, bwd)  torch F.instance_norm (values, running statistics,
                                        autograd), groupnorm with G = C, finite differences
  * conv / dgrad / wgrad .............. reference known answers (impulse response,
                                        asymmetric-pad counts), brute-force 7-loop direct
                                        convolution, torch conv2d with flipped kernel
  * conv_nd / its gradients (k dims) .. the 2-d functions above at k = 2; scipy.signal
                                        convolve / correlate ('valid') at k = 3; an
                                        element-by-element definition with strides, asymmetric
                                        padding, dilation and groups; adjoint identities
  * PARITY UNPINNED: the bit pattern of the reference's dropout masks (drawn from Julia's rng,
    which cannot run here); `rand_uniform` is a Philox stream of the same distribution.
  * NNlib's `tanh_fast`/`sigmoid_fast` rational approximations, exact `gelu` constants and
    Julia's summation order are NOT reproducible without Julia: parity for those is pinned
    to tolerance only (few-ulp effects), not bit-for-bit.
"""
from __future__ import annotations

import math

import numpy as np

# --------------------------------------------------------------------------------------
# Activation table.  Values: NNlib (third party, compat 0.9.33, not vendored in the
# reference tree); derivative forms: ChainRulesCore.derivatives_given_output as used by
# `only_derivative` (utils.jl:81-84) and `∇activation` (impl/activation.jl:135-154).
# swish / sigmoid / tanh derivative forms are visible in ext/SLEEFPiratesExt.jl:20-35;
# gelu is the tanh approximation (ext/CUDAExt/cublaslt.jl:308-315 maps it to
# CUBLASLT_EPILOGUE_GELU).
# --------------------------------------------------------------------------------------
ACTIVATIONS = (
    "identity", "relu", "tanh", "sigmoid", "swish", "gelu", "softplus", "logsigmoid", "lisht",
    "tanh_fast", "sigmoid_fast",
)
_ALIASES = {"tanh_fast": "tanh", "sigmoid_fast": "sigmoid", "gelu_tanh": "gelu"}

_SQRT_2_OVER_PI = math.sqrt(2.0 / math.pi)
_GELU_C = 0.044715


def canonical_act(name: str) -> str:
    name = _ALIASES.get(name, name)
    if name not in ACTIVATIONS:
        raise ValueError(f"unknown activation {name!r}")
    return name


def _sigmoid(x):
    # numerically stable logistic
    t = np.exp(-np.abs(x))
    return np.where(x >= 0, 1 / (1 + t), t / (1 + t)).astype(x.dtype, copy=False)


def act_value(name: str, x: np.ndarray) -> np.ndarray:
    """σ.(x) for the named activation."""
    name = canonical_act(name)
    x = np.asarray(x)
    T = x.dtype.type
    if name == "identity":
        return x.copy()
    if name == "relu":
        return np.maximum(x, T(0))
    if name == "tanh":
        return np.tanh(x)
    if name == "sigmoid":
        return _sigmoid(x)
    if name == "swish":
        return x * _sigmoid(x)
    if name == "gelu":
        u = T(_SQRT_2_OVER_PI) * (x + T(_GELU_C) * x * x * x)
        return T(0.5) * x * (T(1) + np.tanh(u))
    if name == "softplus":
        return np.log1p(np.exp(-np.abs(x))) + np.maximum(x, T(0))
    if name == "logsigmoid":
        return -(np.log1p(np.exp(-np.abs(x))) + np.maximum(-x, T(0)))
    if name == "lisht":
        return x * np.tanh(x)
    raise AssertionError(name)


# Which saved quantity the derivative is computed from (impl/dense.jl:83-112,
# traits.jl:59-70): "out" -> derivative needs only the output Ω (rrule branch 1);
# "pre" -> needs the pre-activation x as well (branch 2).
ACT_NEEDS = {
    "identity": "none", "relu": "out", "tanh": "out", "sigmoid": "out",
    "swish": "pre", "gelu": "pre", "softplus": "pre", "logsigmoid": "pre", "lisht": "pre",
}


def act_derivative(name: str, out: np.ndarray, x: np.ndarray | None) -> np.ndarray:
    """dσ(Ω, x) as LuxLib multiplies Δ by (impl/activation.jl:139-154).

    `out` = Ω = σ(x).  `x` may be None for activations whose derivative needs only Ω
    (the reference passes NotaNumber() there).
    """
    name = canonical_act(name)
    out = np.asarray(out)
    T = out.dtype.type
    if name == "identity":
        return np.ones_like(out)
    if name == "relu":
        return (out > 0).astype(out.dtype)
    if name == "tanh":
        return T(1) - out * out
    if name == "sigmoid":
        return out * (T(1) - out)
    if x is None:
        raise ValueError(f"activation {name} needs the pre-activation for its derivative")
    x = np.asarray(x)
    if name == "swish":
        return out + _sigmoid(x) * (T(1) - out)
    if name == "gelu":
        x2 = x * x
        u = T(_SQRT_2_OVER_PI) * (x + T(_GELU_C) * x2 * x)
        t = np.tanh(u)
        du = T(_SQRT_2_OVER_PI) * (T(1) + T(3 * _GELU_C) * x2)
        return T(0.5) * (T(1) + t) + T(0.5) * x * (T(1) - t * t) * du
    if name == "softplus":
        return _sigmoid(x)
    if name == "logsigmoid":
        return _sigmoid(-x)
    if name == "lisht":
        t = np.tanh(x)
        return t + x * (T(1) - t * t)
    raise AssertionError(name)


def grad_activation(delta, out, name, x=None):
    """∇activation(Δ, out, act, x) = Δ .* only_derivative(out, act, x) (impl/activation.jl:135-141)."""
    if canonical_act(name) == "identity":
        return np.asarray(delta).copy()
    return np.asarray(delta) * act_derivative(name, out, x)


# --------------------------------------------------------------------------------------
# bias_activation  (api/bias_activation.jl:16-45, impl/bias_activation.jl:2-62,
# impl/common_ops.jl:1-38)
# --------------------------------------------------------------------------------------
def _bias_shape(x: np.ndarray, n: int):
    # reshaped_bias_dims (impl/common_ops.jl:1-3): bias lies along dim N-1 (vectors: dim 1)
    if x.ndim == 1:
        return (n,)
    return tuple(n if i == x.ndim - 2 else 1 for i in range(x.ndim))


def bias_add(x, bias):
    x = np.asarray(x)
    if bias is None:
        return x.copy()
    bias = np.asarray(bias)
    want = x.shape[0] if x.ndim == 1 else x.shape[-2]
    if bias.ndim != 1 or bias.shape[0] != want:
        # api/bias_activation.jl:38-45 (@assert length(bias) == size(x, N-1))
        raise AssertionError("length(bias) must equal size(x, ndims(x)-1)")
    return x + bias.reshape(_bias_shape(x, bias.shape[0]))


def bias_activation(act: str, x, bias):
    """y[i,c,n] = σ(x[i,c,n] + b[c])  (impl/bias_activation.jl:207-220,253-270)."""
    return act_value(act, bias_add(x, bias))


def grad_bias_add(bias, delta):
    """∂b = sum of Δ over every dim except N-1 (impl/common_ops.jl:25-38)."""
    if bias is None:
        return None
    delta = np.asarray(delta)
    if delta.ndim == 1:
        return delta.copy()
    axes = tuple(i for i in range(delta.ndim) if i != delta.ndim - 2)
    return delta.sum(axis=axes)


def bias_activation_pullback(act: str, x, bias, delta):
    """rrule of bias_activation (impl/bias_activation.jl:64-104): returns (y, ∂x, ∂b)."""
    pre = bias_add(x, bias)
    y = act_value(act, pre)
    dx = grad_activation(delta, y, act, pre)
    return y, dx, grad_bias_add(bias, dx)


# --------------------------------------------------------------------------------------
# fused_dense_bias_activation  (api/dense.jl:33-37, impl/dense.jl:4-113,290-291,
# impl/matmul.jl:2-129)
# --------------------------------------------------------------------------------------
class DimensionMismatch(ValueError):
    """Mirror of Julia's DimensionMismatch (impl/matmul.jl:21-34)."""


def matmuladd(W, x, b):
    W, x = np.asarray(W), np.asarray(x)
    if W.shape[1] != x.shape[0]:
        raise DimensionMismatch(f"A has shape {W.shape} but B has shape {x.shape}")
    if b is not None and np.asarray(b).shape[0] != W.shape[0]:
        raise DimensionMismatch("bias length does not match rows of A")
    y = W @ x
    if b is not None:
        y = y + np.asarray(b)[:, None]
    return y


def fused_dense_bias_activation(act: str, W, x, b):
    """y = σ.(W*x .+ b), W (out x in), x (in x batch)  (impl/dense.jl:29-57)."""
    return act_value(act, matmuladd(W, x, b))


def fused_dense_pullback(act: str, W, x, b, delta):
    """rrule (impl/dense.jl:71-113) + ∇matmul_bias (:290-291): (y, ∂W, ∂x, ∂b)."""
    pre = matmuladd(W, x, b)
    y = act_value(act, pre)
    dz = grad_activation(delta, y, act, pre)
    db = None if b is None else dz.sum(axis=1)
    dW = dz @ np.asarray(x).T
    dx = np.asarray(W).T @ dz
    return y, dW, dx, db


# --------------------------------------------------------------------------------------
# mean_var and its rrule (impl/common_ops.jl:40-61)
# --------------------------------------------------------------------------------------
def mean_var(x, axes, corrected=False):
    x = np.asarray(x)
    mu = x.mean(axis=axes, keepdims=True)
    n = int(np.prod([x.shape[a] for a in axes]))
    var = ((x - mu) ** 2).sum(axis=axes, keepdims=True) / x.dtype.type(n - (1 if corrected else 0))
    return mu, var


def mean_var_pullback(x, mu, axes, dmu, dvar, corrected=False):
    """∂x = ∂μ/n + (2/(n - corrected)) ∂σ² (x - μ)  (impl/common_ops.jl:45-61)."""
    x = np.asarray(x)
    T = x.dtype.type
    n = int(np.prod([x.shape[a] for a in axes]))
    return dmu / T(n) + T(2.0 / (n - (1 if corrected else 0))) * dvar * (x - mu)


def default_epsilon(dtype) -> float:
    """eps(T)^(5/7)  (utils.jl:130)."""
    return float(np.finfo(dtype).eps) ** (5.0 / 7.0)


# --------------------------------------------------------------------------------------
# batchnorm  (api/batchnorm.jl:31-55, impl/batchnorm.jl:29-147, impl/normalization.jl:20-143)
# --------------------------------------------------------------------------------------
def _bn_axes(x):
    # batchnorm_reduce_dims (impl/batchnorm.jl:4-6): all dims except N-1
    return tuple(i for i in range(x.ndim) if i != x.ndim - 2)


def _chan_shape(x, C):
    return tuple(C if i == x.ndim - 2 else 1 for i in range(x.ndim))


def batchnorm(x, gamma, beta, rmean, rvar, training: bool, act: str = "identity",
              momentum=0.1, eps=None):
    """Returns (y, running_mean', running_var')  (impl/batchnorm.jl:29-49).

    training: batch statistics (biased variance); running stats, when given, become
    (1-m)·r + m·μ and (1-m)·r + m·n/(n-1)·σ² (impl/normalization.jl:95-110, 20-37).
    inference: the running stats are the statistics (batch statistics when none are given,
    impl/normalization.jl:116-127).
    """
    x = np.asarray(x)
    T = x.dtype.type
    if eps is None:
        eps = default_epsilon(x.dtype)
    C = x.shape[-2]
    axes = _bn_axes(x)
    cs = _chan_shape(x, C)
    if training or rmean is None:
        mu, var = mean_var(x, axes, corrected=False)
        if training and rmean is not None:
            n = T(np.prod([x.shape[a] for a in axes]))
            m = T(momentum)
            rmean_new = (T(1) - m) * np.asarray(rmean) + m * mu.reshape(C)
            rvar_new = (T(1) - m) * np.asarray(rvar) + (m * n / (n - T(1))) * var.reshape(C)
        else:
            rmean_new, rvar_new = rmean, rvar
    else:
        mu, var = np.asarray(rmean).reshape(cs), np.asarray(rvar).reshape(cs)
        rmean_new, rvar_new = rmean, rvar
    y = _affine_normalize(act, x, mu, var, gamma, beta, T(eps), cs)
    return y, rmean_new, rvar_new


def _affine_normalize(act, x, mu, var, gamma, beta, eps, pshape):
    """act(x·γ′ + β′), γ′ = γ/√(σ²+ϵ), β′ = β - μγ′  (impl/normalization.jl:3-17,
    impl/batchnorm.jl:149-176)."""
    T = x.dtype.type
    if gamma is None:
        gp = T(1) / np.sqrt(var + eps)
        bp = -mu * gp
    else:
        gp = np.asarray(gamma).reshape(pshape) / np.sqrt(var + eps)
        bp = np.asarray(beta).reshape(pshape) - mu * gp
    return act_value(act, x * gp + bp)


def batchnorm_pullback(x, gamma, beta, act: str, eps, delta, *, training=True,
                       rmean=None, rvar=None):
    """Pullback of batchnorm w.r.t. (x, γ, β): (∂x, ∂γ, ∂β).

    Follows ∇batchnorm_affine_normalize_cpu! (impl/batchnorm.jl:517-570) completed, in
    training mode, by the mean_var rrule (impl/common_ops.jl:45-61).  In inference mode the
    statistics are constants (impl/normalization.jl:39,114 are non-differentiable) so only
    the ∂x̃ = ∂y·γ′ term survives.
    """
    x = np.asarray(x)
    T = x.dtype.type
    C = x.shape[-2]
    axes = _bn_axes(x)
    cs = _chan_shape(x, C)
    if training or rmean is None:
        mu, var = mean_var(x, axes)
        stats_depend_on_x = True
    else:
        mu, var = np.asarray(rmean).reshape(cs), np.asarray(rvar).reshape(cs)
        stats_depend_on_x = False
    eps = T(eps)
    idenom = T(1) / np.sqrt(var + eps)
    g = np.ones(cs, x.dtype) if gamma is None else np.asarray(gamma).reshape(cs)
    b = np.zeros(cs, x.dtype) if beta is None else np.asarray(beta).reshape(cs)
    gp = g * idenom
    pre = x * gp + (b - mu * gp)
    out = act_value(act, pre)
    dy = grad_activation(delta, out, act, pre)
    xmu = x - mu
    dbeta = dy.sum(axis=axes)
    dgamma = (dy * xmu * idenom).sum(axis=axes)
    dxt = dy * gp
    dx = dxt
    if stats_depend_on_x:
        dmu = -dxt.sum(axis=axes, keepdims=True)
        dvar = -(dxt * xmu).sum(axis=axes, keepdims=True) * T(0.5) * idenom * idenom
        dx = dxt + mean_var_pullback(x, mu, axes, dmu, dvar)
    return dx, (None if gamma is None else dgamma), (None if beta is None else dbeta)


# --------------------------------------------------------------------------------------
# groupnorm  (api/groupnorm.jl:26-64, impl/groupnorm.jl:5-85, 477-533)
# --------------------------------------------------------------------------------------
class ArgumentError(ValueError):
    """Mirror of Julia's ArgumentError (api/groupnorm.jl:40-64)."""


def _gn_view(x, groups):
    # x (..., C, N) -> (..., C/G, G, N) in *Julia column-major* order: channel c (0-based)
    # maps to j = c mod C/G, k = c div C/G (impl/groupnorm.jl:13-15).  With numpy logical
    # indices that is x5[..., j, k, n] = x[..., k*Cg + j, n].
    C, N = x.shape[-2], x.shape[-1]
    Cg = C // groups
    lead = x.shape[:-2]
    x5 = x.reshape(lead + (groups, Cg, N))          # [..., k, j, n]
    return np.swapaxes(x5, -3, -2), Cg              # [..., j, k, n]


def groupnorm(x, gamma, beta, groups: int, act: str = "identity", eps=None):
    x = np.asarray(x)
    T = x.dtype.type
    C = x.shape[-2]
    if gamma is not None and (len(gamma) != len(beta) or len(beta) != C):
        raise ArgumentError("Length of `scale` and `bias` must be equal to the number of channels")
    if C % groups != 0:
        raise ArgumentError(f"Number of channels {C} must be divisible by the number of groups {groups}")
    if eps is None:
        eps = default_epsilon(x.dtype)
    xv, Cg = _gn_view(x, groups)
    axes = tuple(range(xv.ndim - 2))                # all but (G, N)  (impl/groupnorm.jl:1)
    mu, var = mean_var(xv, axes)
    pshape = (1,) * (xv.ndim - 3) + (Cg, groups, 1)
    gv = None if gamma is None else np.asarray(gamma).reshape(groups, Cg).T.reshape(pshape)
    bv = None if beta is None else np.asarray(beta).reshape(groups, Cg).T.reshape(pshape)
    yv = _affine_normalize_arr(act, xv, mu, var, gv, bv, T(eps))
    return np.swapaxes(yv, -3, -2).reshape(x.shape)


def _affine_normalize_arr(act, x, mu, var, g, b, eps):
    T = x.dtype.type
    if g is None:
        gp = T(1) / np.sqrt(var + eps)
        bp = -mu * gp
    else:
        gp = g / np.sqrt(var + eps)
        bp = b - mu * gp
    return act_value(act, x * gp + bp)


def groupnorm_pullback(x, gamma, beta, groups: int, act: str, eps, delta):
    """(∂x, ∂γ, ∂β): ∇groupnorm_affine_normalize_cpu! (impl/groupnorm.jl:477-533) completed
    by the mean_var rrule with n = W·H·C/G."""
    x = np.asarray(x)
    T = x.dtype.type
    C = x.shape[-2]
    xv, Cg = _gn_view(x, groups)
    dv, _ = _gn_view(np.asarray(delta), groups)
    axes = tuple(range(xv.ndim - 2))
    mu, var = mean_var(xv, axes)
    eps = T(eps)
    idenom = T(1) / np.sqrt(var + eps)
    pshape = (1,) * (xv.ndim - 3) + (Cg, groups, 1)
    g = np.ones(pshape, x.dtype) if gamma is None else np.asarray(gamma).reshape(groups, Cg).T.reshape(pshape)
    b = np.zeros(pshape, x.dtype) if beta is None else np.asarray(beta).reshape(groups, Cg).T.reshape(pshape)
    gp = g * idenom
    pre = xv * gp + (b - mu * gp)
    out = act_value(act, pre)
    dy = grad_activation(dv, out, act, pre)
    xmu = xv - mu
    par_axes = tuple(range(xv.ndim - 3)) + (xv.ndim - 1,)       # over (i..., n)
    dbeta = dy.sum(axis=par_axes).T.reshape(C)                   # [j,k] -> c = k*Cg + j
    dgamma = (dy * xmu * idenom).sum(axis=par_axes).T.reshape(C)
    dxt = dy * gp
    dmu = -dxt.sum(axis=axes, keepdims=True)
    dvar = -(dxt * xmu).sum(axis=axes, keepdims=True) * T(0.5) * idenom * idenom
    dxv = dxt + mean_var_pullback(xv, mu, axes, dmu, dvar)
    dx = np.swapaxes(dxv, -3, -2).reshape(x.shape)
    return dx, (None if gamma is None else dgamma), (None if beta is None else dbeta)


# --------------------------------------------------------------------------------------
# instancenorm  (api/instancenorm.jl:33-80, impl/normalization.jl:143-208: the generic
# `normalization` with reduce dims 1..N-2)
# --------------------------------------------------------------------------------------
def instancenorm(x, gamma, beta, rmean, rvar, training: bool, act: str = "identity", momentum=0.1, eps=None):
    """Returns (y, running_mean', running_var').  Statistics per (channel, sample) over the
    leading dims (biased variance); with running statistics in training mode the per-sample
    statistics are averaged over the batch first (impl/normalization.jl:104-107) and the
    variance is corrected by m/(m-1), m = number of reduced elements (:108-109).  Inference
    with running statistics uses them for every sample (:122-127)."""
    x = np.asarray(x)
    assert x.ndim > 2, "`ndims(x)` must be at least > 2."       # api/instancenorm.jl:75-78
    T = x.dtype.type
    if eps is None:
        eps = default_epsilon(x.dtype)
    C = x.shape[-2]
    axes = tuple(range(x.ndim - 2))
    cs = _chan_shape(x, C)
    rmean_new, rvar_new = rmean, rvar
    if training or rmean is None:
        mu, var = mean_var(x, axes, corrected=False)
        if training and rmean is not None:
            m = T(np.prod([x.shape[a] for a in axes]))
            mom = T(momentum)
            rmean_new = (T(1) - mom) * np.asarray(rmean) + mom * mu.mean(axis=-1).reshape(C)
            rvar_new = (T(1) - mom) * np.asarray(rvar) + (mom * m / (m - T(1))) * var.mean(axis=-1).reshape(C)
    else:
        mu, var = np.asarray(rmean).reshape(cs), np.asarray(rvar).reshape(cs)
    y = _affine_normalize(act, x, mu, var, gamma, beta, T(eps), cs)
    return y, rmean_new, rvar_new


def instancenorm_pullback(x, gamma, beta, act: str, eps, delta, *, training=True, rmean=None, rvar=None):
    """(∂x, ∂γ, ∂β) of instancenorm: AD of the generic `normalization` (affine_normalize,
    impl/normalization.jl:3-17, and the mean_var rrule, impl/common_ops.jl:45-61, with
    n = the number of reduced elements); running statistics are constants."""
    x = np.asarray(x)
    T = x.dtype.type
    C = x.shape[-2]
    axes = tuple(range(x.ndim - 2))
    par_axes = axes + (x.ndim - 1,)
    cs = _chan_shape(x, C)
    from_x = training or rmean is None
    if from_x:
        mu, var = mean_var(x, axes)
    else:
        mu, var = np.asarray(rmean).reshape(cs), np.asarray(rvar).reshape(cs)
    eps = T(eps)
    idenom = T(1) / np.sqrt(var + eps)
    g = np.ones(cs, x.dtype) if gamma is None else np.asarray(gamma).reshape(cs)
    b = np.zeros(cs, x.dtype) if beta is None else np.asarray(beta).reshape(cs)
    gp = g * idenom
    pre = x * gp + (b - mu * gp)
    dy = grad_activation(delta, act_value(act, pre), act, pre)
    xmu = x - mu
    dbeta = dy.sum(axis=par_axes)
    dgamma = (dy * xmu * idenom).sum(axis=par_axes)
    dx = dy * gp
    if from_x:
        dmu = -dx.sum(axis=axes, keepdims=True)
        dvar = -(dx * xmu).sum(axis=axes, keepdims=True) * T(0.5) * idenom * idenom
        dx = dx + mean_var_pullback(x, mu, axes, dmu, dvar)
    return dx, (None if gamma is None else dgamma), (None if beta is None else dbeta)


# --------------------------------------------------------------------------------------
# batched_matmul  (api/batched_mul.jl, impl/batched_mul.jl:2-58, 171-334) with the default
# (trailing) batching dims
# --------------------------------------------------------------------------------------
def _bmm_operands(x, y, lhs_contracting_dim, rhs_contracting_dim):
    x, y = np.asarray(x), np.asarray(y)
    if x.ndim == 2 and y.ndim >= 3:
        x = x.reshape(x.shape + (1,) * (y.ndim - 2))        # expand_batchdim
    if y.ndim == 2 and x.ndim >= 3:
        y = y.reshape(y.shape + (1,) * (x.ndim - 2))
    if x.ndim < 3 or x.ndim != y.ndim:
        raise ArgumentError("N must be at least 3")
    for a, b in zip(x.shape[2:], y.shape[2:]):
        if a != b and a != 1 and b != 1:
            raise DimensionMismatch("Batching dimensions mismatch")
    xo = x if lhs_contracting_dim == 2 else np.swapaxes(x, 0, 1)      # (M, K, b...)
    yo = y if rhs_contracting_dim == 1 else np.swapaxes(y, 0, 1)      # (K, N, b...)
    if xo.shape[1] != yo.shape[0]:
        raise DimensionMismatch("inconsistent for batched_matmul")
    return x, y, xo, yo


def batched_matmul(x, y, lhs_contracting_dim=2, rhs_contracting_dim=1):
    """z[:, :, b...] = op(x[:, :, b...]) op(y[:, :, b...]); batch dims of extent 1 repeat
    (impl/batched_mul.jl:76-110, 255-268)."""
    _, _, xo, yo = _bmm_operands(x, y, lhs_contracting_dim, rhs_contracting_dim)
    return np.einsum("mk...,kn...->mn...", xo, yo)


def batched_matmul_pullback(x, y, delta, lhs_contracting_dim=2, rhs_contracting_dim=1):
    """(∂x, ∂y): ∂x = Δ ⊠ adjoint(y), ∂y = adjoint(x) ⊠ Δ, summed over the batch dims along which
    the operand was repeated (impl/batched_mul.jl:320-334), in the operand's own layout."""
    x0, y0 = np.asarray(x), np.asarray(y)
    x, y, xo, yo = _bmm_operands(x, y, lhs_contracting_dim, rhs_contracting_dim)
    delta = np.asarray(delta)
    dxo = np.einsum("mn...,kn...->mk...", delta, np.broadcast_to(yo, yo.shape[:2] + delta.shape[2:]))
    dyo = np.einsum("mk...,mn...->kn...", np.broadcast_to(xo, xo.shape[:2] + delta.shape[2:]), delta)
    dx = dxo if lhs_contracting_dim == 2 else np.swapaxes(dxo, 0, 1)
    dy = dyo if rhs_contracting_dim == 1 else np.swapaxes(dyo, 0, 1)
    for ax in range(2, delta.ndim):
        if x.shape[ax] == 1 and delta.shape[ax] != 1:
            dx = dx.sum(axis=ax, keepdims=True)
        if y.shape[ax] == 1 and delta.shape[ax] != 1:
            dy = dy.sum(axis=ax, keepdims=True)
    return dx.reshape(x0.shape), dy.reshape(y0.shape)


def _general_bmm_axes(ndim, contracting_dim, batching_dims):
    """0-based (non-contracting axis, contracting axis, batching axes) for 1-based dims
    (get_non_contracting_dim, impl/batched_mul.jl)."""
    if batching_dims is None:
        batching_dims = tuple(range(3, ndim + 1))
    rest = [d for d in range(1, ndim + 1) if d != contracting_dim and d not in batching_dims]
    assert len(rest) == 1 and len(batching_dims) == ndim - 2, "one contracting, one free and N-2 batching dims"
    return rest[0] - 1, contracting_dim - 1, tuple(d - 1 for d in batching_dims)


def batched_matmul_general(x, y, lhs_contracting_dim=2, rhs_contracting_dim=1, lhs_batching_dims=None, rhs_batching_dims=None):
    """batched_matmul with arbitrary batching dims (api/batched_mul.jl, impl/batched_mul.jl:2-58): the
    operands are permuted to (free, contracting, batch...) / (contracting, free, batch...), batch dims of
    extent 1 repeat, and z = (free_x, free_y, batch...)."""
    x, y = np.asarray(x), np.asarray(y)
    fx, cx, bx = _general_bmm_axes(x.ndim, lhs_contracting_dim, lhs_batching_dims)
    fy, cy, by = _general_bmm_axes(y.ndim, rhs_contracting_dim, rhs_batching_dims)
    xp, yp = np.transpose(x, (fx, cx) + bx), np.transpose(y, (cy, fy) + by)
    for a, b in zip(xp.shape[2:], yp.shape[2:]):
        if a != b and a != 1 and b != 1:
            raise DimensionMismatch("Batching dimensions mismatch")
    return np.einsum("mk...,kn...->mn...", xp, yp)


def batched_matmul_general_pullback(x, y, delta, lhs_contracting_dim=2, rhs_contracting_dim=1, lhs_batching_dims=None,
                                    rhs_batching_dims=None):
    """(∂x, ∂y) in the operands' own layouts: the rrule of the permuted product (impl/batched_mul.jl:320-334),
    summed over repeated batch dims, taken back through the permutation."""
    x, y, delta = np.asarray(x), np.asarray(y), np.asarray(delta)
    fx, cx, bx = _general_bmm_axes(x.ndim, lhs_contracting_dim, lhs_batching_dims)
    fy, cy, by = _general_bmm_axes(y.ndim, rhs_contracting_dim, rhs_batching_dims)
    px, py = (fx, cx) + bx, (cy, fy) + by
    xp, yp = np.transpose(x, px), np.transpose(y, py)
    full = delta.shape[2:]
    dxp = np.einsum("mn...,kn...->mk...", delta, np.broadcast_to(yp, yp.shape[:2] + full))
    dyp = np.einsum("mk...,mn...->kn...", np.broadcast_to(xp, xp.shape[:2] + full), delta)
    for ax in range(2, delta.ndim):
        if xp.shape[ax] == 1 and delta.shape[ax] != 1:
            dxp = dxp.sum(axis=ax, keepdims=True)
        if yp.shape[ax] == 1 and delta.shape[ax] != 1:
            dyp = dyp.sum(axis=ax, keepdims=True)
    return np.transpose(dxp, np.argsort(px)), np.transpose(dyp, np.argsort(py))


# --------------------------------------------------------------------------------------
# scaled_dot_product_attention  (api/attention.jl, impl/attention.jl:5-134), head_dim = 1
# --------------------------------------------------------------------------------------
def _attn_canonical(a, token_dim):
    """[E, heads, tokens, B] view (B = the flattened trailing dims) of an operand whose token dim is 2 or 3."""
    a = np.asarray(a)
    a4 = a.reshape(a.shape[:3] + (-1,))
    return a4 if token_dim == 3 else np.swapaxes(a4, 1, 2)


def scaled_dot_product_attention(q, k, v, token_dim=3, scale=None, mask=None, is_causal=None, bias=None, weights=None):
    """Returns (output [Ev, H, L, B...], weights [S, L, H, B...]).
    `weights` (optional): the weights as an earlier call stored them (bf16 storage: rounded); the output is then
    the product of v with these, which is what the reference's second batched product computes from its stored
    softmax result (impl/attention.jl:107-117).
    logits[s,l,h,b] = (1/scale) Σ_d k[d,h,s,b] q[d,h,l,b] (+ bias), -inf where the mask is false
    (impl/attention.jl:90-104, 119-128); weights = softmax over s; output[e,h,l,b] =
    Σ_s v[e,h,s,b] weights[s,l,h,b] (:107-117).  Fewer key/value heads than query heads: each is
    used by H/G consecutive query heads (repeat_inner_gqa, :1-3, 44-48).  scale defaults to
    sqrt(E) (:50-51).  is_causal keeps s <= l (make_causal_mask: triu!, :130-134)."""
    assert not (mask is not None and is_causal is not None), "`mask` and `is_causal` cannot both be specified"
    tail = np.asarray(q).shape[3:]
    q4, k4, v4 = (_attn_canonical(a, token_dim) for a in (q, k, v))
    E, H, L, B = q4.shape
    G, S = k4.shape[1], k4.shape[2]
    assert H % G == 0, "num_heads must be divisible by num_kv_groups"
    k4, v4 = np.repeat(k4, H // G, axis=1), np.repeat(v4, H // G, axis=1)
    T = q4.dtype.type
    inv = T(1) / (np.sqrt(T(E)) if scale is None else T(scale))
    logits = np.einsum("dhsb,dhlb->slhb", k4, q4 * inv)
    if bias is not None:
        logits = logits + np.asarray(bias).reshape(np.asarray(bias).shape[:3] + (-1,))
    if is_causal:
        mask = np.triu(np.ones((S, L), bool))
    if mask is not None:
        m = np.asarray(mask, bool)
        m = m.reshape(m.shape + (1,) * (4 - m.ndim)) if m.ndim < 4 else m.reshape(m.shape[:3] + (-1,))
        logits = np.where(m, logits, -np.inf)
    z = logits - logits.max(axis=0, keepdims=True)
    w = np.exp(z)
    w = w / w.sum(axis=0, keepdims=True)
    if weights is not None:
        w = np.asarray(weights, dtype=q4.dtype).reshape(w.shape)
    out = np.einsum("ehsb,slhb->ehlb", v4, w)
    return out.reshape(out.shape[:3] + tail), w.reshape(w.shape[:3] + tail)


def scaled_dot_product_attention_pullback(q, k, v, d_out, token_dim=3, scale=None, mask=None, is_causal=None, bias=None,
                                          weights=None, stored=None):
    """(∂q, ∂k, ∂v) for a cotangent of the output only: the chain of the batched_matmul rrules
    (impl/batched_mul.jl:320-334), the softmax rule dS = W ∘ (dW - Σ_s dW ∘ W), the scale, and the
    sum over the query heads that share a key/value head.
    The reference's pullbacks work on the arrays that the forward pass stored: `weights` (optional)
    are the attention weights as the forward pass returned them (in bf16 storage: rounded), used in
    place of the exact ones; `stored` (optional) is applied to the arrays of the storage type that the
    pullback itself passes from one rule to the next: the cotangent of the logits (softmax rule ->
    the two products) and the per-query-head gradients of k and v (products -> the sum over the heads
    of a key/value group, the pullback of repeat_inner_gqa), e.g. `round_to_bf16`."""
    q0, k0, v0 = np.asarray(q), np.asarray(k), np.asarray(v)
    q4, k4, v4 = (_attn_canonical(a, token_dim) for a in (q0, k0, v0))
    E, H, L, B = q4.shape
    G, S = k4.shape[1], k4.shape[2]
    r = H // G
    kr, vr = np.repeat(k4, r, axis=1), np.repeat(v4, r, axis=1)
    T = q4.dtype.type
    inv = T(1) / (np.sqrt(T(E)) if scale is None else T(scale))
    if weights is None:
        _, w = scaled_dot_product_attention(q, k, v, token_dim, scale, mask, is_causal, bias)
    else:
        w = np.asarray(weights, dtype=q4.dtype)
    w = w.reshape(w.shape[:3] + (-1,))
    do = np.asarray(d_out).reshape(np.asarray(d_out).shape[:3] + (-1,))       # [Ev, H, L, B]
    dw = np.einsum("ehsb,ehlb->slhb", vr, do)
    dvr = np.einsum("ehlb,slhb->ehsb", do, w)
    ds = w * (dw - (dw * w).sum(axis=0, keepdims=True)) * inv
    if stored is not None:
        ds = np.asarray(stored(ds), dtype=q4.dtype)
    dq4 = np.einsum("dhsb,slhb->dhlb", kr, ds)
    dkr = np.einsum("dhlb,slhb->dhsb", q4, ds)
    if stored is not None:
        dkr, dvr = np.asarray(stored(dkr), dtype=q4.dtype), np.asarray(stored(dvr), dtype=q4.dtype)
    dk4 = dkr.reshape(E, G, r, S, B).sum(axis=2)
    dv4 = dvr.reshape(v4.shape[0], G, r, S, B).sum(axis=2)
    back = (lambda a, like: (a if token_dim == 3 else np.swapaxes(a, 1, 2)).reshape(like.shape))
    return back(dq4, q0), back(dk4, k0), back(dv4, v0)


# --------------------------------------------------------------------------------------
# dropout / alpha_dropout  (api/dropout.jl, impl/dropout.jl).  The reference draws its noise
# with `rand!(rng, y)` from Julia's generators, whose streams cannot be reproduced without
# Julia; the arithmetic that follows the noise is restated here, and the noise itself comes
# from Philox4x32-10 (Salmon et al., SC'11; the Random123 library's known-answer vectors pin it).
# --------------------------------------------------------------------------------------
_PHILOX_M0, _PHILOX_M1 = 0xD2511F53, 0xCD9E8D57
_PHILOX_W0, _PHILOX_W1 = 0x9E3779B9, 0xBB67AE85


def philox4x32_10(counter, key):
    """counter: (..., 4) uint32, key: (2,) uint32 -> (..., 4) uint32."""
    c = [np.asarray(counter)[..., i].astype(np.uint64) for i in range(4)]
    k0, k1 = int(key[0]), int(key[1])
    mask = np.uint64(0xFFFFFFFF)
    for _ in range(10):
        p0 = np.uint64(_PHILOX_M0) * c[0]
        p1 = np.uint64(_PHILOX_M1) * c[2]
        hi0, lo0, hi1, lo1 = p0 >> np.uint64(32), p0 & mask, p1 >> np.uint64(32), p1 & mask
        c = [hi1 ^ c[1] ^ np.uint64(k0), lo1, hi0 ^ c[3] ^ np.uint64(k1), lo0]
        k0, k1 = (k0 + _PHILOX_W0) & 0xFFFFFFFF, (k1 + _PHILOX_W1) & 0xFFFFFFFF
    return np.stack(c, axis=-1).astype(np.uint32)


def rand_uniform(n, seed, offset, bf16=False):
    """The first n values of the stream (seed, offset): element e = lane e % 4 of the block with
    counter (offset + e // 4, 0) under the key (seed mod 2^32, seed div 2^32); a word u becomes
    (u >> 8) 2^-24, or (u >> 24) 2^-8 for bf16 storage.  float32 values in [0, 1)."""
    nb = (n + 3) // 4
    ctr = (np.arange(nb, dtype=np.uint64) + np.uint64(offset))
    counter = np.zeros((nb, 4), np.uint32)
    counter[:, 0] = (ctr & np.uint64(0xFFFFFFFF)).astype(np.uint32)
    counter[:, 1] = (ctr >> np.uint64(32)).astype(np.uint32)
    u = philox4x32_10(counter, (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF)).reshape(-1)[:n]
    if bf16:
        return (u >> np.uint32(24)).astype(np.float32) * np.float32(2.0 ** -8)
    return (u >> np.uint32(8)).astype(np.float32) * np.float32(2.0 ** -24)


def dropout_shape(x_shape, dims):
    """impl/dropout.jl:74-78; dims: None (Julia's `:`) or 1-based dims that keep their extent."""
    if dims is None:
        return tuple(x_shape)
    return tuple(s if (i + 1) in dims else 1 for i, s in enumerate(x_shape))


def generate_dropout_mask(noise, p, invp):
    """(noise > T(p)) * T(invp) in noise's dtype T (impl/dropout.jl:200-218)."""
    T = noise.dtype.type
    return (noise > T(p)).astype(noise.dtype) * T(invp)


def dropout(noise, x, p, training, invp, mask=None, update_mask=True):
    """(y, mask) of api/dropout.jl:40-69 / impl/dropout.jl:3-47 given the uniform noise (an array
    of dropout_shape(x, dims), column-major order of draws) that `rand!` would have produced.
    Not training: (x, x) without a mask argument (the returned mask is meaningless), (x, mask)
    with one."""
    if mask is not None and not update_mask:
        if not training:
            return x, mask
        assert all(m in (1, s) for m, s in zip(mask.shape, x.shape)) and mask.ndim == x.ndim, \
            "`mask` is not of the same size as `LuxLib.dropout_shape(x, dims)`."
        return x * mask, mask
    if not training:
        return x, (x if mask is None else mask)
    m = generate_dropout_mask(noise, p, invp)
    return x * m, m


def alpha_dropout_coefficients(p):
    """impl/dropout.jl:57-62."""
    alpha = -1.7580993408473766
    A = 1.0 / math.sqrt((1 - p) * (1 + p * alpha ** 2))
    return alpha, A, -A * alpha * p


def alpha_dropout(noise, p, x, alpha, A, B):
    """muladd(ifelse(noise > p, x, α), A, B) with α, A, B in x's dtype (impl/dropout.jl:84-89)."""
    T = x.dtype.type
    return np.where(noise > p, x, T(alpha)) * T(A) + T(B)


def alpha_dropout_pullback(noise, p, delta, A):
    """∂x = Δ · (noise > p) · A (impl/dropout.jl:137-150)."""
    return delta * (noise > p) * delta.dtype.type(A)


# --------------------------------------------------------------------------------------
# layernorm  (api/layernorm.jl:32-43, impl/layernorm.jl:3-51, impl/normalization.jl:3-17)
# --------------------------------------------------------------------------------------
def layernorm(x, gamma, beta, act: str = "identity", dims=None, eps=None):
    """`dims` are 0-based numpy axes here (Julia's 1:(N-1) default = all but the last).
    γ, β must broadcast against x (the reference requires ndims(γ) == ndims(x) when dims is
    given, impl/layernorm.jl:47-51)."""
    x = np.asarray(x)
    T = x.dtype.type
    if dims is None:
        dims = tuple(range(x.ndim - 1))
    if eps is None:
        eps = default_epsilon(x.dtype)
    mu, var = mean_var(x, tuple(dims))
    g = None if gamma is None else np.asarray(gamma)
    b = None if beta is None else np.asarray(beta)
    return _affine_normalize_arr(act, x, mu, var, g, b, T(eps))


def _sum_to_shape(a, shape):
    axes = tuple(i for i, (s, t) in enumerate(zip(a.shape, shape)) if t == 1 and s != 1)
    return a.sum(axis=axes, keepdims=True).reshape(shape)


def layernorm_pullback(x, gamma, beta, act: str, dims, eps, delta):
    """(∂x, ∂γ, ∂β).  The reference has no custom rrule: AD differentiates the broadcasts
    of impl/normalization.jl:11-17 and chains into the mean_var rrule
    (impl/common_ops.jl:45-61).  This is that chain written out."""
    x = np.asarray(x)
    T = x.dtype.type
    if dims is None:
        dims = tuple(range(x.ndim - 1))
    dims = tuple(dims)
    eps = T(eps)
    mu, var = mean_var(x, dims)
    idenom = T(1) / np.sqrt(var + eps)
    g = np.ones((1,) * x.ndim, x.dtype) if gamma is None else np.asarray(gamma)
    b = np.zeros((1,) * x.ndim, x.dtype) if beta is None else np.asarray(beta)
    gp = g * idenom
    bp = b - mu * gp
    pre = x * gp + bp
    out = act_value(act, pre)
    dy = grad_activation(np.asarray(delta), out, act, pre)
    # y = x·γ′ + β′ ;  γ′ = γ·idenom ; β′ = β - μ γ′
    dgp = _sum_to_shape(dy * x, np.broadcast_shapes(g.shape, idenom.shape))   # ∂γ′ (direct)
    dbp = _sum_to_shape(dy, np.broadcast_shapes(b.shape, mu.shape))           # ∂β′
    dgp = dgp - dbp * mu                                                     # via β′ = β - μγ′
    dmu = _sum_to_shape(-dbp * gp, mu.shape)
    dgamma = _sum_to_shape(dgp * idenom, g.shape)
    dbeta = _sum_to_shape(dbp, b.shape)
    didenom = _sum_to_shape(dgp * g, idenom.shape)
    dvar = didenom * (T(-0.5) * idenom * idenom * idenom)
    dx = dy * gp + mean_var_pullback(x, mu, dims, dmu, dvar)
    return dx, (None if gamma is None else dgamma), (None if beta is None else dbeta)


# --------------------------------------------------------------------------------------
# fused_conv_bias_activation  (api/conv.jl:30-38, impl/conv.jl:138-275).  The arithmetic
# lives in NNlib (third party, compat 0.9.33, not vendored): its published algorithm is the
# direct / im2col convolution over WHCN tensors; orientation and padding order are anchored
# on the reference's own known-answer tests (test/core_layers/conv_tests.jl:54-69,145-190).
# --------------------------------------------------------------------------------------
class ConvDims:
    """The fields of NNlib.DenseConvDims that the path consumes (2 spatial dims)."""

    def __init__(self, x_shape, w_shape, stride=(1, 1), padding=(0, 0, 0, 0), dilation=(1, 1),
                 groups=1, flipkernel=False):
        if isinstance(stride, int):
            stride = (stride, stride)
        if isinstance(dilation, int):
            dilation = (dilation, dilation)
        if isinstance(padding, int):
            padding = (padding,) * 4
        elif len(padding) == 2:
            padding = (padding[0], padding[0], padding[1], padding[1])
        self.x_shape = tuple(x_shape)
        self.w_shape = tuple(w_shape)
        self.stride = tuple(stride)
        self.padding = tuple(padding)          # (w_lo, w_hi, h_lo, h_hi)
        self.dilation = tuple(dilation)
        self.groups = int(groups)
        self.flipkernel = bool(flipkernel)
        W, H, Cin, _ = self.x_shape
        kW, kH, Cin_g, Cout = self.w_shape
        if Cin_g * self.groups != Cin:
            raise DimensionMismatch("input channels do not match weight channels x groups")
        if Cout % self.groups != 0:
            raise DimensionMismatch("output channels must be divisible by groups")

    @classmethod
    def one_spatial_dim(cls, x_shape, w_shape, stride=1, padding=(0, 0), dilation=1, groups=1, flipkernel=False):
        """x (W, C, N), w (K, C/groups, Cout): the problem of height 1 over x (W, 1, C, N) that NNlib
        itself reduces fewer-than-3-d convolutions to (it inserts singleton spatial dims).
        padding = (lo, hi) or one int."""
        if isinstance(padding, int):
            padding = (padding, padding)
        W, C, N = x_shape
        K, Cg, Cout = w_shape
        return cls((W, 1, C, N), (K, 1, Cg, Cout), (int(np.ravel(stride)[0]), 1), tuple(padding) + (0, 0),
                   (int(np.ravel(dilation)[0]), 1), groups, flipkernel)

    @property
    def out_spatial(self):
        W, H = self.x_shape[:2]
        kW, kH = self.w_shape[:2]
        ow = (W + self.padding[0] + self.padding[1] - self.dilation[0] * (kW - 1) - 1) // self.stride[0] + 1
        oh = (H + self.padding[2] + self.padding[3] - self.dilation[1] * (kH - 1) - 1) // self.stride[1] + 1
        return ow, oh

    def y_shape(self, N=None):
        ow, oh = self.out_spatial
        return (ow, oh, self.w_shape[3], self.x_shape[3] if N is None else N)


def _tap_slices(cd: ConvDims, a, b):
    """For kernel tap (a, b) (0-based): the output index range and the matching input
    index range per spatial dim.  Input position for output o and tap a is
    o·stride + koff·dil - pad_lo with koff = K-1-a (true convolution, flipkernel=false)
    or a (cross-correlation, flipkernel=true)."""
    W, H = cd.x_shape[:2]
    kW, kH = cd.w_shape[:2]
    OW, OH = cd.out_spatial
    res = []
    for (L, K, O, s, d, plo, t) in ((W, kW, OW, cd.stride[0], cd.dilation[0], cd.padding[0], a),
                                     (H, kH, OH, cd.stride[1], cd.dilation[1], cd.padding[2], b)):
        koff = t if cd.flipkernel else (K - 1 - t)
        base = koff * d - plo                   # input index at o = 0
        o_lo = 0 if base >= 0 else (-base + s - 1) // s
        o_hi = min(O - 1, (L - 1 - base) // s) if (L - 1 - base) >= 0 else -1
        if o_hi < o_lo:
            res.append(None)
        else:
            res.append((slice(o_lo, o_hi + 1), slice(base + o_lo * s, base + o_hi * s + 1, s)))
    return res


def conv(x, w, cd: ConvDims):
    """NNlib.conv(x, w, cdims) over WHCN (call site impl/conv.jl:39,56)."""
    x, w = np.asarray(x), np.asarray(w)
    N = x.shape[3]
    OW, OH = cd.out_spatial
    kW, kH, Cin_g, Cout = w.shape
    G = cd.groups
    Cout_g = Cout // G
    y = np.zeros((OW, OH, Cout, N), dtype=np.result_type(x, w))
    for a in range(kW):
        for b in range(kH):
            sl = _tap_slices(cd, a, b)
            if sl[0] is None or sl[1] is None:
                continue
            (ow, iw), (oh, ih) = sl
            for g in range(G):
                xs = x[iw, ih, g * Cin_g:(g + 1) * Cin_g, :]            # (ow, oh, Cin_g, N)
                wk = w[a, b, :, g * Cout_g:(g + 1) * Cout_g]            # (Cin_g, Cout_g)
                y[ow, oh, g * Cout_g:(g + 1) * Cout_g, :] += np.einsum("whcn,co->whon", xs, wk)
    return y


def conv_data_grad(dy, w, cd: ConvDims):
    """NNlib.∇conv_data(∂y, w, cdims) (call site impl/conv.jl:130): adjoint of conv in x."""
    dy, w = np.asarray(dy), np.asarray(w)
    kW, kH, Cin_g, Cout = w.shape
    G = cd.groups
    Cout_g = Cout // G
    dx = np.zeros(cd.x_shape[:3] + (dy.shape[3],), dtype=np.result_type(dy, w))
    for a in range(kW):
        for b in range(kH):
            sl = _tap_slices(cd, a, b)
            if sl[0] is None or sl[1] is None:
                continue
            (ow, iw), (oh, ih) = sl
            for g in range(G):
                d = dy[ow, oh, g * Cout_g:(g + 1) * Cout_g, :]
                wk = w[a, b, :, g * Cout_g:(g + 1) * Cout_g]
                dx[iw, ih, g * Cin_g:(g + 1) * Cin_g, :] += np.einsum("whon,co->whcn", d, wk)
    return dx


def conv_filter_grad(x, dy, cd: ConvDims):
    """NNlib.∇conv_filter(x, ∂y, cdims) (call site impl/conv.jl:135): adjoint of conv in w."""
    x, dy = np.asarray(x), np.asarray(dy)
    kW, kH, Cin_g, Cout = cd.w_shape
    G = cd.groups
    Cout_g = Cout // G
    dw = np.zeros(cd.w_shape, dtype=np.result_type(x, dy))
    for a in range(kW):
        for b in range(kH):
            sl = _tap_slices(cd, a, b)
            if sl[0] is None or sl[1] is None:
                continue
            (ow, iw), (oh, ih) = sl
            for g in range(G):
                xs = x[iw, ih, g * Cin_g:(g + 1) * Cin_g, :]
                d = dy[ow, oh, g * Cout_g:(g + 1) * Cout_g, :]
                dw[a, b, :, g * Cout_g:(g + 1) * Cout_g] = np.einsum("whcn,whon->co", xs, d)
    return dw


def fused_conv_bias_activation(act: str, w, x, b, cd: ConvDims):
    """y = σ(conv(x, w) .+ b[cout])  (impl/conv.jl:138-155)."""
    return bias_activation(act, conv(x, w, cd), b)


def fused_conv_pullback(act: str, w, x, b, cd: ConvDims, delta):
    """rrule (impl/conv.jl:204-248) + ∇fused_conv (:261-275): (y, ∂w, ∂x, ∂b)."""
    pre = bias_add(conv(x, w, cd), b)
    y = act_value(act, pre)
    dy = grad_activation(delta, y, act, pre)
    db = grad_bias_add(b, dy)
    return y, conv_filter_grad(x, dy, cd), conv_data_grad(dy, w, cd), db


# --------------------------------------------------------------------------------------
# convolutions with any number of spatial dims (the reference passes 1-, 2- and 3-d problems to the
# same NNlib calls, impl/conv.jl:29-60,128-136): x (S1..Sk, C, N), w (K1..Kk, C/groups, Cout)
# --------------------------------------------------------------------------------------
class ConvDimsND:
    """The fields of NNlib.DenseConvDims for k spatial dims.  padding = (lo1, hi1, lo2, hi2, ...)."""

    def __init__(self, x_shape, w_shape, stride=1, padding=0, dilation=1, groups=1, flipkernel=False):
        k = len(x_shape) - 2
        self.k = k
        self.x_shape, self.w_shape = tuple(x_shape), tuple(w_shape)
        self.stride = (stride,) * k if isinstance(stride, int) else tuple(stride)
        self.dilation = (dilation,) * k if isinstance(dilation, int) else tuple(dilation)
        if isinstance(padding, int):
            padding = (padding,) * (2 * k)
        elif len(padding) == k:
            padding = tuple(p for q in padding for p in (q, q))
        self.padding = tuple(padding)
        self.groups, self.flipkernel = int(groups), bool(flipkernel)
        if self.w_shape[k] * self.groups != self.x_shape[k]:
            raise DimensionMismatch("input channels do not match weight channels x groups")
        if self.w_shape[k + 1] % self.groups != 0:
            raise DimensionMismatch("output channels must be divisible by groups")

    @property
    def out_spatial(self):
        return tuple((self.x_shape[d] + self.padding[2 * d] + self.padding[2 * d + 1]
                      - self.dilation[d] * (self.w_shape[d] - 1) - 1) // self.stride[d] + 1 for d in range(self.k))


def _tap_slices_nd(cd: ConvDimsND, tap):
    """Per spatial dim: (output slice, input slice) for weight index `tap`, or None when the tap
    never meets the input.  Input position = o*stride + koff*dil - pad_lo with koff = K-1-t for true
    convolution and t for flipkernel (the rule of _tap_slices)."""
    res = []
    O = cd.out_spatial
    for d in range(cd.k):
        L, K, s, dl, plo, t = cd.x_shape[d], cd.w_shape[d], cd.stride[d], cd.dilation[d], cd.padding[2 * d], tap[d]
        koff = t if cd.flipkernel else (K - 1 - t)
        base = koff * dl - plo
        o_lo = 0 if base >= 0 else (-base + s - 1) // s
        o_hi = min(O[d] - 1, (L - 1 - base) // s) if (L - 1 - base) >= 0 else -1
        if o_hi < o_lo:
            return None
        res.append((slice(o_lo, o_hi + 1), slice(base + o_lo * s, base + o_hi * s + 1, s)))
    return res


def _conv_nd_terms(cd: ConvDimsND):
    k = cd.k
    Cin_g, Cout = cd.w_shape[k], cd.w_shape[k + 1]
    Cout_g = Cout // cd.groups
    for tap in np.ndindex(*cd.w_shape[:k]):
        sl = _tap_slices_nd(cd, tap)
        if sl is None:
            continue
        osl = tuple(s[0] for s in sl)
        isl = tuple(s[1] for s in sl)
        for g in range(cd.groups):
            yield tap, osl, isl, slice(g * Cin_g, (g + 1) * Cin_g), slice(g * Cout_g, (g + 1) * Cout_g)


def conv_nd(x, w, cd: ConvDimsND):
    x, w = np.asarray(x), np.asarray(w)
    y = np.zeros(cd.out_spatial + (cd.w_shape[-1], x.shape[-1]), dtype=np.result_type(x, w))
    for tap, osl, isl, cs, os_ in _conv_nd_terms(cd):
        y[osl + (os_, slice(None))] += np.einsum("...cn,co->...on", x[isl + (cs, slice(None))], w[tap + (slice(None), os_)])
    return y


def conv_nd_data_grad(dy, w, cd: ConvDimsND):
    dy, w = np.asarray(dy), np.asarray(w)
    dx = np.zeros(cd.x_shape[:-1] + (dy.shape[-1],), dtype=np.result_type(dy, w))
    for tap, osl, isl, cs, os_ in _conv_nd_terms(cd):
        dx[isl + (cs, slice(None))] += np.einsum("...on,co->...cn", dy[osl + (os_, slice(None))], w[tap + (slice(None), os_)])
    return dx


def conv_nd_filter_grad(x, dy, cd: ConvDimsND):
    x, dy = np.asarray(x), np.asarray(dy)
    dw = np.zeros(cd.w_shape, dtype=np.result_type(x, dy))
    for tap, osl, isl, cs, os_ in _conv_nd_terms(cd):
        xs, ds = x[isl + (cs, slice(None))], dy[osl + (os_, slice(None))]
        dw[tap + (slice(None), os_)] = np.einsum("scn,son->co", xs.reshape((-1,) + xs.shape[-2:]), ds.reshape((-1,) + ds.shape[-2:]))
    return dw


def fused_conv_nd_pullback(act: str, w, x, b, cd: ConvDimsND, delta):
    """(y, ∂w, ∂x, ∂b) as fused_conv_pullback, for k spatial dims."""
    pre = bias_add(conv_nd(x, w, cd), b)
    y = act_value(act, pre)
    dy = grad_activation(delta, y, act, pre)
    return y, conv_nd_filter_grad(x, dy, cd), conv_nd_data_grad(dy, w, cd), grad_bias_add(b, dy)


# --------------------------------------------------------------------------------------
# helpers shared by the tests
# --------------------------------------------------------------------------------------
def generate_fixed_array(dtype, shape):
    """reshape(T.((1:n)./n), sz) in Julia column-major order
    (lib/LuxLib/test/shared_testsetup.jl:69-73)."""
    n = int(np.prod(shape))
    return (np.arange(1, n + 1, dtype=np.float64) / n).astype(dtype).reshape(shape, order="F")


def to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """float32 -> bfloat16 bit patterns (uint16), round-to-nearest-even."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    rounded = u + (np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1)))
    return (rounded >> np.uint32(16)).astype(np.uint16)


def from_bf16_bits(b: np.ndarray) -> np.ndarray:
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def round_to_bf16(a: np.ndarray) -> np.ndarray:
    """float32 array whose values are exactly representable in bfloat16."""
    return from_bf16_bits(to_bf16_bits(a)).reshape(np.shape(a))
