"""Host-side mirror of LuxLib's public fused-operator API on top of libluxhip.

Same names, argument order and error behaviour as lib/LuxLib/src/api/*.jl of the reference
(Julia is not available where this runs, so this module plays the role the Julia glue in
`julia/LuxHIP.jl` plays inside LuxLib): arguments are checked on the host before anything is
launched (DimensionMismatch / ArgumentError / AssertionError), the device work goes through
the C ABI, and every operator has an `rrule` that returns `(y, pullback)` like its
ChainRulesCore counterpart.  `pullback(f, *args)` is the `Zygote.pullback` analogue.

Activations are passed by name ("relu", "tanh", "gelu", ...).  Tensors are `DeviceArray`s in
Julia's column-major layout and logical shapes (W, H, C, N) / (features, batch).
"""
from __future__ import annotations

import ctypes as C
import math
from dataclasses import dataclass, field
from typing import Optional, Sequence, Tuple

import numpy as np

from . import _lib
from .array import DeviceArray, StatArray, current_stream


# ------------------------------------------------------------------------------- errors
class DimensionMismatch(ValueError):
    """Julia's DimensionMismatch (impl/matmul.jl:21-34 of the reference)."""


class ArgumentError(ValueError):
    """Julia's ArgumentError (api/groupnorm.jl:40-64 of the reference)."""


def _act_id(act) -> int:
    try:
        return _lib.ACT_IDS[act]
    except (KeyError, TypeError):
        raise _lib.Unsupported(_lib.UNSUPPORTED, f"activation {act!r} has no device kernel") from None


# Activations without a device kernel (arbitrary closures: branch 3 of the reference's rules, impl/dense.jl:103-112,
# impl/conv.jl:271-275, impl/bias_activation.jl:96-104; its dense tests use `x -> x^3`).  The contraction and the bias
# run on the device with the identity; σ is applied, and differentiated, on a staged host copy: slow, correct.
# A closure is any Python callable that maps a float64 numpy array to one of the same shape, elementwise; its derivative
# is `act.derivative` (same calling convention) if it has one, central differences in float64 otherwise.
def _is_closure(act) -> bool:
    return callable(act) and not isinstance(act, str)


def _closure_derivative(act, z: np.ndarray) -> np.ndarray:
    d = getattr(act, "derivative", None)
    if d is not None:
        return np.asarray(d(z), np.float64)
    h = 1e-6 * np.maximum(1.0, np.abs(z))
    return (np.asarray(act(z + h), np.float64) - np.asarray(act(z - h), np.float64)) / (2.0 * h)


def _closure_rule(act, z: DeviceArray):
    """(σ.(z), Δ -> Δ .* σ'.(z)) through a host copy of z (what `rrule_via_ad(cfg, broadcast, σ, z)` gives the reference)."""
    zh = z.to_numpy().astype(np.float64)
    y = DeviceArray.from_numpy(np.asarray(act(zh), np.float64).astype(np.float32), z.dtype)

    def back(delta: DeviceArray) -> DeviceArray:
        dz = delta.to_numpy().astype(np.float64) * _closure_derivative(act, zh)
        return DeviceArray.from_numpy(dz.astype(np.float32), z.dtype)

    return y, back


_NEEDS_PRE = {4, 5, 6, 7, 8}   # swish, gelu, softplus, logsigmoid, lisht (rrule branch 2)


def _p(a) -> Optional[int]:
    return None if a is None else a.ptr


def _same_dtype(*arrs):
    dts = {a.dtype for a in arrs if a is not None}
    if len(dts) > 1:
        # the reference promotes mixed inputs with a one-time warning (impl/conv.jl:11-19,
        # ext/CUDAExt/cublaslt.jl:46-63); the device kernels want one storage type
        raise _lib.Unsupported(_lib.UNSUPPORTED, f"mixed storage types {sorted(dts)}")
    return dts.pop()


_warned_mixed = [False]


def _convert(a: DeviceArray, dtype: str) -> DeviceArray:
    out = DeviceArray(a.shape, dtype)
    _lib.call("luxhip_convert", current_stream(), a.code, out.code, a.size, a.ptr, out.ptr)
    return out


def _promote(*arrs):
    """Operands of mixed storage types are promoted to the widest one, with a warning the first time, as the
    reference's fused dense and convolution do (ext/CUDAExt/cublaslt.jl:46-63, impl/conv.jl:11-19).  Returns
    (operands, None) when there is nothing to do, else (promoted operands, the original types)."""
    dts = {a.dtype for a in arrs if a is not None}
    if len(dts) <= 1:
        return arrs, None
    if not _warned_mixed[0]:
        _warned_mixed[0] = True
        import warnings
        warnings.warn(f"Mixed-precision operands {sorted(dts)}: promoting to f32 (this warning is shown once).")
    return (tuple(a if a is None or a.dtype == "f32" else _convert(a, "f32") for a in arrs),
            tuple(None if a is None else a.dtype for a in arrs))


def _promoted_rule(rule, orig, *args):
    """The rule on promoted operands; gradients go back to each operand's own storage type."""
    y, back = rule(*args)

    def back_cast(delta, *rest):
        grads = back(delta if delta.dtype == "f32" else _convert(delta, "f32"), *rest)
        return tuple(g if g is None or dt_ is None or g.dtype == dt_ else _convert(g, dt_) for g, dt_ in zip(grads, orig))

    return y, back_cast


def default_epsilon(dtype: str) -> float:
    """eps(T)^(5/7) (utils.jl:130); eps(BFloat16) = 2^-7."""
    eps = 2.0 ** -23 if dtype == "f32" else 2.0 ** -7
    return eps ** (5.0 / 7.0)


def _icn(x: DeviceArray) -> Tuple[int, int, int]:
    """(I, C, N) view of an array whose channel dim is ndims-1 (vectors: (len, 1))."""
    if x.ndim == 1:
        return 1, x.shape[0], 1
    I = 1
    for s in x.shape[:-2]:
        I *= s
    return I, x.shape[-2], x.shape[-1]


# ------------------------------------------------------------------------------- bias_activation
def _check_bias(x: DeviceArray, bias: Optional[DeviceArray]):
    if bias is None:
        return
    want = x.shape[0] if x.ndim == 1 else x.shape[-2]
    # api/bias_activation.jl:38-45
    assert bias.ndim == 1 and bias.shape[0] == want, "length(bias) must equal size(x, ndims(x) - 1)"


def bias_activation(act: str, x: DeviceArray, bias: Optional[DeviceArray]) -> DeviceArray:
    """`bias_activation(σ, x, bias)` (api/bias_activation.jl:16-21)."""
    _check_bias(x, bias)
    if _is_closure(act):
        return _closure_rule(act, bias_activation("identity", x, bias))[0]
    aid = _act_id(act)
    y = DeviceArray(x.shape, _same_dtype(x, bias))
    I, Cc, N = _icn(x)
    _lib.call("luxhip_bias_activation_fwd", current_stream(), x.code, aid, I, Cc, N, x.ptr, _p(bias), y.ptr, None)
    return y


def bias_activation_inplace(act: str, x: DeviceArray, bias: Optional[DeviceArray]) -> DeviceArray:
    """`bias_activation!!(σ, x, bias)` (api/bias_activation.jl:31-36): overwrites and returns x."""
    _check_bias(x, bias)
    _same_dtype(x, bias)
    if _is_closure(act):
        y = _closure_rule(act, bias_activation_inplace("identity", x, bias))[0]
        _lib.call("luxhip_memcpy_d2d", x.ptr, y.ptr, x.nbytes, current_stream())
        return x
    I, Cc, N = _icn(x)
    _lib.call("luxhip_bias_activation_fwd", current_stream(), x.code, _act_id(act), I, Cc, N, x.ptr, _p(bias), x.ptr, None)
    return x


def rrule_bias_activation(act: str, x: DeviceArray, bias: Optional[DeviceArray]):
    """CRC.rrule(bias_activation) (impl/bias_activation.jl:64-104): (y, Δ -> (∂x, ∂b))."""
    _check_bias(x, bias)
    if _is_closure(act):
        z, back_z = rrule_bias_activation("identity", x, bias)
        y, back_act = _closure_rule(act, z)
        return y, (lambda delta: back_z(back_act(delta)))
    aid = _act_id(act)
    dt = _same_dtype(x, bias)
    I, Cc, N = _icn(x)
    y = DeviceArray(x.shape, dt)
    pre = DeviceArray(x.shape, dt) if aid in _NEEDS_PRE else None
    _lib.call("luxhip_bias_activation_fwd", current_stream(), x.code, aid, I, Cc, N, x.ptr, _p(bias), y.ptr, _p(pre))

    def back(delta: DeviceArray):
        dx = DeviceArray(x.shape, dt)
        db = None if bias is None else DeviceArray(bias.shape, dt)
        _lib.call("luxhip_bias_activation_bwd", current_stream(), x.code, aid, I, Cc, N, delta.ptr, y.ptr, _p(pre),
                  dx.ptr, _p(db))
        return dx, db

    return y, back


# ------------------------------------------------------------------------------- fast_activation
def fast_activation(act: str, x: DeviceArray) -> DeviceArray:
    """`fast_activation(σ, x)` (api/activation.jl:55-57): σ.(x) into a new array."""
    if _is_closure(act):
        return _closure_rule(act, x)[0]
    aid = _act_id(act)
    y = DeviceArray(x.shape, x.dtype)
    _lib.call("luxhip_bias_activation_fwd", current_stream(), x.code, aid, 1, 1, x.size, x.ptr, None, y.ptr, None)
    return y


def fast_activation_inplace(act: str, x: DeviceArray) -> DeviceArray:
    """`fast_activation!!(σ, x)` (api/activation.jl:27-29): overwrites and returns x."""
    if _is_closure(act):
        y = _closure_rule(act, x)[0]
        _lib.call("luxhip_memcpy_d2d", x.ptr, y.ptr, x.nbytes, current_stream())
        return x
    _lib.call("luxhip_bias_activation_fwd", current_stream(), x.code, _act_id(act), 1, 1, x.size, x.ptr, None, x.ptr, None)
    return x


def rrule_fast_activation(act: str, x: DeviceArray):
    """CRC.rrule(activation!!) (impl/activation.jl:20-49): (y, Δ -> (∂x,)); ∂x = Δ·dσ(y, x)
    (∇activation, impl/activation.jl:135-154).  x itself is the saved pre-activation."""
    if _is_closure(act):
        y, back_act = _closure_rule(act, x)
        return y, (lambda delta: (back_act(delta),))
    aid = _act_id(act)
    y = DeviceArray(x.shape, x.dtype)
    _lib.call("luxhip_bias_activation_fwd", current_stream(), x.code, aid, 1, 1, x.size, x.ptr, None, y.ptr, None)

    def back(delta: DeviceArray):
        dx = DeviceArray(x.shape, x.dtype)
        _lib.call("luxhip_bias_activation_bwd", current_stream(), x.code, aid, 1, 1, x.size, delta.ptr, y.ptr,
                  x.ptr if aid in _NEEDS_PRE else None, dx.ptr, None)
        return (dx,)

    return y, back


# ------------------------------------------------------------------------------- dropout
@dataclass(frozen=True)
class PhiloxRNG:
    """The generator state handed to dropout in place of Julia's `rng`: a counter-based Philox4x32-10
    stream (seed = key, offset = first counter block).  Like `LuxCore.replicate(rng)` followed by
    `rand!`, drawing n values returns a new state and leaves this one untouched."""
    seed: int = 0
    offset: int = 0

    def advanced(self, n: int) -> "PhiloxRNG":
        return PhiloxRNG(self.seed, self.offset + (n + 3) // 4)


def dropout_shape(x_shape, dims):
    """`dropout_shape(x, dims)` (impl/dropout.jl:74-78): dims is None (Julia's `:`) or the 1-based
    dims along which the mask varies."""
    if dims is None:
        return tuple(x_shape)
    return tuple(s if (i + 1) in dims else 1 for i, s in enumerate(x_shape))


def rand_uniform(rng: PhiloxRNG, shape, dtype="f32"):
    """`rand!(rng, similar(x, shape))`: (noise, advanced rng)."""
    out = DeviceArray(tuple(shape), dtype)
    _lib.call("luxhip_rand_uniform", current_stream(), out.code, out.size, rng.seed, rng.offset, out.ptr)
    return out, rng.advanced(out.size)


def _shape_arg(shape):
    return (C.c_int64 * max(len(shape), 1))(*shape)


def dropout_dot_mul(x: DeviceArray, mask: DeviceArray) -> DeviceArray:
    """`dropout_dot_mul(x, mask)` = x .* mask (impl/dropout.jl:220), mask broadcast over its
    singleton dims."""
    if mask.ndim != x.ndim or any(m not in (1, sx) for m, sx in zip(mask.shape, x.shape)):
        raise AssertionError("`mask` is not of the same size as `LuxLib.dropout_shape(x, dims)`.")   # impl/dropout.jl:49-52
    _same_dtype(x, mask)
    y = DeviceArray(x.shape, x.dtype)
    _lib.call("luxhip_dropout_mul", current_stream(), x.code, x.ndim, _shape_arg(x.shape), _shape_arg(mask.shape),
              x.ptr, mask.ptr, y.ptr)
    return y


def _dropout_fwd(rng, x, p, training, invp, dims, mask, update_mask):
    if mask is not None and not update_mask:
        if not training:
            return x, mask, rng                                   # impl/dropout.jl:36-47
        if tuple(mask.shape) != dropout_shape(x.shape, dims):
            raise AssertionError("`mask` is not of the same size as `LuxLib.dropout_shape(x, dims)`.")
        return dropout_dot_mul(x, mask), mask, rng                # impl/dropout.jl:22-34
    if not training:
        return x, (x if mask is None else mask), rng              # impl/dropout.jl:8
    mshape = dropout_shape(x.shape, dims)
    new_mask = DeviceArray(mshape, x.dtype)
    if mshape == tuple(x.shape):
        y = DeviceArray(x.shape, x.dtype)
        _lib.call("luxhip_dropout_fwd", current_stream(), x.code, x.size, rng.seed, rng.offset, float(p), float(invp),
                  x.ptr, y.ptr, new_mask.ptr)
    else:
        _lib.call("luxhip_dropout_fwd", current_stream(), x.code, new_mask.size, rng.seed, rng.offset, float(p), float(invp),
                  None, None, new_mask.ptr)
        y = dropout_dot_mul(x, new_mask)
    return y, new_mask, rng.advanced(new_mask.size)


def dropout(rng: PhiloxRNG, x: DeviceArray, p, training, invp, dims=None, *, mask=None, update_mask=True):
    """`dropout(rng, x, p, training, invp, dims)` and, with `mask=`/`update_mask=`,
    `dropout(rng, x, mask, p, training, update_mask, invp, dims)` (api/dropout.jl:40-69):
    returns `(y, mask, rng′)`.  dims=None is Julia's `:`."""
    return _dropout_fwd(rng, x, p, bool(training), invp, dims, mask, bool(update_mask))


def rrule_dropout(rng, x, p, training, invp, dims=None, *, mask=None, update_mask=True):
    """((y, mask, rng′), Δ -> (∂x,)): only dropout_dot_mul is differentiable
    (impl/dropout.jl:222-228): ∂x = Δ .* mask; not training: ∂x = Δ."""
    training = bool(training)
    y, m, rng2 = _dropout_fwd(rng, x, p, training, invp, dims, mask, bool(update_mask))

    def back(delta: DeviceArray):
        return (dropout_dot_mul(delta, m) if training else delta,)

    return (y, m, rng2), back


def _alpha_coefficients(p, alpha, A, B):
    if alpha is None:                                             # impl/dropout.jl:57-62
        alpha = -1.7580993408473766
        A = 1.0 / math.sqrt((1 - p) * (1 + p * alpha ** 2))
        B = -A * alpha * p
    return float(alpha), float(A), float(B)


def alpha_dropout(rng: PhiloxRNG, x: DeviceArray, p, training, alpha=None, A=None, B=None):
    """`alpha_dropout(rng, x, p, training[, α, A, B])` (api/dropout.jl:107-115): `(y, rng′)`."""
    return rrule_alpha_dropout(rng, x, p, training, alpha, A, B)[0]


def rrule_alpha_dropout(rng, x, p, training, alpha=None, A=None, B=None):
    """((y, rng′), Δ -> (∂x,)); ∂x = Δ · (noise > p) · A (impl/dropout.jl:137-150)."""
    if not bool(training):
        return (x, rng), (lambda delta: (delta,))                 # impl/dropout.jl:71
    alpha, A, B = _alpha_coefficients(float(p), alpha, A, B)
    noise, rng2 = rand_uniform(rng, x.shape, x.dtype)             # generate_alpha_dropout_noise, impl/dropout.jl:171-177
    y = DeviceArray(x.shape, x.dtype)
    _lib.call("luxhip_alpha_dropout_fwd", current_stream(), x.code, x.size, noise.ptr, float(p), x.ptr, alpha, A, B, y.ptr)

    def back(delta: DeviceArray):
        dx = DeviceArray(x.shape, x.dtype)
        _lib.call("luxhip_alpha_dropout_bwd", current_stream(), x.code, x.size, noise.ptr, float(p), delta.ptr, A, dx.ptr)
        return (dx,)

    return (y, rng2), back


# ------------------------------------------------------------------------------- dense
def _check_dense(weight, x, b):
    if weight.ndim != 2 or x.ndim != 2:
        raise DimensionMismatch("weight and x must be matrices")
    if weight.shape[1] != x.shape[0]:
        raise DimensionMismatch(f"A has shape {weight.shape} but B has shape {x.shape}")
    if b is not None and (b.ndim != 1 or b.shape[0] != weight.shape[0]):
        raise DimensionMismatch(f"bias has length {b.shape} but the output has {weight.shape[0]} rows")


def fused_dense_bias_activation(act: str, weight: DeviceArray, x: DeviceArray, b: Optional[DeviceArray]) -> DeviceArray:
    """`fused_dense_bias_activation(σ, weight, x, b)` (api/dense.jl:33-37): σ.(weight * x .+ b)."""
    _check_dense(weight, x, b)
    if _is_closure(act):
        return _closure_rule(act, fused_dense_bias_activation("identity", weight, x, b))[0]
    (weight, x, b), _ = _promote(weight, x, b)
    dt = _same_dtype(weight, x, b)
    M, K = weight.shape
    N = x.shape[1]
    y = DeviceArray((M, N), dt)
    _lib.call("luxhip_fused_dense_fwd", current_stream(), y.code, _act_id(act), M, K, N, weight.ptr, max(M, 1), x.ptr,
              max(K, 1), _p(b), y.ptr, max(M, 1), None)
    return y


def rrule_fused_dense_bias_activation(act: str, weight: DeviceArray, x: DeviceArray, b: Optional[DeviceArray]):
    """CRC.rrule(fused_dense) (impl/dense.jl:71-134): (y, Δ -> (∂W, ∂x, ∂b))."""
    _check_dense(weight, x, b)
    if _is_closure(act):                      # impl/dense.jl:103-112: matmuladd on the device, σ and its pullback around it
        z, back_z = rrule_fused_dense_bias_activation("identity", weight, x, b)
        y, back_act = _closure_rule(act, z)
        return y, (lambda delta: back_z(back_act(delta)))
    (pw, px, pb), orig = _promote(weight, x, b)
    if orig is not None:
        return _promoted_rule(lambda *a: rrule_fused_dense_bias_activation(act, *a), orig, pw, px, pb)
    aid = _act_id(act)
    dt = _same_dtype(weight, x, b)
    M, K = weight.shape
    N = x.shape[1]
    y = DeviceArray((M, N), dt)
    pre = DeviceArray((M, N), dt) if aid in _NEEDS_PRE else None
    _lib.call("luxhip_fused_dense_fwd", current_stream(), y.code, aid, M, K, N, weight.ptr, max(M, 1), x.ptr, max(K, 1),
              _p(b), y.ptr, max(M, 1), _p(pre))

    def back(delta: DeviceArray):
        dW = DeviceArray((M, K), dt)
        dx = DeviceArray((K, N), dt)
        db = None if b is None else DeviceArray((M,), dt)
        dz = None if aid == 0 else DeviceArray((M, N), dt)
        _lib.call("luxhip_fused_dense_bwd", current_stream(), y.code, aid, M, K, N, delta.ptr, y.ptr, _p(pre), weight.ptr,
                  max(M, 1), x.ptr, max(K, 1), _p(dz), dW.ptr, dx.ptr, _p(db))
        return dW, dx, db

    return y, back


def matmul(A: DeviceArray, B: DeviceArray, bias: Optional[DeviceArray] = None, transA=False, transB=False) -> DeviceArray:
    """`matmul` / `matmuladd` (impl/matmul.jl:2-94) with optionally transposed operands."""
    am, ak = (A.shape[1], A.shape[0]) if transA else A.shape
    bk, bn = (B.shape[1], B.shape[0]) if transB else B.shape
    if ak != bk:
        raise DimensionMismatch(f"A has shape {(am, ak)} but B has shape {(bk, bn)}")
    if bias is not None and bias.shape[0] != am:
        raise DimensionMismatch("bias length does not match rows of A")
    dt = _same_dtype(A, B, bias)
    out = DeviceArray((am, bn), dt)
    _lib.call("luxhip_matmul", current_stream(), out.code, int(transA), int(transB), am, bn, ak, A.ptr, max(A.shape[0], 1),
              B.ptr, max(B.shape[0], 1), _p(bias), out.ptr, max(am, 1))
    return out


# ------------------------------------------------------------------------------- batched_matmul
def _as_batched(a: DeviceArray, what: str):
    """(rows, cols, batch, batch_shape) of an N-d operand whose batching dims are the trailing ones."""
    if a.ndim < 3:
        raise ArgumentError(f"{what}: N must be at least 3")       # impl/batched_mul.jl:127
    b = 1
    for sdim in a.shape[2:]:
        b *= sdim
    return a.shape[0], a.shape[1], b, tuple(a.shape[2:])


def _bmm(A, tA, B, tB, M, N, K, batch, sA, sB, dtype):
    out = DeviceArray((M, N, batch), dtype)
    _lib.call("luxhip_batched_matmul", current_stream(), out.code, int(tA), int(tB), M, N, K, batch,
              A.ptr, max(A.shape[0], 1), sA, B.ptr, max(B.shape[0], 1), sB, out.ptr, max(M, 1), M * N)
    return out


def _batched_geometry(x, y, lhs_contracting_dim, rhs_contracting_dim):
    if x.ndim == 2 and y.ndim >= 3:
        x = x.reshape(x.shape + (1,) * (y.ndim - 2))               # expand_batchdim, api/batched_mul.jl
    if y.ndim == 2 and x.ndim >= 3:
        y = y.reshape(y.shape + (1,) * (x.ndim - 2))
    if x.ndim != y.ndim:
        raise ArgumentError("batched_matmul: x and y must have the same number of dims")
    if lhs_contracting_dim not in (1, 2) or rhs_contracting_dim not in (1, 2):
        raise _lib.Unsupported(_lib.UNSUPPORTED, "batched_matmul: the batching dims must be the trailing ones")
    xr, xc, xb, xbs = _as_batched(x, "x")
    yr, yc, yb, ybs = _as_batched(y, "y")
    for a_, b_ in zip(xbs, ybs):
        if a_ != b_ and a_ != 1 and b_ != 1:
            raise DimensionMismatch(f"Batching dimensions mismatch: {xbs} vs {ybs}")      # impl/batched_mul.jl:133-141
    bshape = tuple(max(a_, b_) for a_, b_ in zip(xbs, ybs))
    batch = 1
    for sdim in bshape:
        batch *= sdim
    if not (xb in (1, batch) and yb in (1, batch)):
        raise _lib.Unsupported(_lib.UNSUPPORTED, "batched_matmul: batch dims that repeat only some of several dims")
    tA, tB = lhs_contracting_dim == 1, rhs_contracting_dim == 2
    M, Kx = (xc, xr) if tA else (xr, xc)
    Ky, N = (yc, yr) if tB else (yr, yc)
    if Kx != Ky:
        raise DimensionMismatch(f"size(x) = {x.shape}, size(y) = {y.shape} inconsistent for batched_matmul.")
    return x, y, tA, tB, M, N, Kx, batch, xb, yb, bshape


def batched_matmul(x: DeviceArray, y: DeviceArray, lhs_contracting_dim: int = 2, rhs_contracting_dim: int = 1,
                   lhs_batching_dims=None, rhs_batching_dims=None):
    """`batched_matmul(x, y; lhs_contracting_dim, rhs_contracting_dim, lhs_batching_dims, rhs_batching_dims)`
    (api/batched_mul.jl, impl/batched_mul.jl:2-58): z[:, :, b...] = op(x[.., b...]) op(y[.., b...]); batch
    dims of extent 1 are shared among the products.  The batching dims default to the trailing ones."""
    return rrule_batched_matmul(x, y, lhs_contracting_dim, rhs_contracting_dim, lhs_batching_dims, rhs_batching_dims,
                                _need_back=False)[0]


def _dense_strides(shape):
    st, p = [], 1
    for e in shape:
        st.append(p)
        p *= e
    return st


class _BmmOperand:
    """One operand of the general product: where its (free x contracting) matrix and its batching dims lie."""

    def __init__(self, a: DeviceArray, contracting_dim: int, batching_dims, what: str):
        nd = a.ndim
        if nd < 3:
            raise ArgumentError(f"{what}: N must be at least 3")
        bd = tuple(range(3, nd + 1)) if batching_dims is None else tuple(int(d) for d in batching_dims)
        rest = [d for d in range(1, nd + 1) if d != contracting_dim and d not in bd]
        if len(bd) != nd - 2 or len(set(bd)) != len(bd) or len(rest) != 1 or not 1 <= contracting_dim <= nd:
            raise ArgumentError(f"{what}: one contracting dim, one free dim and N - 2 distinct batching dims are needed")
        st = _dense_strides(a.shape)
        self.a, self.bd = a, bd
        self.F, self.K = a.shape[rest[0] - 1], a.shape[contracting_dim - 1]
        self.sf, self.sk = st[rest[0] - 1], st[contracting_dim - 1]
        self.bext = [a.shape[d - 1] for d in bd]
        self.bst = [st[d - 1] for d in bd]
        # free-major: the free index is the contiguous one
        if self.sf == 1 or self.F == 1:
            self.free_major, self.ld = True, (self.sk if self.K > 1 else max(self.F, 1))
        elif self.sk == 1 or self.K == 1:
            self.free_major, self.ld = False, (self.sf if self.F > 1 else max(self.K, 1))
        else:
            raise _lib.Unsupported(_lib.UNSUPPORTED, f"batched_matmul: neither matrix dim of {what} is contiguous")


def _launch_general(tA, tB, M, N, K, pairs, A, lda, B, ldb, Cm, ldc):
    """pairs: (extent, stride in A, stride in B, stride in C) per batch dim, innermost first."""
    pairs = [p for p in pairs if p[0] != 1]
    merged = []
    for p in pairs:
        if merged:
            e, sa, sb, sc = merged[-1]
            if p[1] == sa * e and p[2] == sb * e and p[3] == sc * e:
                merged[-1] = (e * p[0], sa, sb, sc)
                continue
        merged.append(p)
    if len(merged) > 3:
        raise _lib.Unsupported(_lib.UNSUPPORTED, "batched_matmul: more than three batch dims that cannot be merged")
    merged += [(1, 0, 0, 0)] * (3 - len(merged))
    _bmm_strided(tA, tB, M, N, K, [p[0] for p in merged], A, lda, [p[1] for p in merged], B, ldb, [p[2] for p in merged],
                 Cm, ldc, [p[3] for p in merged])


def _rrule_batched_matmul_general(x, y, cx, cy, bx, by):
    dt = _same_dtype(x, y)
    X, Y = _BmmOperand(x, cx, bx, "x"), _BmmOperand(y, cy, by, "y")
    if X.K != Y.K:
        raise DimensionMismatch(f"size(x) = {x.shape}, size(y) = {y.shape} inconsistent for batched_matmul.")
    for a_, b_ in zip(X.bext, Y.bext):
        if a_ != b_ and a_ != 1 and b_ != 1:
            raise DimensionMismatch(f"Batching dimensions mismatch: {X.bext} vs {Y.bext}")      # impl/batched_mul.jl:133-141
    M, N, K = X.F, Y.F, X.K
    ext = [max(a_, b_) if min(a_, b_) > 0 else 0 for a_, b_ in zip(X.bext, Y.bext)]
    zst = _dense_strides((M, N) + tuple(ext))[2:]
    sx = [st if e > 1 else 0 for st, e in zip(X.bst, X.bext)]
    sy = [st if e > 1 else 0 for st, e in zip(Y.bst, Y.bext)]
    tA, tB = not X.free_major, Y.free_major          # A is M x K: transposed storage = contracting-major; B is K x N
    z = DeviceArray((M, N) + tuple(ext), dt)
    if z.size:
        _launch_general(tA, tB, M, N, K, list(zip(ext, sx, sy, zst)), x, X.ld, y, Y.ld, z, M)

    def grad(op, other_is_y):
        """Gradient of one operand, in its own layout."""
        a = op.a
        shared = [i for i in range(len(ext)) if op.bext[i] == 1 and ext[i] > 1]
        shared_total = int(np.prod([ext[i] for i in shared], dtype=np.int64)) if shared else 1
        target = DeviceArray(tuple(a.shape) + ((shared_total,) if shared else ()), dt)
        # a repeated operand gets one slab in its own layout per repetition, summed afterwards (the repeated
        # dims have extent 1 in the operand, so they do not enter its layout)
        sc, p = [0] * len(ext), a.size
        for i in range(len(ext)):
            sc[i] = op.bst[i] if op.bext[i] > 1 else 0
        for i in shared:
            sc[i] = p
            p *= ext[i]
        return a, shared, shared_total, target, sc

    def back(delta: DeviceArray):
        out = []
        for op, is_x in ((X, True), (Y, False)):
            a, shared, shared_total, target, sc = grad(op, is_x)
            if target.size:
                pairs = lambda sother: list(zip(ext, zst, sother, sc))
                if is_x:
                    if X.free_major:        # dx (M x K) = Δ op(y)ᵀ
                        _launch_general(False, not tB, M, K, N, pairs(sy), delta, M, y, Y.ld, target, X.ld)
                    else:                   # stored K x M: op(y) Δᵀ
                        _launch_general(tB, True, K, M, N, [(e, b_, a_, c_) for e, a_, b_, c_ in pairs(sy)], y, Y.ld, delta, M,
                                        target, X.ld)
                else:
                    if not Y.free_major:    # dy (K x N) = op(x)ᵀ Δ
                        _launch_general(not tA, False, K, N, M, [(e, b_, a_, c_) for e, a_, b_, c_ in pairs(sx)], x, X.ld, delta, M,
                                        target, Y.ld)
                    else:                   # stored N x K: Δᵀ op(x)
                        _launch_general(True, tA, N, K, M, pairs(sx), delta, M, x, X.ld, target, Y.ld)
            if shared:
                red = DeviceArray(a.shape, dt)
                _lib.call("luxhip_batch_sum", current_stream(), red.code, a.size, shared_total, target.ptr, red.ptr)
                target = red
            out.append(target)
        return tuple(out)

    return z, back


def rrule_batched_matmul(x, y, lhs_contracting_dim=2, rhs_contracting_dim=1, lhs_batching_dims=None, rhs_batching_dims=None,
                         _need_back=True):
    """CRC.rrule(batched_matmul_fallback) (impl/batched_mul.jl:320-334): (z, Δ -> (∂x, ∂y)) with
    ∂x = Δ ⊠ adjoint(y), ∂y = adjoint(x) ⊠ Δ, summed over the batch for a shared operand."""
    x_shape, y_shape = x.shape, y.shape
    dt = _same_dtype(x, y)
    trailing = lambda a, bd: bd is None or tuple(bd) == tuple(range(3, a.ndim + 1))
    simple = (trailing(x, lhs_batching_dims) and trailing(y, rhs_batching_dims) and lhs_contracting_dim in (1, 2)
              and rhs_contracting_dim in (1, 2))
    if simple and x.ndim == y.ndim and x.ndim >= 3:
        xb_, yb_ = x.shape[2:], y.shape[2:]
        full = tuple(max(a_, b_) for a_, b_ in zip(xb_, yb_))
        simple = all(a_ in (b_, 1) or b_ == 1 for a_, b_ in zip(xb_, yb_)) and all(
            tuple(o) == full or int(np.prod(o, dtype=np.int64)) == 1 for o in (xb_, yb_))
    if not simple and x.ndim == y.ndim and x.ndim >= 3:
        return _rrule_batched_matmul_general(x, y, lhs_contracting_dim, rhs_contracting_dim, lhs_batching_dims, rhs_batching_dims)
    x, y, tA, tB, M, N, K, batch, xb, yb, bshape = _batched_geometry(x, y, lhs_contracting_dim, rhs_contracting_dim)
    sx, sy = (x.shape[0] * x.shape[1] if xb > 1 else 0), (y.shape[0] * y.shape[1] if yb > 1 else 0)
    z = _bmm(x, tA, y, tB, M, N, K, batch, sx, sy, dt).reshape((M, N) + bshape)

    def back(delta: DeviceArray):
        g = delta.reshape((M, N, batch))
        # ∂(op(x)) = Δ op(y)ᵀ, stored as x is: transposed when x is contracted along dim 1
        if not tA:
            dx = _bmm(g, False, y, not tB, M, K, N, batch, M * N, sy, dt)
        else:
            dx = _bmm(y, tB, g, True, K, M, N, batch, sy, M * N, dt)
        if not tB:
            dy = _bmm(x, not tA, g, False, K, N, M, batch, sx, M * N, dt)
        else:
            dy = _bmm(g, True, x, tA, N, K, M, batch, M * N, sx, dt)
        out = []
        for grad, shared, shape in ((dx, xb == 1 and batch > 1, x_shape), (dy, yb == 1 and batch > 1, y_shape)):
            if shared:
                n = grad.shape[0] * grad.shape[1]
                red = DeviceArray((grad.shape[0], grad.shape[1], 1), dt)
                _lib.call("luxhip_batch_sum", current_stream(), grad.code, n, batch, grad.ptr, red.ptr)
                grad = red
            out.append(grad.reshape(shape))
        return tuple(out)

    return z, back


# ------------------------------------------------------------------------------- attention
def _i64x3(v):
    return (C.c_int64 * 3)(*v)


_BF16_WIDE = 2      # LUXHIP_BF16_WIDE: bf16 storage with the logits / their cotangent in fp32


def _bmm_strided(tA, tB, M, N, K, bdims, A, lda, sA, B, ldb, sB, Cm, ldc, sC, structure=0):
    code = _BF16_WIDE if (A.dtype == "bf16" and Cm.dtype == "f32") else Cm.code
    _lib.call("luxhip_batched_matmul_strided", current_stream(), code, int(tA), int(tB), M, N, K, _i64x3(bdims),
              A.ptr, max(lda, 1), _i64x3(sA), B.ptr, max(ldb, 1), _i64x3(sB), Cm.ptr, max(ldc, 1), _i64x3(sC), int(structure))


class _AttnLayout:
    """Strides (elements) of an attention operand whose embedding dim is the first: token / heads
    dims are 2 and 3 in either order, everything after is one flattened batch dim."""

    def __init__(self, a: DeviceArray, token_dim: int):
        self.E, d2, d3 = a.shape[0], a.shape[1], a.shape[2]
        self.tokens, self.heads = (d2, d3) if token_dim == 2 else (d3, d2)
        self.st, self.sh = (self.E, self.E * d2) if token_dim == 2 else (self.E * d2, self.E)
        self.sb = self.E * d2 * d3
        self.batch = a.size // self.sb if self.sb else 0


def _permute_leading3(a: DeviceArray, perm) -> DeviceArray:
    """permutedims(a, (perm..., 4:N...))."""
    out = DeviceArray(tuple(a.shape[p - 1] for p in perm) + tuple(a.shape[3:]), a.dtype)
    outer = int(np.prod(a.shape[3:], dtype=np.int64)) if a.ndim > 3 else 1
    _lib.call("luxhip_permute_leading3", current_stream(), a.code, a.shape[0], a.shape[1], a.shape[2], outer, *perm, a.ptr, out.ptr)
    return out


def attention_dropout(rng: "PhiloxRNG", p: float):
    """An `fdrop` for scaled_dot_product_attention: dropout of the attention weights with rate p
    (what `Base.Fix2(fdrop, p)` is in test/common_ops/attention_tests.jl:291-299).  Called with the
    weights, returns (weights′, Δweights′ -> Δweights)."""
    def fdrop(weights: DeviceArray):
        (y, _, _), back = rrule_dropout(rng, weights, p, True, 1.0 / (1.0 - p))
        return y, (lambda d: back(d)[0])
    return fdrop


def scaled_dot_product_attention(q: DeviceArray, k: DeviceArray, v: DeviceArray, head_dim: int = 1, token_dim: int = 3,
                                 scale=None, mask=None, is_causal=None, bias=None, fdrop=None):
    """`scaled_dot_product_attention(q, k, v; head_dim, token_dim, scale, mask, is_causal, bias, fdrop)`
    (api/attention.jl, impl/attention.jl:5-117): returns `(output [Ev, H, L, B...], attention weights
    [S, L, H, B...])`.  `mask` / `bias`: host arrays or DeviceArrays of shape [S, L, H or 1, B or 1].
    `fdrop`: None (identity) or a callable weights -> (weights′, pullback), e.g. `attention_dropout`."""
    return rrule_scaled_dot_product_attention(q, k, v, head_dim, token_dim, scale, mask, is_causal, bias, fdrop)[0]


def rrule_scaled_dot_product_attention(q, k, v, head_dim=1, token_dim=3, scale=None, mask=None, is_causal=None, bias=None,
                                       fdrop=None):
    """((output, weights), (Δoutput[, Δweights]) -> (∂q, ∂k, ∂v)): the pullbacks of the two batched
    products (impl/batched_mul.jl:320-334), of NNlib.softmax and of repeat_inner_gqa, composed as the
    reference's AD does.  The gradient of `bias` is not computed."""
    N = q.ndim
    # impl/attention.jl:16-43
    assert N >= 4 and k.ndim == N and v.ndim == N, "N must be at least 4"
    assert 1 <= head_dim <= 3 and 1 <= token_dim <= 3 and head_dim != token_dim, "head_dim and token_dim must differ, in 1:3"
    assert q.shape[head_dim - 1] == k.shape[head_dim - 1], "`q` and `k` must have the same number of heads."
    for i in range(3, N):
        if not (q.shape[i] == k.shape[i] == v.shape[i]):
            raise DimensionMismatch("All dimensions (except first 3) of q, k, v must be the same.")
    if head_dim != 1:
        # the kernels want the embedding dim first: bring the operands to (E, H, L, B...) and take the
        # gradients back (the results' layout does not depend on the operands', impl/attention.jl:107-117)
        heads_dim = ({1, 2, 3} - {head_dim, token_dim}).pop()
        perm = (head_dim, heads_dim, token_dim)
        inv = tuple(perm.index(d) + 1 for d in (1, 2, 3))
        res, back_c = rrule_scaled_dot_product_attention(*(_permute_leading3(a, perm) for a in (q, k, v)), 1, 3, scale, mask,
                                                         is_causal, bias, fdrop)
        return res, (lambda d_out, d_probs=None: tuple(_permute_leading3(g, inv) for g in back_c(d_out, d_probs)))
    dt = _same_dtype(q, k, v)
    lq, lk, lv = _AttnLayout(q, token_dim), _AttnLayout(k, token_dim), _AttnLayout(v, token_dim)
    assert lv.tokens == lk.tokens, "`v` and `k` must have the same number of tokens."
    assert lk.heads == lv.heads and lq.heads % max(lk.heads, 1) == 0, "num_heads must be divisible by num_kv_groups"
    if mask is not None and is_causal is not None:
        raise AssertionError("`mask` and `is_causal` cannot both be specified")
    E, Ev, H, G, L, S, B = lq.E, lv.E, lq.heads, lk.heads, lq.tokens, lk.tokens, lq.batch
    r = H // G if G else 1
    bshape = tuple(q.shape[3:])
    scale_inv = 1.0 / (math.sqrt(E) if scale is None else float(scale))      # impl/attention.jl:50-51
    bdims = (r, G, B)

    def side(arr, what, kind):
        if arr is None:
            return None, 0, 0
        if not isinstance(arr, DeviceArray):
            arr = DeviceArray.from_numpy(np.asarray(arr, np.uint8 if kind == "mask" else np.float32),
                                         "u8" if kind == "mask" else dt)
        shp = tuple(arr.shape) + (1,) * (4 - arr.ndim) if arr.ndim < 4 else (arr.shape[0], arr.shape[1], arr.shape[2],
                                                                              int(np.prod(arr.shape[3:])))
        if shp[0] != S or shp[1] != L or shp[2] not in (1, H) or shp[3] not in (1, B):
            raise DimensionMismatch(f"{what} of shape {arr.shape} does not broadcast to the logits {(S, L, H) + bshape}")
        return arr, (S * L if shp[2] == H and H > 1 else 0), (S * L * shp[2] if shp[3] == B and B > 1 else 0)

    mask_a, mask_sh, mask_sb = side(mask, "mask", "mask")
    bias_a, bias_sh, bias_sb = side(bias, "bias", "bias")
    # bf16: the logits and the cotangent of the weights stay in fp32 between the products and the softmax passes
    # (a logit rounded to bf16 is off by 2^-9 |logit|, the weight then by that relative amount)
    wide = "f32" if dt == "bf16" else dt
    sm_code = _BF16_WIDE if dt == "bf16" else None
    logits = DeviceArray((S, L, H) + bshape, wide)
    sC = (S * L, S * L * r, S * L * H)
    # a causal mask (keep s <= l) leaves whole tiles of the logits unused and makes the weights and every
    # cotangent of the same shape triangular: the products skip what is known to be zero or unused
    causal = bool(is_causal)
    tri = causal and fdrop is None       # an arbitrary fdrop need not keep the masked weights at zero
    _bmm_strided(True, False, S, L, E, bdims, k, lk.st, (0, lk.sh, lk.sb), q, lq.st, (lq.sh, lq.sh * r, lq.sb), logits, S, sC,
                 1 if causal else 0)
    probs = DeviceArray((S, L, H) + bshape, dt)
    _lib.call("luxhip_attention_softmax_fwd", current_stream(), probs.code if sm_code is None else sm_code, S, L, H, B, logits.ptr, scale_inv,
              int(causal), _p(mask_a), mask_sh, mask_sb, _p(bias_a), bias_sh, bias_sb, probs.ptr)
    softmax_out, fdrop_back = probs, None
    if fdrop is not None:
        probs, fdrop_back = fdrop(softmax_out)         # impl/attention.jl:88-104: fdrop(softmax(...))
    so = (Ev, Ev * r, Ev * H * L)
    # bf16 without an fdrop: the product is written unrounded (fp32) and kept for the pullback, whose softmax rule takes
    # its inner product from it; the array that is returned is its rounded copy
    out_wide = DeviceArray((Ev, H, L) + bshape, wide) if (fdrop is None and wide != dt) else None
    out = out_wide if out_wide is not None else DeviceArray((Ev, H, L) + bshape, dt)
    _bmm_strided(False, False, Ev, L, S, bdims, v, lv.st, (0, lv.sh, lv.sb), probs, S, sC, out, Ev * H, so, 2 if tri else 0)
    if out_wide is not None:
        out = _convert(out_wide, dt)

    def back(d_out: DeviceArray, d_probs: Optional[DeviceArray] = None):
        if d_probs is not None:
            raise _lib.Unsupported(_lib.UNSUPPORTED, "attention: a cotangent for the returned weights")
        dlogits = logits if logits.dtype == dt else DeviceArray(logits.shape, dt)   # the logits are no longer needed
        if fdrop_back is None:
            # the cotangent of the weights (v' d_out) and the softmax rule in one: the cotangent stays in the product's
            # fp32 accumulators, its inner product with the weights comes from d_out and out
            _lib.call("luxhip_attention_weights_pullback", current_stream(), softmax_out.code if out_wide is None else _BF16_WIDE, S, L,
                      Ev, _i64x3(bdims), v.ptr, max(lv.st, 1), _i64x3((0, lv.sh, lv.sb)), d_out.ptr,
                      (out if out_wide is None else out_wide).ptr, max(Ev * H, 1), _i64x3(so), softmax_out.ptr,
                      scale_inv, dlogits.ptr, max(S, 1), _i64x3(sC), 1 if tri else 0)
        else:
            # with an fdrop the cotangent passes through its pullback in the storage type first
            dp = DeviceArray(probs.shape, dt)
            _bmm_strided(True, False, S, L, Ev, bdims, v, lv.st, (0, lv.sh, lv.sb), d_out, Ev * H, so, dp, S, sC, 1 if tri else 0)
            dp = fdrop_back(dp)
            # the causal shortcut of the softmax pullback leaves dlogits beyond the diagonal block untouched, which
            # only the triangular products that follow tolerate: with an fdrop those run in full, so the whole
            # column is computed (masked weights are zero, hence so is their dlogits)
            _lib.call("luxhip_attention_softmax_bwd", current_stream(), softmax_out.code, S, L, L * H * B, int(tri), dp.ptr,
                      softmax_out.ptr, scale_inv, dlogits.ptr)
        dq = DeviceArray(q.shape, dt)
        _bmm_strided(False, False, E, L, S, bdims, k, lk.st, (0, lk.sh, lk.sb), dlogits, S, sC, dq, lq.st,
                     (lq.sh, lq.sh * r, lq.sb), 2 if tri else 0)

        def kv_grad(like, lay, A, lda, sA, Bm):
            # (rows of `like`) x S = A (rows x L) * Bm' (L x S), one product per head; the heads that share
            # a key/value group are summed afterwards (pullback of repeat_inner_gqa)
            full = DeviceArray(((r,) if r > 1 else ()) + tuple(like.shape), dt)
            _bmm_strided(False, True, lay.E, S, L, bdims, A, lda, sA, Bm, S, sC, full, lay.st,
                         (like.size if r > 1 else 0, lay.sh, lay.sb), 3 if tri else 0)
            if r == 1:
                return full
            red = DeviceArray(like.shape, dt)
            _lib.call("luxhip_batch_sum", current_stream(), red.code, like.size, r, full.ptr, red.ptr)
            return red

        dv = kv_grad(v, lv, d_out, Ev * H, so, probs)
        dk = kv_grad(k, lk, q, lq.st, (lq.sh, lq.sh * r, lq.sb), dlogits)
        return dq, dk, dv

    return (out, probs), back


# ------------------------------------------------------------------------------- batchnorm
def batchnorm(x: DeviceArray, scale, bias, running_mean, running_var, training, act: str = "identity",
              momentum: float = 0.1, epsilon: Optional[float] = None):
    """`batchnorm(x, scale, bias, running_mean, running_var, training, σ, momentum, epsilon)`
    (api/batchnorm.jl:31-55): returns `(y, {"running_mean": .., "running_var": ..})`."""
    y, stats, _ = _batchnorm_fwd(x, scale, bias, running_mean, running_var, bool(training), act, momentum, epsilon, False)
    return y, stats


def _batchnorm_fwd(x, scale, bias, rmean, rvar, training, act, momentum, epsilon, save):
    dt = _same_dtype(x, scale, bias, rmean, rvar)
    I, Cc, N = _icn(x)
    for v in (scale, bias, rmean, rvar):
        if v is not None and (v.ndim != 1 or v.shape[0] != Cc):
            raise ArgumentError("Invalid Dimensions!")      # get_norm_reshape_dims, impl/normalization.jl:178-185
    if (scale is None) != (bias is None):
        raise ArgumentError("scale and bias must be given together")
    if epsilon is None:
        epsilon = default_epsilon(dt)
    y = DeviceArray(x.shape, dt)
    upd = training and rmean is not None
    rm_out = DeviceArray((Cc,), dt) if upd else None
    rv_out = DeviceArray((Cc,), dt) if upd else None
    sm = StatArray(Cc) if save else None
    si = StatArray(Cc) if save else None
    _lib.call("luxhip_batchnorm_fwd", current_stream(), x.code, _act_id(act), I, Cc, N, x.ptr, _p(scale), _p(bias),
              _p(rmean), _p(rvar), int(training), float(momentum), float(epsilon), y.ptr, _p(rm_out), _p(rv_out),
              _p(sm), _p(si))
    stats = {"running_mean": rm_out if upd else rmean, "running_var": rv_out if upd else rvar}
    return y, stats, (sm, si, float(epsilon))


def rrule_batchnorm(x, scale, bias, running_mean, running_var, training, act="identity", momentum=0.1, epsilon=None):
    """Whole-op rrule (precedent: ext/cuDNNExt/cuDNNExt.jl:26-54): ((y, stats), Δ -> (∂x, ∂γ, ∂β))."""
    training = bool(training)
    y, stats, (sm, si, eps) = _batchnorm_fwd(x, scale, bias, running_mean, running_var, training, act, momentum, epsilon, True)
    I, Cc, N = _icn(x)
    from_batch = training or running_mean is None
    aid = _act_id(act)

    def back(delta: DeviceArray):
        dx = DeviceArray(x.shape, x.dtype)
        dg = None if scale is None else DeviceArray((Cc,), x.dtype)
        db = None if bias is None else DeviceArray((Cc,), x.dtype)
        _lib.call("luxhip_batchnorm_bwd", current_stream(), x.code, aid, I, Cc, N, delta.ptr, x.ptr, _p(scale), _p(bias),
                  sm.ptr, si.ptr, int(from_batch), dx.ptr, _p(dg), _p(db))
        return dx, dg, db

    return (y, stats), back


# ------------------------------------------------------------------------------- groupnorm
def _check_groupnorm(x, scale, bias, groups):
    Cc = x.shape[-2]
    if scale is not None or bias is not None:
        if scale is None or bias is None or scale.shape[0] != bias.shape[0] or bias.shape[0] != Cc:
            raise ArgumentError("Length of `scale` and `bias` must be equal to the number of channels "
                                "((N - 1) dim of the input array).")
    if Cc % groups != 0:
        raise ArgumentError(f"Number of channels {Cc} must be divisible by the number of groups {groups}.")


def groupnorm(x: DeviceArray, scale, bias, groups: int, act: str = "identity", epsilon: Optional[float] = None):
    """`groupnorm(x, scale, bias, groups, σ, epsilon)` (api/groupnorm.jl:26-39)."""
    return _groupnorm_fwd(x, scale, bias, groups, act, epsilon, False)[0]


def _groupnorm_fwd(x, scale, bias, groups, act, epsilon, save):
    if x.ndim < 2:
        raise ArgumentError("groupnorm needs at least 2 dimensions")
    _check_groupnorm(x, scale, bias, groups)
    dt = _same_dtype(x, scale, bias)
    if epsilon is None:
        epsilon = default_epsilon(dt)
    I, Cc, N = _icn(x)
    y = DeviceArray(x.shape, dt)
    sm = StatArray(groups * N) if save else None
    si = StatArray(groups * N) if save else None
    _lib.call("luxhip_groupnorm_fwd", current_stream(), x.code, _act_id(act), I, Cc, groups, N, x.ptr, _p(scale), _p(bias),
              float(epsilon), y.ptr, _p(sm), _p(si))
    return y, (sm, si)


def rrule_groupnorm(x, scale, bias, groups, act="identity", epsilon=None):
    """CRC.rrule(groupnorm_affine_normalize_internal) + mean_var rrule (impl/groupnorm.jl:349-404,
    impl/common_ops.jl:45-61): (y, Δ -> (∂x, ∂γ, ∂β))."""
    y, (sm, si) = _groupnorm_fwd(x, scale, bias, groups, act, epsilon, True)
    I, Cc, N = _icn(x)
    aid = _act_id(act)

    def back(delta):
        dx = DeviceArray(x.shape, x.dtype)
        dg = None if scale is None else DeviceArray((Cc,), x.dtype)
        db = None if bias is None else DeviceArray((Cc,), x.dtype)
        _lib.call("luxhip_groupnorm_bwd", current_stream(), x.code, aid, I, Cc, groups, N, delta.ptr, x.ptr, _p(scale),
                  _p(bias), sm.ptr, si.ptr, dx.ptr, _p(dg), _p(db))
        return dx, dg, db

    return y, back


# ------------------------------------------------------------------------------- instancenorm
def _instancenorm_fwd(x, scale, bias, rmean, rvar, training, act, momentum, epsilon, save):
    if x.ndim <= 2:
        raise AssertionError(f"`ndims(x) = {x.ndim}` must be at least > 2.")      # api/instancenorm.jl:75-78
    dt = _same_dtype(x, scale, bias, rmean, rvar)
    I, Cc, N = _icn(x)
    for v in (scale, bias, rmean, rvar):
        if v is not None and (v.ndim != 1 or v.shape[0] != Cc):
            raise ArgumentError("Invalid Dimensions!")      # get_norm_reshape_dims, impl/normalization.jl:178-185
    if (scale is None) != (bias is None) or (rmean is None) != (rvar is None):
        raise ArgumentError("scale/bias and running_mean/running_var must be given in pairs")
    if epsilon is None:
        epsilon = default_epsilon(dt)
    if not training and rmean is not None:
        # the running statistics stand in for every sample's statistics: the inference batchnorm
        # kernels compute exactly that (impl/normalization.jl:122-127)
        y, stats, saved = _batchnorm_fwd(x, scale, bias, rmean, rvar, False, act, 0.0, epsilon, save)
        return y, stats, ("running",) + tuple(saved)
    upd = training and rmean is not None
    if upd and x.size:
        # one launch: the groupnorm forward kernel with G = C, whose workgroups also update the running statistics
        y = DeviceArray(x.shape, dt)
        sm, si = StatArray(Cc * N), StatArray(Cc * N)
        rm_out, rv_out = DeviceArray((Cc,), dt), DeviceArray((Cc,), dt)
        _lib.call("luxhip_instancenorm_fwd", current_stream(), x.code, _act_id(act), I, Cc, N, x.ptr, _p(scale), _p(bias),
                  float(epsilon), y.ptr, sm.ptr, si.ptr, float(momentum), rmean.ptr, rvar.ptr, rm_out.ptr, rv_out.ptr)
        return y, {"running_mean": rm_out, "running_var": rv_out}, ("sample", sm, si, float(epsilon))
    y, (sm, si) = _groupnorm_fwd(x, scale, bias, Cc, act, epsilon, save or upd)
    stats = {"running_mean": rmean, "running_var": rvar}
    if upd:
        rm_out, rv_out = DeviceArray((Cc,), dt), DeviceArray((Cc,), dt)
        _lib.call("luxhip_instancenorm_running_stats", current_stream(), x.code, I, Cc, N, sm.ptr, si.ptr, float(epsilon),
                  float(momentum), rmean.ptr, rvar.ptr, rm_out.ptr, rv_out.ptr)
        stats = {"running_mean": rm_out, "running_var": rv_out}
    return y, stats, ("sample", sm, si, float(epsilon))


def instancenorm(x: DeviceArray, scale, bias, running_mean, running_var, training, act: str = "identity",
                 momentum: float = 0.1, epsilon: Optional[float] = None):
    """`instancenorm(x, scale, bias, running_mean, running_var, training, σ, momentum, epsilon)`
    (api/instancenorm.jl:45-73): statistics per channel and sample over the leading dims; returns
    `(y, {"running_mean": .., "running_var": ..})`.  The legacy form without running statistics
    (:33-43) is `instancenorm(x, scale, bias, None, None, training, σ)`."""
    y, stats, _ = _instancenorm_fwd(x, scale, bias, running_mean, running_var, bool(training), act, momentum, epsilon, False)
    return y, stats


def rrule_instancenorm(x, scale, bias, running_mean, running_var, training, act="identity", momentum=0.1, epsilon=None):
    """((y, stats), Δ -> (∂x, ∂γ, ∂β)): the pullback of the generic `normalization`
    (impl/normalization.jl:143-165) with reduce dims 1..N-2; running statistics are constants."""
    y, stats, saved = _instancenorm_fwd(x, scale, bias, running_mean, running_var, bool(training), act, momentum, epsilon, True)
    I, Cc, N = _icn(x)
    aid = _act_id(act)

    def back(delta: DeviceArray):
        dx = DeviceArray(x.shape, x.dtype)
        dg = None if scale is None else DeviceArray((Cc,), x.dtype)
        db = None if bias is None else DeviceArray((Cc,), x.dtype)
        if saved[0] == "running":
            _lib.call("luxhip_batchnorm_bwd", current_stream(), x.code, aid, I, Cc, N, delta.ptr, x.ptr, _p(scale), _p(bias),
                      saved[1].ptr, saved[2].ptr, 0, dx.ptr, _p(dg), _p(db))
        else:
            _lib.call("luxhip_groupnorm_bwd", current_stream(), x.code, aid, I, Cc, Cc, N, delta.ptr, x.ptr, _p(scale),
                      _p(bias), saved[1].ptr, saved[2].ptr, dx.ptr, _p(dg), _p(db))
        return dx, dg, db

    return (y, stats), back


# ------------------------------------------------------------------------------- layernorm
COLON = ":"                 # Julia's `Colon()` as a `dims` argument: every dim
DEFAULT_DIMS = "1:(N-1)"


def _layernorm_geometry(x, scale, bias, dims):
    """Returns (L, R, channel_view): statistics run over the L elements of the leading dims, R
    columns.  channel_view is None when scale/bias span exactly the normalised dims (one fused
    kernel), else the (I, C, N) view of x in which the expanded scale/bias vary along C only (the
    affine part then runs as a per-channel pass after the normalisation).  Other layouts raise
    Unsupported (the host would fall back to the generic broadcast path, impl/layernorm.jl:3-14)."""
    if scale is None and bias is None and dims is None:
        raise ArgumentError("`dims` must be passed explicitly if `scale` and `bias` are `nothing`")
    if (scale is None) != (bias is None):
        raise ArgumentError("scale and bias must be given together")
    nd = x.ndim
    pshape = None if scale is None else tuple(scale.shape)
    if scale is not None and tuple(bias.shape) != pshape:
        raise DimensionMismatch("scale and bias must have the same shape")
    if dims is None:
        # compute_layernorm_dims / expand_layernorm_dims (impl/layernorm.jl:21-28,40-46): dims = 1:(N - M),
        # parameters reshaped to (size(γ)..., 1, ..., 1)
        assert nd > scale.ndim, "`x` must have more dimensions than `scale` and `bias` when `dims` is `nothing`"
        dims = tuple(range(1, nd - scale.ndim + 1))
        pshape = pshape + (1,) * (nd - scale.ndim)
    elif isinstance(dims, str) and dims == COLON:
        dims = tuple(range(1, nd + 1))
    elif isinstance(dims, str) and dims == DEFAULT_DIMS:
        dims = tuple(range(1, nd))
    if isinstance(dims, int):
        dims = (dims,)
    dims = tuple(sorted(dims))
    if dims != tuple(range(1, len(dims) + 1)):
        raise _lib.Unsupported(_lib.UNSUPPORTED, f"layernorm over non-leading dims {dims}")
    k = len(dims)
    L = 1
    for d in dims:
        L *= x.shape[d - 1]
    R = x.size // max(L, 1)
    if scale is None:
        return L, R, None
    if len(pshape) != nd:
        raise ArgumentError("scale and bias must have the same number of dimensions as x when dims is given")
    if any(g not in (1, sx) for g, sx in zip(pshape, x.shape)):
        raise DimensionMismatch(f"scale/bias of shape {pshape} do not broadcast against x {x.shape}")
    if pshape == tuple(x.shape[:k]) + (1,) * (nd - k):
        return L, R, None
    # the per-channel pass wants the parameters to vary along one contiguous run of dims [a, b); parameters
    # with gaps in between (e.g. (3, 1, 3, 1)) are first repeated along the gaps (_expand_parameters)
    varying = [d for d in range(nd) if pshape[d] != 1]
    a, b = (varying[0], varying[-1] + 1) if varying else (nd, nd)
    prod = lambda t: int(np.prod(t, dtype=np.int64)) if len(t) else 1
    return L, R, (prod(x.shape[:a]), prod(x.shape[a:b]), prod(x.shape[b:]))


def _expand_parameters(x, pshape, *params):
    """Parameters of (expanded) shape `pshape` repeated along the dims that lie between the first and the
    last dim they vary along, and the function that sums a gradient of the repeated shape back."""
    nd = x.ndim
    varying = [d for d in range(nd) if pshape[d] != 1]
    a, b = (varying[0], varying[-1] + 1) if varying else (nd, nd)
    gaps = [d for d in range(a, b) if pshape[d] == 1 and x.shape[d] != 1]
    if not gaps:
        return params, (lambda g: g)
    full = tuple(x.shape[d] if a <= d < b else 1 for d in range(nd))
    ones = DeviceArray.from_numpy(np.ones(full, np.float32), x.dtype)
    expanded = tuple(dropout_dot_mul(ones, p_.reshape(pshape)) for p_ in params)

    def reduce(g):
        shape = list(full)
        for d in gaps:                       # sum over dim d: (A, B, C) x ones(B) -> (A, 1, C)
            A, B = int(np.prod(shape[:d], dtype=np.int64)), shape[d]
            Cc = int(np.prod(shape[d + 1:], dtype=np.int64))
            vec = DeviceArray.from_numpy(np.ones((B, 1, 1), np.float32), x.dtype)
            g = batched_matmul(g.reshape(A, B, Cc), vec)
            shape[d] = 1
        return g.reshape(pshape)

    return expanded, reduce


def layernorm(x: DeviceArray, scale, bias, act: str = "identity", dims=DEFAULT_DIMS, epsilon: Optional[float] = None):
    """`layernorm(x, scale, bias, σ, dims, epsilon)` (api/layernorm.jl:32-43).  `dims` uses
    Julia's 1-based numbering; the default is 1:(N-1); `None` is Julia's `nothing` (dims inferred
    from the parameters' rank), `COLON` is `Colon()`."""
    return _layernorm_fwd(x, scale, bias, act, dims, epsilon, False)[0]


def _layernorm_fwd(x, scale, bias, act, dims, epsilon, save):
    L, R, view = _layernorm_geometry(x, scale, bias, dims)
    dt = _same_dtype(x, scale, bias)
    if epsilon is None:
        epsilon = default_epsilon(dt)
    y = DeviceArray(x.shape, dt)
    sm = StatArray(R) if save else None
    si = StatArray(R) if save else None
    if view is None:
        _lib.call("luxhip_layernorm_fwd", current_stream(), x.code, _act_id(act), L, R, x.ptr, _p(scale), _p(bias),
                  float(epsilon), y.ptr, _p(sm), _p(si))
        return y, (sm, si, L, R, None)
    # parameters that vary along other dims than the normalised ones: x̂ first, then the per-channel
    # affine transform and activation as a batchnorm in inference mode with mean 0, variance 1, ε = 0
    _lib.call("luxhip_layernorm_fwd", current_stream(), x.code, 0, L, R, x.ptr, None, None, float(epsilon), y.ptr, _p(sm), _p(si))
    I, Cc, Nn = view
    pshape = tuple(scale.shape) + (1,) * (x.ndim - scale.ndim)
    (gam, bet), reduce = _expand_parameters(x, pshape, scale, bias)
    zeros = DeviceArray.from_numpy(np.zeros(Cc, np.float32), dt)
    ones = DeviceArray.from_numpy(np.ones(Cc, np.float32), dt)
    args = (y.reshape(I, Cc, Nn), gam.reshape(Cc), bet.reshape(Cc), zeros, ones, False, act, 0.1, 0.0)
    if save:
        (out, _), bn_back = rrule_batchnorm(*args)

        def affine_back(delta3):
            dxhat, dg, db = bn_back(delta3)
            return dxhat, reduce(dg), reduce(db)
    else:
        (out, _), affine_back = batchnorm(*args), None
    return out.reshape(x.shape), (sm, si, L, R, affine_back)


def rrule_layernorm(x, scale, bias, act="identity", dims=DEFAULT_DIMS, epsilon=None):
    """Pullback of layernorm: the chain AD derives from impl/normalization.jl:11-17 and the
    mean_var rrule (impl/common_ops.jl:45-61), as one fused device pass (two when the parameters
    vary along other dims than the normalised ones)."""
    y, (sm, si, L, R, affine_back) = _layernorm_fwd(x, scale, bias, act, dims, epsilon, True)
    aid = _act_id(act)

    def back(delta):
        dx = DeviceArray(x.shape, x.dtype)
        if affine_back is not None:
            dxhat, dg, db = affine_back(delta.reshape(dxhat_shape))
            _lib.call("luxhip_layernorm_bwd", current_stream(), x.code, 0, L, R, dxhat.ptr, x.ptr, None, None,
                      sm.ptr, si.ptr, dx.ptr, None, None)
            return dx, dg.reshape(scale.shape), db.reshape(bias.shape)
        dg = None if scale is None else DeviceArray(scale.shape, x.dtype)
        db = None if bias is None else DeviceArray(bias.shape, x.dtype)
        _lib.call("luxhip_layernorm_bwd", current_stream(), x.code, aid, L, R, delta.ptr, x.ptr, _p(scale), _p(bias),
                  sm.ptr, si.ptr, dx.ptr, _p(dg), _p(db))
        return dx, dg, db

    if affine_back is not None:
        dxhat_shape = _layernorm_geometry(x, scale, bias, dims)[2]
    return y, back


# ------------------------------------------------------------------------------- conv
@dataclass
class DenseConvDims:
    """The fields of NNlib.DenseConvDims this path consumes (1, 2 or 3 spatial dims: x (W, C, N),
    (W, H, C, N) or (W, H, D, C, N)).  padding = (w_lo, w_hi[, h_lo, h_hi[, d_lo, d_hi]]);
    flipkernel=False is true convolution.  Three spatial dims run as the two-dimensional problem
    `inner` on the depth-unfolded input (kD*C channels, Dout*N samples)."""
    x_shape: Tuple[int, ...]
    w_shape: Tuple[int, ...]
    stride: Tuple[int, ...] = 1
    padding: Tuple[int, ...] = 0
    dilation: Tuple[int, ...] = 1
    groups: int = 1
    flipkernel: bool = False
    _c: Optional[_lib.ConvDimsStruct] = field(default=None, repr=False, compare=False)

    def __post_init__(self):
        self.x_shape, self.w_shape = tuple(self.x_shape), tuple(self.w_shape)
        if len(self.x_shape) != len(self.w_shape) or len(self.x_shape) not in (3, 4, 5):
            raise _lib.Unsupported(_lib.UNSUPPORTED, "only 1, 2 or 3 spatial dimensions are handled on the device")
        self.spatial = len(self.x_shape) - 2
        one = self.spatial == 1           # (W, C, N): the same memory as (W, 1, C, N), a 2-d problem of height 1
        if isinstance(self.stride, int):
            self.stride = (self.stride,) * self.spatial
        if isinstance(self.dilation, int):
            self.dilation = (self.dilation,) * self.spatial
        if isinstance(self.padding, int):
            self.padding = (self.padding,) * (2 * self.spatial)
        elif len(self.padding) == self.spatial:
            self.padding = tuple(p for q in self.padding for p in (q, q))
        self.stride, self.dilation, self.padding = tuple(self.stride), tuple(self.dilation), tuple(self.padding)
        if len(self.stride) != self.spatial or len(self.dilation) != self.spatial or len(self.padding) != 2 * self.spatial:
            raise DimensionMismatch("stride, dilation and padding must match the number of spatial dimensions")
        self.inner = None
        if self.spatial == 3:
            W, H, D, Cin, N = self.x_shape
            kW, kH, kD, Cg, Cout = self.w_shape
            if Cg * self.groups != Cin:
                raise DimensionMismatch(f"input channels {Cin} != weight channels {Cg} x groups {self.groups}")
            dout = self.out_spatial[2]
            self.inner = DenseConvDims((W, H, kD * Cin, dout * N), (kW, kH, kD * Cg, Cout), self.stride[:2], self.padding[:4],
                                       self.dilation[:2], self.groups, self.flipkernel)
            return
        stride, dil, pad = ((self.stride + (1,), self.dilation + (1,), self.padding + (0, 0)) if one
                            else (self.stride, self.dilation, self.padding))
        W, H, Cin, N = (self.x_shape[0], 1) + self.x_shape[1:] if one else self.x_shape
        kW, kH, Cg, Cout = (self.w_shape[0], 1) + self.w_shape[1:] if one else self.w_shape
        if Cg * self.groups != Cin:
            raise DimensionMismatch(f"input channels {Cin} != weight channels {Cg} x groups {self.groups}")
        if Cout % self.groups != 0:
            raise DimensionMismatch("output channels must be divisible by groups")
        self._c = _lib.ConvDimsStruct(W, H, Cin, N, kW, kH, Cout, stride[0], stride[1], *pad,
                                      dil[0], dil[1], self.groups, int(self.flipkernel))

    @property
    def out_spatial(self):
        return tuple((self.x_shape[d] + self.padding[2 * d] + self.padding[2 * d + 1]
                      - self.dilation[d] * (self.w_shape[d] - 1) - 1) // self.stride[d] + 1 for d in range(self.spatial))

    @property
    def y_shape(self):
        return self.out_spatial + (self.w_shape[-1], self.x_shape[-1])


def _check_conv(weight, x, b, cdims):
    if tuple(x.shape) != cdims.x_shape or tuple(weight.shape) != cdims.w_shape:
        raise DimensionMismatch(f"x {x.shape} / weight {weight.shape} do not match cdims {cdims.x_shape} / {cdims.w_shape}")
    if b is not None:
        assert b.ndim == 1 and b.shape[0] == cdims.w_shape[-1], "length(bias) must equal the number of output channels"


def fused_conv_bias_activation(act: str, weight: DeviceArray, x: DeviceArray, b, cdims: DenseConvDims) -> DeviceArray:
    """`fused_conv_bias_activation(σ, weight, x, b, cdims)` (api/conv.jl:30-38)."""
    _check_conv(weight, x, b, cdims)
    if _is_closure(act):
        return _closure_rule(act, fused_conv_bias_activation("identity", weight, x, b, cdims))[0]
    (weight, x, b), _ = _promote(weight, x, b)
    dt = _same_dtype(weight, x, b)
    if cdims.inner is not None:
        return _from_inner_output(cdims, fused_conv_bias_activation(act, _inner_weight(cdims, weight), _depth_unfold(cdims, x), b,
                                                                    cdims.inner))
    y = DeviceArray(cdims.y_shape, dt)
    _lib.call("luxhip_conv_fwd", current_stream(), y.code, _act_id(act), C.byref(cdims._c), x.ptr, weight.ptr, _p(b),
              y.ptr, None, None)
    return y


# Three spatial dims: the depth-unfolded two-dimensional problem.
def _depth_args(cdims, N):
    W, H, D, Cin, _ = cdims.x_shape
    return (W * H, D, Cin, N, cdims.w_shape[2], cdims.out_spatial[2], cdims.stride[2], cdims.padding[4], cdims.dilation[2],
            int(cdims.flipkernel))


def _depth_unfold(cdims, x):
    xu = DeviceArray(cdims.inner.x_shape, x.dtype)
    _lib.call("luxhip_conv_depth_unfold", current_stream(), x.code, *_depth_args(cdims, x.shape[-1]), x.ptr, xu.ptr)
    return xu


def _depth_fold(cdims, dxu):
    dx = DeviceArray(cdims.x_shape, dxu.dtype)
    _lib.call("luxhip_conv_depth_fold", current_stream(), dx.code, *_depth_args(cdims, cdims.x_shape[-1]), dxu.ptr, dx.ptr)
    return dx


def _inner_weight(cdims, weight):
    return weight.reshape(cdims.inner.w_shape)        # the same memory: channel kd + kD*c


def _from_inner_output(cdims, y2):
    """(OW, OH, Cout, Dout*N) of the inner problem -> (OW, OH, Dout, Cout, N)."""
    ow, oh, dout = cdims.out_spatial
    cout, n = cdims.w_shape[-1], cdims.x_shape[-1]
    y = DeviceArray((ow, oh, dout, cout, n), y2.dtype)
    _lib.call("luxhip_swap_middle_dims", current_stream(), y.code, ow * oh, cout, dout, n, y2.ptr, y.ptr)
    return y


def _to_inner_output(cdims, dy):
    """(OW, OH, Dout, Cout, N) -> (OW, OH, Cout, Dout*N)."""
    ow, oh, dout = cdims.out_spatial
    cout, n = cdims.w_shape[-1], cdims.x_shape[-1]
    d2 = DeviceArray((ow, oh, cout, dout * n), dy.dtype)
    _lib.call("luxhip_swap_middle_dims", current_stream(), dy.code, ow * oh, dout, cout, n, dy.ptr, d2.ptr)
    return d2


def rrule_fused_conv_bias_activation(act: str, weight, x, b, cdims: DenseConvDims):
    """CRC.rrule(fused_conv) + ∇fused_conv (impl/conv.jl:204-275): (y, Δ -> (∂w, ∂x, ∂b))."""
    _check_conv(weight, x, b, cdims)
    if _is_closure(act):                      # impl/conv.jl:271-275
        z, back_z = rrule_fused_conv_bias_activation("identity", weight, x, b, cdims)
        y, back_act = _closure_rule(act, z)
        return y, (lambda delta: back_z(back_act(delta)))
    (pw, px, pb), orig = _promote(weight, x, b)
    if orig is not None:
        return _promoted_rule(lambda *a: rrule_fused_conv_bias_activation(act, *a, cdims), orig, pw, px, pb)
    aid = _act_id(act)
    dt = _same_dtype(weight, x, b)
    if cdims.inner is not None:
        y2, back2 = rrule_fused_conv_bias_activation(act, _inner_weight(cdims, weight), _depth_unfold(cdims, x), b, cdims.inner)

        def back3(delta):
            dw2, dxu, db = back2(_to_inner_output(cdims, delta))
            return dw2.reshape(cdims.w_shape), _depth_fold(cdims, dxu), db

        return _from_inner_output(cdims, y2), back3
    y = DeviceArray(cdims.y_shape, dt)
    pre = DeviceArray(cdims.y_shape, dt) if aid in _NEEDS_PRE else None
    xt = DeviceArray(x.shape, dt)      # the channel-contiguous copy of x, kept for the filter gradient
    _lib.call("luxhip_conv_fwd", current_stream(), y.code, aid, C.byref(cdims._c), x.ptr, weight.ptr, _p(b), y.ptr, _p(pre),
              xt.ptr)

    def back(delta):
        dw = DeviceArray(weight.shape, dt)
        dx = DeviceArray(x.shape, dt)
        db = None if b is None else DeviceArray(b.shape, dt)
        dz = None if aid == 0 else DeviceArray(cdims.y_shape, dt)
        _lib.call("luxhip_fused_conv_bwd", current_stream(), y.code, aid, C.byref(cdims._c), delta.ptr, y.ptr, _p(pre),
                  x.ptr, weight.ptr, _p(dz), dw.ptr, dx.ptr, _p(db), xt.ptr)
        return dw, dx, db

    return y, back


def conv(x, weight, cdims):
    """`Impl.conv(x, weight, cdims)` (impl/conv.jl:62-72)."""
    return fused_conv_bias_activation("identity", weight, x, None, cdims)


def conv_data_grad(dy, weight, cdims):
    """`Impl.∇conv_data` (impl/conv.jl:128-131)."""
    if cdims.inner is not None:
        return _depth_fold(cdims, conv_data_grad(_to_inner_output(cdims, dy), _inner_weight(cdims, weight), cdims.inner))
    dx = DeviceArray(cdims.x_shape, dy.dtype)
    _lib.call("luxhip_conv_bwd_data", current_stream(), dy.code, C.byref(cdims._c), dy.ptr, weight.ptr, dx.ptr)
    return dx


def conv_filter_grad(x, dy, cdims):
    """`Impl.∇conv_filter` (impl/conv.jl:133-136)."""
    if cdims.inner is not None:
        return conv_filter_grad(_depth_unfold(cdims, x), _to_inner_output(cdims, dy), cdims.inner).reshape(cdims.w_shape)
    dw = DeviceArray(cdims.w_shape, x.dtype)
    _lib.call("luxhip_conv_bwd_filter", current_stream(), x.code, C.byref(cdims._c), x.ptr, dy.ptr, dw.ptr)
    return dw


# ------------------------------------------------------------------------------- Zygote.pullback analogue
_RRULES = {
    bias_activation: rrule_bias_activation,
    fused_dense_bias_activation: rrule_fused_dense_bias_activation,
    batchnorm: rrule_batchnorm,
    groupnorm: rrule_groupnorm,
    instancenorm: rrule_instancenorm,
    fast_activation: rrule_fast_activation,
    dropout: rrule_dropout,
    batched_matmul: rrule_batched_matmul,
    scaled_dot_product_attention: rrule_scaled_dot_product_attention,
    alpha_dropout: rrule_alpha_dropout,
    layernorm: rrule_layernorm,
    fused_conv_bias_activation: rrule_fused_conv_bias_activation,
}


def pullback(f, *args, **kwargs):
    """`y, back = pullback(f, args...)`; `back(Δ)` returns the tangents of the array
    arguments in the order the rrule lists them."""
    try:
        rule = _RRULES[f]
    except KeyError:
        raise TypeError(f"no rrule registered for {f}") from None
    return rule(*args, **kwargs)
