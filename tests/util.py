"""Shared helpers of the GPU parity tests."""
import numpy as np

from oracle import luxlib_oracle as O

# Parity bars stated by the benchmark definition: fp32 within rel 1e-5, bf16 within rel 1e-2
# of the CPU restatement on identical inputs.  "rel" is applied per element against
# |want| + rms(want): a pure per-element relative bound is meaningless where the exact
# result crosses zero.
REL = {"f32": 1e-5, "bf16": 1e-2}


# every comparison made by assert_close in this process: (what, dtype, rel, worst error as a multiple of |want| + rms,
# worst error of the float32 oracle in the same unit or None, elements compared)
ERROR_LOG = []


def assert_close(got, want, dtype, what="", rel=None, scale=0.0, want32=None):
    """`scale`: magnitude of the terms the result is a sum of, for results that are small
    through cancellation (gradients of normalisations); the absolute floor is
    rel * max(rms(want), scale).
    `want32`: the same oracle evaluated in float32 arithmetic (what a CPU run of the reference
    produces); where the problem is so ill-conditioned that fp32 arithmetic itself misses the
    exact answer by more than the bar, the allowance grows to 4x that fp32 error.
    Returns the worst error found, as a multiple of |want| + max(rms(want), scale) (the unit `rel` is in)."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, f"{what}: shape {got.shape} != {want.shape}"
    if want.size == 0:
        return 0.0
    rel = REL[dtype] if rel is None else rel
    rms = max(float(np.sqrt(np.mean(want * want))), float(scale))
    unit = np.abs(want) + rms + 1e-30
    bound = rel * unit
    err32 = None
    if want32 is not None:
        d32 = np.abs(np.asarray(want32, dtype=np.float64) - want)
        bound = np.maximum(bound, 4.0 * d32)
        err32 = float(np.max(d32 / unit))
    err = np.abs(got - want)
    worst = float(np.max(err / unit)) if np.isfinite(err).all() else float("inf")
    ERROR_LOG.append((what, dtype, rel, worst, err32, int(want.size)))
    bad = ~(err <= bound)
    if bad.any():
        i = np.unravel_index(np.argmax(err / bound), err.shape)
        raise AssertionError(
            f"{what}: {bad.sum()}/{bad.size} elements outside rel {rel:g}; worst at {i}: got {got[i]!r} want {want[i]!r} "
            f"(err {err[i]:.3e}, bound {bound[i]:.3e})")
    return worst


def host_inputs(dtype, *arrays):
    """fp32 host arrays as the device will see them (bf16: rounded to representable values)."""
    out = []
    for a in arrays:
        if a is None:
            out.append(None)
            continue
        a = np.asarray(a, dtype=np.float32)
        out.append(O.round_to_bf16(a) if dtype == "bf16" else a)
    return out


def dev(lux, a, dtype):
    return None if a is None else lux.DeviceArray.from_numpy(a, dtype)


def f64(a):
    return None if a is None else np.asarray(a, dtype=np.float64)


def rms(a):
    a = np.asarray(a, dtype=np.float64)
    return float(np.sqrt(np.mean(a * a))) if a.size else 0.0


def stable_seed(*parts):
    """Seed that does not depend on Python's per-process string hashing."""
    import zlib
    return zlib.crc32(repr(parts).encode()) & 0x7FFFFFFF
