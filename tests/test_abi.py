"""The C-ABI shared library loads (no GPU needed) and exports every symbol include/luxhip.h
declares; the ctypes prototypes cover exactly the same set; calls fail loudly without a
device instead of falling back to anything."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "luxhip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(luxhip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(lux):
    lib = lux._lib.load()
    syms = declared_symbols()
    assert len(syms) >= 30
    for s in syms:
        assert hasattr(lib, s), f"{s} is declared in include/luxhip.h but not exported by libluxhip.so"


def test_ctypes_prototypes_match_header(lux):
    declared = set(declared_symbols())
    bound = set(lux._lib.SIGNATURES) | {"luxhip_last_error"}
    assert declared == bound, (sorted(declared - bound), sorted(bound - declared))


def test_header_argument_counts_match_prototypes(lux):
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    for name, argtypes in lux._lib.SIGNATURES.items():
        m = re.search(r"\b" + name + r"\s*\(([^;]*?)\)\s*;", text, flags=re.S)
        assert m, name
        args = m.group(1).strip()
        n = 0 if args in ("", "void") else len(args.split(","))
        assert n == len(argtypes), f"{name}: header has {n} parameters, ctypes prototype {len(argtypes)}"


def test_ops_fail_loudly_without_init(lux):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present; this checks the no-device behaviour")
    lib = lux._lib.load()
    rc = lib.luxhip_bias_activation_fwd(None, 0, 1, 4, 4, 4, None, None, None, None)
    assert rc == lux._lib.NOT_INITIALIZED
    assert "luxhip_init" in lux._lib.last_error()
    with pytest.raises(lux.LuxHipError):
        lux.init(0)


def test_tuning_switches_validate_their_arguments(lux):
    """luxhip_set_option needs no device: unknown names and out-of-range values are rejected with a
    message, known switches are accepted and can be put back to their defaults."""
    with pytest.raises(lux.LuxHipError, match="unknown option"):
        lux.set_option("no_such_switch", 1)
    with pytest.raises(lux.LuxHipError, match="gemm_tile"):
        lux.set_option("gemm_tile", 7)
    with pytest.raises(lux.LuxHipError, match="gemm_pretranspose"):
        lux.set_option("gemm_pretranspose", 2)
    with pytest.raises(lux.LuxHipError, match="bn_spin_limit"):
        lux.set_option("bn_spin_limit", -1)
    for name, value in (("bn_resident", 0), ("bn_resident", 1), ("bn_spin_limit", 0), ("bn_spin_limit", 1 << 22),
                        ("gemm_tile", 82), ("gemm_tile", 0), ("conv_tile", 84), ("conv_tile", 0),
                        ("gemm_pretranspose", 0), ("gemm_pretranspose", 1)):
        lux.set_option(name, value)


def test_host_side_argument_checks_need_no_device(lux):
    """Shape errors are raised on the host before anything is launched
    (impl/matmul.jl:21-34, api/groupnorm.jl:40-64, api/bias_activation.jl:38-45)."""
    class Fake:
        def __init__(self, shape, dtype="f32"):
            self.shape, self.dtype, self.ndim, self.ptr = tuple(shape), dtype, len(shape), 0
    with pytest.raises(lux.DimensionMismatch):
        lux.fused_dense_bias_activation("relu", Fake((3, 4)), Fake((5, 2)), None)
    with pytest.raises(lux.DimensionMismatch):
        lux.fused_dense_bias_activation("relu", Fake((3, 4)), Fake((4, 2)), Fake((4,)))
    with pytest.raises(lux.ArgumentError):
        lux.groupnorm(Fake((4, 6, 2)), Fake((6,)), Fake((6,)), 4)
    with pytest.raises(lux.ArgumentError):
        lux.groupnorm(Fake((4, 6, 2)), Fake((5,)), Fake((5,)), 2)
    with pytest.raises(AssertionError):
        lux.bias_activation("relu", Fake((3, 4)), Fake((4,)))
    with pytest.raises(lux.ArgumentError):
        lux.layernorm(Fake((3, 4)), None, None, "identity", None)
    with pytest.raises(lux.DimensionMismatch):
        lux.DenseConvDims((8, 8, 4, 2), (3, 3, 3, 6))
    with pytest.raises(lux.Unsupported):
        lux.bias_activation("x^3", Fake((3, 4)), None)


def test_fastdiv_matches_integer_division():
    """The multiply-high division used for index math, restated on the host."""
    import random
    random.seed(1)

    def fastdiv(n, d):
        l = 0
        while (1 << l) < d:
            l += 1
        m = ((1 << 32) * ((1 << l) - d)) // d + 1
        m &= 0xFFFFFFFF
        t = (n * m) >> 32
        return ((t + n) & 0xFFFFFFFF) >> l

    ds = [1, 2, 3, 5, 7, 8, 64, 100, 255, 256, 257, 1024, 4096, 11008, 65535, 65536, 1 << 20, (1 << 31) - 1]
    ds += [random.randrange(1, 1 << 31) for _ in range(200)]
    for d in ds:
        ns = [0, 1, d - 1, d, d + 1, 2 * d - 1, 2 * d, (1 << 31) - 1, (1 << 31) - d] + \
             [random.randrange(0, 1 << 31) for _ in range(200)]
        for n in ns:
            if 0 <= n < (1 << 31):
                assert fastdiv(n, d) == n // d, (n, d)
