"""The C-ABI shared library loads (no GPU needed) and exports every symbol include/luxhip.h
declares; the ctypes prototypes cover exactly the same set; calls fail loudly without a
device instead of falling back to anything."""
import ctypes
import os
import re

import numpy as np

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


class _Fake:
    """An array stand-in for the host-side planning code (shapes only, nothing is launched)."""

    def __init__(self, shape, dtype="f32"):
        self.shape, self.dtype, self.ndim, self.ptr = tuple(shape), dtype, len(shape), 0
        self.size = int(np.prod(shape)) if len(shape) else 1


def test_layernorm_planning(lux):
    """Which dims are normalised and how the parameters are applied (impl/layernorm.jl:21-46)."""
    from lux_jl_amd import luxlib as L
    x = _Fake((3, 3, 2, 5))
    assert L._layernorm_geometry(x, None, None, L.DEFAULT_DIMS) == (18, 5, None)
    assert L._layernorm_geometry(x, None, None, L.COLON) == (90, 1, None)
    assert L._layernorm_geometry(x, _Fake((3, 3, 2, 1)), _Fake((3, 3, 2, 1)), (1, 2, 3)) == (18, 5, None)        # one fused kernel
    # the reference's test configurations: Colon() with (1, 1, C, 1), nothing with (1, 1, C) -> dims 1:1
    assert L._layernorm_geometry(x, _Fake((1, 1, 2, 1)), _Fake((1, 1, 2, 1)), L.COLON) == (90, 1, (9, 2, 5))
    assert L._layernorm_geometry(x, _Fake((1, 1, 2)), _Fake((1, 1, 2)), None) == (3, 30, (9, 2, 5))
    assert L._layernorm_geometry(x, _Fake((3, 1, 2, 1)), _Fake((3, 1, 2, 1)), L.COLON) == (90, 1, (1, 18, 5))    # a gap: repeated first
    with pytest.raises(lux.Unsupported):
        L._layernorm_geometry(x, None, None, (2, 3))
    with pytest.raises(lux.DimensionMismatch):
        L._layernorm_geometry(x, _Fake((2, 1, 1, 1)), _Fake((2, 1, 1, 1)), L.COLON)
    with pytest.raises(AssertionError):
        L._layernorm_geometry(_Fake((2, 3)), _Fake((2, 1)), _Fake((2, 1)), None)


def test_batched_matmul_planning(lux):
    """Where the matrices and the batching dims of batched_matmul's operands lie (impl/batched_mul.jl:2-58)."""
    from lux_jl_amd import luxlib as L
    op = L._BmmOperand(_Fake((3, 5, 2, 4)), 4, (2, 3), "x")           # generalized_bmm_tests.jl:36-58, left operand
    assert (op.F, op.K, op.free_major, op.ld, op.bext, op.bst) == (3, 4, True, 30, [5, 2], [3, 15])
    op = L._BmmOperand(_Fake((4, 5, 1, 5)), 1, (4, 3), "y")           # its right operand
    assert (op.F, op.K, op.free_major, op.ld, op.bext, op.bst) == (5, 4, False, 4, [5, 1], [20, 20])
    op = L._BmmOperand(_Fake((5, 4, 5, 1)), 2, None, "y")             # :8-22: contracted along dim 2, trailing batch dims
    assert (op.F, op.K, op.free_major, op.ld) == (5, 4, True, 5)
    with pytest.raises(lux.Unsupported):
        L._BmmOperand(_Fake((2, 3, 6, 7, 5)), 3, (1, 2, 5), "y")     # neither matrix dim contiguous
    with pytest.raises(lux.ArgumentError):
        L._BmmOperand(_Fake((2, 3, 4)), 2, (2,), "x")                 # the contracting dim among the batching dims


def test_conv_dims_with_three_spatial_dims(lux):
    cd = lux.DenseConvDims((7, 6, 8, 4, 2), (2, 3, 3, 2, 6), stride=(1, 2, 2), padding=(1, 0, 2, 1, 1, 2), dilation=(2, 1, 2), groups=2)
    assert cd.out_spatial == (6, 4, 4) and cd.y_shape == (6, 4, 4, 6, 2)
    inner = cd.inner                                                   # the two-dimensional problem on the unfolded input
    assert inner.x_shape == (7, 6, 3 * 4, 4 * 2) and inner.w_shape == (2, 3, 3 * 2, 6)
    assert inner.stride == (1, 2) and inner.padding == (1, 0, 2, 1) and inner.dilation == (2, 1) and inner.groups == 2
    assert inner.y_shape == (6, 4, 6, 4 * 2)
    with pytest.raises(lux.Unsupported):
        lux.DenseConvDims((4, 4, 4, 4, 2, 1), (2, 2, 2, 2, 2, 3))


# ----------------------------------------------------------------------------- the Julia glue file
JULIA_GLUE = os.path.join(ROOT, "lux.jl_amd", "julia", "LuxHIP.jl")


def header_prototypes():
    """name -> (return type, [parameter types]) of include/luxhip.h, as C type strings without parameter names."""
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    protos = {}
    for m in re.finditer(r"\b((?:const\s+)?[A-Za-z_0-9]+\s*\**)\s*\b(luxhip_[a-z0-9_]+)\s*\(([^;{}]*?)\)\s*;", text, flags=re.S):
        params = []
        for a in m.group(3).split(","):
            a = " ".join(a.split())
            if a in ("", "void"):
                continue
            t = re.sub(r"\b[A-Za-z_0-9]+$", "", a).strip()          # drop the parameter name
            params.append(t.replace(" *", "*"))
        protos[m.group(2)] = (" ".join(m.group(1).split()).replace(" *", "*"), params)
    return protos


def _matching_paren(text, i):
    """Index of the parenthesis closing the one at text[i] (Julia strings and comments in the glue file hold no
    unbalanced parentheses inside a ccall)."""
    depth = 0
    for j in range(i, len(text)):
        if text[j] == "(":
            depth += 1
        elif text[j] == ")":
            depth -= 1
            if depth == 0:
                return j
    raise ValueError("unbalanced parentheses")


def _split_top_level(s):
    out, depth, cur = [], 0, ""
    for ch in s:
        if ch in "({[":
            depth += 1
        elif ch in ")}]":
            depth -= 1
        if ch == "," and depth == 0:
            out.append(cur.strip())
            cur = ""
        else:
            cur += ch
    if cur.strip():
        out.append(cur.strip())
    return out


def julia_ccalls():
    """Every `ccall((:luxhip_x, libluxhip), Ret, (Types...,), args...)` of the glue file:
    (symbol, return type, [argument types], number of values passed, line)."""
    text = open(JULIA_GLUE).read()
    text = "\n".join(line if not line.lstrip().startswith("#") else "" for line in text.split("\n"))
    calls = []
    for m in re.finditer(r"ccall\(\(:(luxhip_[a-z0-9_]+),\s*libluxhip\)", text):
        start = text.index("(", m.start())
        end = _matching_paren(text, start)
        parts = _split_top_level(text[start + 1:end])
        ret, types = parts[1], parts[2]
        # Julia wants the type tuple spelled out in the call and takes no splatted values
        assert types.startswith("(") and types.endswith(")"), f"{m.group(1)}: the argument types must be a literal tuple, got `{types}`"
        assert not any(v.endswith("...") for v in parts[3:]), f"{m.group(1)}: a ccall cannot splat its arguments"
        calls.append((m.group(1), ret, _split_top_level(types[1:-1]), len(parts) - 3, text.count("\n", 0, m.start()) + 1))
    return calls


# which Julia ccall types may stand for a C parameter type
_JULIA_FOR_C = {
    "int": {"Cint"}, "int64_t": {"Int64", "Clonglong"}, "uint64_t": {"UInt64", "Culonglong"}, "size_t": {"Csize_t"},
    "double": {"Cdouble"}, "float": {"Cfloat"}, "const char*": {"Cstring", "Ptr{UInt8}", "Ptr{Cchar}"},
    "char*": {"Ptr{UInt8}", "Ptr{Cchar}"}, "luxhip_stream_t": {"Ptr{Cvoid}"}, "luxhip_event_t": {"Ptr{Cvoid}"},
    "luxhip_stream_t*": {"Ptr{Ptr{Cvoid}}"}, "luxhip_event_t*": {"Ptr{Ptr{Cvoid}}"}, "void**": {"Ptr{Ptr{Cvoid}}"},
    "void*": {"Ptr{Cvoid}"}, "const void*": {"Ptr{Cvoid}"}, "int*": {"Ptr{Cint}", "Ref{Cint}"},
    "int64_t*": {"Ptr{Int64}", "Ref{Int64}"}, "const int64_t*": {"Ptr{Int64}", "Ref{Int64}"},
    "double*": {"Ptr{Cdouble}", "Ref{Cdouble}"}, "float*": {"Ptr{Cfloat}", "Ptr{Cvoid}"}, "const float*": {"Ptr{Cfloat}", "Ptr{Cvoid}"},
    "const uint8_t*": {"Ptr{UInt8}", "Ptr{Cvoid}"}, "const luxhip_conv_dims_t*": {"Ptr{ConvDimsC}", "Ref{ConvDimsC}"},
}


def test_julia_glue_ccalls_match_the_header():
    """There is no Julia toolchain to run the glue file with, so the one check that needs none: every ccall names a
    symbol the header declares, passes as many values as it lists types, lists as many types as the C prototype has
    parameters, and each type is one that has the C parameter's size and meaning."""
    protos = header_prototypes()
    assert set(protos) == set(declared_symbols())
    calls = julia_ccalls()
    assert len(calls) >= 40
    for name, ret, types, nvalues, line in calls:
        where = f"LuxHIP.jl:{line} {name}"
        assert name in protos, f"{where}: not declared in include/luxhip.h"
        cret, cparams = protos[name]
        assert ret in _JULIA_FOR_C.get(cret, {cret}) or (cret == "int" and ret == "Cint"), f"{where}: returns {cret}, ccall says {ret}"
        assert len(types) == len(cparams), f"{where}: {len(cparams)} C parameters, {len(types)} ccall types"
        assert nvalues == len(types), f"{where}: {len(types)} ccall types but {nvalues} values passed"
        for k, (jt, ct) in enumerate(zip(types, cparams)):
            assert jt in _JULIA_FOR_C[ct], f"{where}: parameter {k + 1} is `{ct}`, ccall passes `{jt}`"


def test_julia_struct_mirrors_the_conv_descriptor():
    """ConvDimsC in the glue file lists the fields of luxhip_conv_dims_t in the same order with the same widths."""
    htext = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    m = re.search(r"typedef\s+struct\s*(?:\w+\s*)?\{(.*?)\}\s*luxhip_conv_dims_t\s*;", htext, flags=re.S)
    assert m
    cfields = []
    for decl in m.group(1).split(";"):
        decl = " ".join(re.sub(r"//[^\n]*", "", decl).split())
        if not decl:
            continue
        ctype, names = decl.split(" ", 1)
        for nm in names.split(","):
            nm = nm.strip()
            arr = re.match(r"(\w+)\[(\d+)\]", nm)
            cfields.append((arr.group(1), ctype, int(arr.group(2))) if arr else (nm, ctype, 1))
    jtext = open(JULIA_GLUE).read()
    m = re.search(r"struct ConvDimsC\n(.*?)\nend", jtext, flags=re.S)
    assert m
    jfields = []
    for line in m.group(1).split("\n"):
        line = line.split("#")[0].strip()
        if not line:
            continue
        for part in line.split(";"):
            nm, jt = (s.strip() for s in part.split("::"))
            jfields.append((nm, jt))
    width = {"int": "Cint", "int64_t": "Int64"}
    flat = []
    for nm, ct, n in cfields:
        flat += [(nm, width[ct], n)]
    assert len(flat) == len(jfields), (flat, jfields)
    for (cn, jt_want, n), (jn, jt) in zip(flat, jfields):
        want = jt_want if n == 1 else f"NTuple{{{n},{jt_want}}}"
        assert jt.replace(" ", "") == want, f"field {cn}/{jn}: C {n} x {jt_want}, Julia {jt}"
