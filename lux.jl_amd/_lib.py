"""ctypes binding of libluxhip's C ABI (include/luxhip.h).  The library must have been built
(`make -C lux.jl_amd/csrc`); nothing here falls back to a CPU path."""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libluxhip.so")

OK, UNSUPPORTED, INVALID, HIP_ERROR, NOT_INITIALIZED = 0, -1, -2, -3, -4
F32, BF16 = 0, 1

ACT_IDS = {
    "identity": 0, "relu": 1, "tanh": 2, "sigmoid": 3, "swish": 4, "gelu": 5, "softplus": 6,
    "logsigmoid": 7, "lisht": 8,
    # NNlib.fast_act aliases and synonyms
    "tanh_fast": 2, "sigmoid_fast": 3, "gelu_tanh": 5, "silu": 4,
}


class LuxHipError(RuntimeError):
    def __init__(self, status, message):
        super().__init__(f"libluxhip status {status}: {message}")
        self.status = status


class Unsupported(LuxHipError):
    """Status -1: the caller is expected to fall back to its generic path."""


class ConvDimsStruct(C.Structure):
    _fields_ = [(n, C.c_int64) for n in (
        "W", "H", "Cin", "N", "kW", "kH", "Cout", "stride_w", "stride_h", "pad_w_lo", "pad_w_hi",
        "pad_h_lo", "pad_h_hi", "dil_w", "dil_h", "groups", "flipkernel")]


_vp, _i, _i64, _d, _sz, _u64 = C.c_void_p, C.c_int, C.c_int64, C.c_double, C.c_size_t, C.c_uint64
_fp = C.c_void_p  # float* passed as raw address
_ip64 = C.POINTER(C.c_int64)

# name -> argtypes; every function returns int
SIGNATURES = {
    "luxhip_init": [_i],
    "luxhip_shutdown": [],
    "luxhip_device_info": [C.c_char_p, _sz, C.POINTER(_i), C.POINTER(_i64)],
    "luxhip_stream_create": [C.POINTER(_vp)],
    "luxhip_stream_synchronize": [_vp],
    "luxhip_stream_destroy": [_vp],
    "luxhip_reserve": [_vp, _sz],
    "luxhip_event_create": [C.POINTER(_vp)],
    "luxhip_event_record": [_vp, _vp],
    "luxhip_event_elapsed_ms": [C.POINTER(C.c_float), _vp, _vp],
    "luxhip_event_destroy": [_vp],
    "luxhip_profile_enable": [_i],
    "luxhip_profile_report": [C.c_char_p, _sz],
    "luxhip_set_option": [C.c_char_p, _i64],
    "luxhip_measure_peaks": [_vp, C.POINTER(_d), C.POINTER(_d), C.POINTER(_d)],
    "luxhip_malloc": [C.POINTER(_vp), _sz],
    "luxhip_free": [_vp],
    "luxhip_trim": [],
    "luxhip_memcpy_h2d": [_vp, _vp, _sz, _vp],
    "luxhip_memcpy_d2h": [_vp, _vp, _sz, _vp],
    "luxhip_memcpy_d2d": [_vp, _vp, _sz, _vp],
    "luxhip_fill_zero": [_vp, _sz, _vp],
    "luxhip_bias_activation_fwd": [_vp, _i, _i, _i64, _i64, _i64, _vp, _vp, _vp, _vp],
    "luxhip_bias_activation_bwd": [_vp, _i, _i, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp],
    "luxhip_bias_activation_bwd_noalloc": [_vp, _i, _i, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp],
    "luxhip_batchnorm_fwd": [_vp, _i, _i, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _i, _d, _d, _vp, _vp, _vp, _fp, _fp],
    "luxhip_batchnorm_bwd": [_vp, _i, _i, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _fp, _fp, _i, _vp, _vp, _vp],
    "luxhip_groupnorm_fwd": [_vp, _i, _i, _i64, _i64, _i64, _i64, _vp, _vp, _vp, _d, _vp, _fp, _fp],
    "luxhip_groupnorm_bwd": [_vp, _i, _i, _i64, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _fp, _fp, _vp, _vp, _vp],
    "luxhip_instancenorm_fwd": [_vp, _i, _i, _i64, _i64, _i64, _vp, _vp, _vp, _d, _vp, _fp, _fp, _d, _vp, _vp, _vp, _vp],
    "luxhip_instancenorm_running_stats": [_vp, _i, _i64, _i64, _i64, _fp, _fp, _d, _d, _vp, _vp, _vp, _vp],
    "luxhip_attention_softmax_fwd": [_vp, _i, _i64, _i64, _i64, _i64, _vp, _d, _i, _vp, _i64, _i64, _vp, _i64, _i64, _vp],
    "luxhip_attention_softmax_bwd": [_vp, _i, _i64, _i64, _i64, _i, _vp, _vp, _d, _vp],
    "luxhip_rand_uniform": [_vp, _i, _i64, _u64, _u64, _vp],
    "luxhip_dropout_fwd": [_vp, _i, _i64, _u64, _u64, _d, _d, _vp, _vp, _vp],
    "luxhip_dropout_mask": [_vp, _i, _i64, _d, _d, _vp],
    "luxhip_dropout_mul": [_vp, _i, _i, _ip64, _ip64, _vp, _vp, _vp],
    "luxhip_alpha_dropout_fwd": [_vp, _i, _i64, _vp, _d, _vp, _d, _d, _d, _vp],
    "luxhip_alpha_dropout_bwd": [_vp, _i, _i64, _vp, _d, _vp, _d, _vp],
    "luxhip_layernorm_fwd": [_vp, _i, _i, _i64, _i64, _vp, _vp, _vp, _d, _vp, _fp, _fp],
    "luxhip_layernorm_bwd": [_vp, _i, _i, _i64, _i64, _vp, _vp, _vp, _vp, _fp, _fp, _vp, _vp, _vp],
    "luxhip_matmul": [_vp, _i, _i, _i, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _i64],
    "luxhip_batched_matmul": [_vp, _i, _i, _i, _i64, _i64, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64],
    "luxhip_batched_matmul_strided": [_vp, _i, _i, _i, _i64, _i64, _i64, _ip64, _vp, _i64, _ip64, _vp, _i64, _ip64, _vp, _i64, _ip64, _i],
    "luxhip_attention_weights_pullback": [_vp, _i, _i64, _i64, _i64, _ip64, _vp, _i64, _ip64, _vp, _vp, _i64, _ip64, _vp, _d, _vp, _i64,
                                          _ip64, _i],
    "luxhip_batch_sum": [_vp, _i, _i64, _i64, _vp, _vp],
    "luxhip_fused_dense_fwd": [_vp, _i, _i, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _i64, _vp],
    "luxhip_fused_dense_bwd": [_vp, _i, _i, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp],
    "luxhip_conv_fwd": [_vp, _i, _i, C.POINTER(ConvDimsStruct), _vp, _vp, _vp, _vp, _vp, _vp],
    "luxhip_conv_bwd_data": [_vp, _i, C.POINTER(ConvDimsStruct), _vp, _vp, _vp],
    "luxhip_conv_bwd_filter": [_vp, _i, C.POINTER(ConvDimsStruct), _vp, _vp, _vp],
    "luxhip_fused_conv_bwd": [_vp, _i, _i, C.POINTER(ConvDimsStruct), _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp],
    "luxhip_conv_depth_unfold": [_vp, _i, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i, _vp, _vp],
    "luxhip_conv_depth_fold": [_vp, _i, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i, _vp, _vp],
    "luxhip_swap_middle_dims": [_vp, _i, _i64, _i64, _i64, _i64, _vp, _vp],
    "luxhip_convert": [_vp, _i, _i, _i64, _vp, _vp],
    "luxhip_permute_leading3": [_vp, _i, _i64, _i64, _i64, _i64, _i, _i, _i, _vp, _vp],
}

_lib = None


def load():
    """dlopen libluxhip.so (idempotent) and declare every prototype of include/luxhip.h."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
            "(there is no CPU fallback)")
    lib = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if the symbol is not exported
        fn.argtypes = argtypes
        fn.restype = C.c_int
    lib.luxhip_last_error.argtypes = []
    lib.luxhip_last_error.restype = C.c_char_p
    _lib = lib
    return lib


def last_error() -> str:
    return load().luxhip_last_error().decode("utf-8", "replace")


def check(status: int):
    if status == OK:
        return
    msg = last_error()
    if status == UNSUPPORTED:
        raise Unsupported(status, msg)
    raise LuxHipError(status, msg)


def call(name: str, *args):
    """Call an entry point and raise on a non-zero status."""
    check(getattr(load(), name)(*args))
