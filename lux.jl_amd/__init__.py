"""MI355X (gfx950) backend for LuxLib's fused operators: Python host side over libluxhip.

    import lux_jl_amd as lux          # loaded from the directory `lux.jl_amd`
    lux.init()
    x = lux.DeviceArray.from_numpy(a)                       # column-major, fp32 or bf16
    y = lux.fused_dense_bias_activation("tanh", W, x, b)
    y, back = lux.pullback(lux.fused_dense_bias_activation, "tanh", W, x, b)
    dW, dx, db = back(delta)

There is no CPU fallback: importing works anywhere (the library is dlopen'ed lazily), but
`init()` and every operator need the built library and a gfx950 device.
"""
from __future__ import annotations

import ctypes as _C

from . import _lib
from ._lib import LuxHipError, Unsupported
from .array import DeviceArray, StatArray, current_stream, set_stream
from .luxlib import (ArgumentError, PhiloxRNG, scaled_dot_product_attention, rrule_scaled_dot_product_attention, batched_matmul, rrule_batched_matmul, alpha_dropout, dropout, dropout_dot_mul, dropout_shape, rand_uniform,
                     rrule_alpha_dropout, rrule_dropout, attention_dropout, DenseConvDims, DimensionMismatch, DEFAULT_DIMS, COLON, batchnorm, bias_activation,
                     bias_activation_inplace, conv, conv_data_grad, conv_filter_grad, default_epsilon,
                     fast_activation, fast_activation_inplace, fused_conv_bias_activation, fused_dense_bias_activation,
                     groupnorm, instancenorm, layernorm, matmul, pullback, rrule_fast_activation, rrule_instancenorm,
                     rrule_batchnorm, rrule_bias_activation, rrule_fused_conv_bias_activation,
                     rrule_fused_dense_bias_activation, rrule_groupnorm, rrule_layernorm)

_initialised = False


def init(device: int = 0, own_stream: bool = True):
    """Initialise the library on `device` and (by default) make a library-owned stream current."""
    global _initialised
    _lib.call("luxhip_init", int(device))
    if own_stream and not _initialised:
        s = _C.c_void_p()
        _lib.call("luxhip_stream_create", _C.byref(s))
        set_stream(s)
    _initialised = True


def set_option(name: str, value: int):
    """Tuning switch of the library (luxhip_set_option): "bn_resident", "bn_spin_limit", "gemm_tile"."""
    _lib.call("luxhip_set_option", name.encode(), int(value))


def synchronize():
    _lib.call("luxhip_stream_synchronize", current_stream())


def device_info():
    name = _C.create_string_buffer(256)
    cus, mem = _C.c_int(), _C.c_int64()
    _lib.call("luxhip_device_info", name, 256, _C.byref(cus), _C.byref(mem))
    return {"name": name.value.decode(), "compute_units": cus.value, "total_mem": mem.value}


class Event:
    """HIP event on the library's streams (timing happens on the stream kernels run on)."""

    def __init__(self):
        self._e = _C.c_void_p()
        _lib.call("luxhip_event_create", _C.byref(self._e))

    def record(self, stream=None):
        _lib.call("luxhip_event_record", self._e, stream if stream is not None else current_stream())

    def elapsed_ms(self, stop: "Event") -> float:
        ms = _C.c_float()
        _lib.call("luxhip_event_elapsed_ms", _C.byref(ms), self._e, stop._e)
        return ms.value

    def __del__(self):
        try:
            if self._e:
                _lib.load().luxhip_event_destroy(self._e)
        except Exception:
            pass
