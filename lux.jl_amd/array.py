"""Device arrays owned by libluxhip: dense, column-major (Julia order), fp32 or bf16."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib

# "u8": boolean masks (one byte per element, non-zero = true); no arithmetic entry point takes it as a storage type
DTYPES = {"f32": (_lib.F32, 4), "bf16": (_lib.BF16, 2), "u8": (-1, 1)}

_stream = C.c_void_p(None)


def current_stream() -> C.c_void_p:
    return _stream


def set_stream(s):
    global _stream
    _stream = s if isinstance(s, C.c_void_p) else C.c_void_p(s)


def _to_bf16_bits(a32: np.ndarray) -> np.ndarray:
    u = a32.view(np.uint32)
    r = u + (np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1)))
    return (r >> np.uint32(16)).astype(np.uint16)


def _from_bf16_bits(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << np.uint32(16)).view(np.float32)


class DeviceArray:
    """A dense column-major tensor in HBM.  `shape` is the Julia-style logical shape."""

    __slots__ = ("shape", "dtype", "ptr", "_owner", "_base")

    def __init__(self, shape, dtype="f32", ptr=None, base=None):
        if dtype not in DTYPES:
            raise TypeError(f"unsupported dtype {dtype!r} (use 'f32' or 'bf16'; 'u8' for masks)")
        self.shape = tuple(int(s) for s in shape)
        self.dtype = dtype
        self._base = base
        if ptr is None:
            p = C.c_void_p()
            _lib.call("luxhip_malloc", C.byref(p), max(self.nbytes, 1))
            self.ptr = p.value
            self._owner = True
        else:
            self.ptr = int(ptr)
            self._owner = False

    # ------------------------------------------------------------------ properties
    @property
    def size(self) -> int:
        n = 1
        for s in self.shape:
            n *= s
        return n

    @property
    def ndim(self) -> int:
        return len(self.shape)

    @property
    def itemsize(self) -> int:
        return DTYPES[self.dtype][1]

    @property
    def nbytes(self) -> int:
        return self.size * self.itemsize

    @property
    def code(self) -> int:
        return DTYPES[self.dtype][0]

    # ------------------------------------------------------------------ transfers
    @classmethod
    def from_numpy(cls, a, dtype="f32") -> "DeviceArray":
        a = np.asarray(a)
        out = cls(a.shape, dtype)
        if dtype == "u8":
            host = np.ascontiguousarray((a != 0).astype(np.uint8).ravel(order="F"))
        else:
            host = np.ascontiguousarray(np.asarray(a, dtype=np.float32).ravel(order="F"))
        if dtype == "bf16":
            host = _to_bf16_bits(host)
        if host.nbytes:
            _lib.call("luxhip_memcpy_h2d", out.ptr, host.ctypes.data, host.nbytes, current_stream())
        return out

    def to_numpy(self) -> np.ndarray:
        """float32 numpy array with the logical shape (bf16 is widened exactly; masks stay bytes)."""
        host = np.empty(self.size, dtype={"f32": np.float32, "bf16": np.uint16, "u8": np.uint8}[self.dtype])
        if host.nbytes:
            _lib.call("luxhip_memcpy_d2h", host.ctypes.data, self.ptr, host.nbytes, current_stream())
        if self.dtype == "bf16":
            host = _from_bf16_bits(host)
        return host.reshape(self.shape, order="F")

    def copy(self) -> "DeviceArray":
        out = DeviceArray(self.shape, self.dtype)
        if self.nbytes:
            _lib.call("luxhip_memcpy_d2d", out.ptr, self.ptr, self.nbytes, current_stream())
        return out

    def reshape(self, *shape) -> "DeviceArray":
        """Column-major reshape: a view on the same memory (keeps the owner alive)."""
        if len(shape) == 1 and isinstance(shape[0], (tuple, list)):
            shape = tuple(shape[0])
        n = 1
        for s in shape:
            n *= s
        if n != self.size:
            raise ValueError(f"cannot reshape {self.shape} to {shape}")
        return DeviceArray(shape, self.dtype, ptr=self.ptr, base=self)

    def __del__(self):
        if getattr(self, "_owner", False) and self.ptr:
            try:
                _lib.load().luxhip_free(C.c_void_p(self.ptr))
            except Exception:
                pass
            self.ptr = 0

    def __repr__(self):
        return f"DeviceArray(shape={self.shape}, dtype={self.dtype}, ptr=0x{self.ptr:x})"


class StatArray:
    """fp32 statistics buffer (saved mean / inverse std) of `n` entries."""

    __slots__ = ("n", "ptr")

    def __init__(self, n: int):
        self.n = int(n)
        p = C.c_void_p()
        _lib.call("luxhip_malloc", C.byref(p), max(4 * self.n, 4))
        self.ptr = p.value

    def to_numpy(self):
        host = np.empty(self.n, np.float32)
        if self.n:
            _lib.call("luxhip_memcpy_d2h", host.ctypes.data, self.ptr, host.nbytes, current_stream())
        return host

    def __del__(self):
        if self.ptr:
            try:
                _lib.load().luxhip_free(C.c_void_p(self.ptr))
            except Exception:
                pass
            self.ptr = 0
