"""Raw device memory over the C ABI: allocation through the library's caching allocator and
blocking host<->device copies.  The Tensor class and the tests build on this."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib


class AxhipError(RuntimeError):
    """A C-ABI call returned a non-OK status (same integer values as the reference's Status)."""

    def __init__(self, op: str, code: int):
        # message shape of the reference binding: "<op> 失败, 错误代码: <int>"
        super().__init__(f"{op} 失败, 错误代码: {code}")
        self.op = op
        self.code = code


def check(code: int, op: str) -> None:
    if code != 0:
        raise AxhipError(op, int(code))


class DeviceBuffer:
    """A block of device memory owned by this object (returned to the allocator on release)."""

    __slots__ = ("ptr", "nbytes", "_lib", "_owned")

    def __init__(self, nbytes: int, zero: bool = False):
        self._lib = _lib.load()
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        check(self._lib.axhip_alloc(self.nbytes, 1 if zero else 0, C.byref(p)), "alloc")
        self.ptr = p.value or 0
        # blocks handed out while a capture pool records or a graph captures belong to the pool /
        # the graph: this object must never free them (the address may be reused after a reset)
        owned = C.c_int(0)
        self._owned = True
        if self.ptr and self._lib.axhip_block_is_capture_owned(self.ptr, C.byref(owned)) == 0 and owned.value:
            self._owned = False

    @classmethod
    def from_numpy(cls, arr: np.ndarray) -> "DeviceBuffer":
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes)
        buf.upload(arr)
        return buf

    def upload(self, arr: np.ndarray, offset: int = 0) -> None:
        arr = np.ascontiguousarray(arr)
        if offset + arr.nbytes > self.nbytes:
            raise ValueError("upload larger than the buffer")
        if arr.nbytes:
            check(self._lib.axhip_memcpy_h2d(self.ptr + offset, arr.ctypes.data, arr.nbytes), "memcpy_h2d")

    def download(self, dtype, shape, offset: int = 0) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        if offset + out.nbytes > self.nbytes:
            raise ValueError("download larger than the buffer")
        if out.nbytes:
            check(self._lib.axhip_memcpy_d2h(out.ctypes.data, self.ptr + offset, out.nbytes), "memcpy_d2h")
        return out

    def release(self) -> None:
        if self.ptr:
            if self._owned:
                self._lib.axhip_free(self.ptr)
            self.ptr = 0

    def __del__(self):
        try:
            self.release()
        except Exception:  # interpreter shutdown
            pass


def current_stream() -> int:
    return _lib.load().axhip_current_stream() or 0


def synchronize() -> None:
    check(_lib.load().axhip_synchronize(), "synchronize")
