"""Tensor: dtype + shape + device string + reference-counted storage, contiguous row-major.

Mirrors the reference's `core::Tensor` (include/axono/core/tensor.h:24-129, src/core/tensor.cpp) as
the binding exposes it (axono/python/src/nanobind_module.cpp:206-377) together with the Python
conveniences the reference patches on (axono/python/axono/core/tensor.py:473-519).  Devices are
strings: "cpu" or "hip" / "hip:<id>".  Host tensors exist to carry data in and out; operators run
on hip tensors only.

Semantics kept from the reference: new tensors are zero-initialised (tensor.cpp:228-231); copying a
Tensor aliases its storage (:75-97); `reshape` is metadata-only and in place, `resize` reallocates
only when the element count changes (:236-255); `to(same device)` returns self;
`to_numpy()` of a host tensor is a view sharing memory, of a device tensor a host copy, and FLOAT16
comes back as int16 bit patterns (nanobind_module.cpp:343-353).
"""
from __future__ import annotations

import numpy as np

from .. import _lib
from ..device import AxhipError, DeviceBuffer, check
from .types import DTYPE_SIZE, DTYPE_TO_NUMPY, NUMPY_TO_DTYPE, DataType, Status

_DEFAULT_DEVICE = "cpu"


def parse_device(device: str):
    """'cpu' -> ('cpu', None); 'hip' / 'hip:3' -> ('hip', id)."""
    if not isinstance(device, str) or not device:
        raise ValueError("device 必须是非空字符串, 如 'cpu' / 'hip' / 'hip:0'")
    name, _, idx = device.partition(":")
    name = name.lower()
    if name == "cpu":
        return "cpu", None
    if name == "hip":
        try:
            return "hip", int(idx) if idx else 0
        except ValueError:
            raise ValueError(f"Invalid HIP device format: {device}") from None
    raise ValueError(f"未知设备 '{device}', 可选: cpu / hip / hip:<id>")


def set_default_device(device: str) -> None:
    global _DEFAULT_DEVICE
    parse_device(device)
    _DEFAULT_DEVICE = device


def get_default_device() -> str:
    return _DEFAULT_DEVICE


def hip_available() -> bool:
    """True when the HIP library is loaded and sees a device (the reference's cuda_available())."""
    return _lib.device_count() > 0


class _Storage:
    """Shared by every alias of a tensor (the reference's shared_ptr<void>)."""

    __slots__ = ("host", "dev", "keep", "version")

    def __init__(self, host=None, dev=None, keep=None):
        self.host = host  # np.ndarray of uint8, or None
        self.dev = dev    # DeviceBuffer, or None
        self.keep = keep  # object kept alive for borrowed host memory
        self.version = 0  # bumped by every host-initiated write (copy_from, copy_from_numpy, fill*):
        #                   holders of data derived from the contents (packed Linear weights) compare it


def _numel(shape):
    if len(shape) == 0:
        return 0  # the reference counts an empty shape as no elements (types.h:73-80)
    n = 1
    for s in shape:
        n *= int(s)
    return n


class Tensor:
    def __init__(self, dtype: DataType = DataType.FLOAT32, shape=None, device: str | None = None,
                 _storage: _Storage | None = None, _zero: bool = True):
        self._dtype = DataType(dtype)
        self._shape = [int(s) for s in shape] if shape is not None else []
        if any(s < 0 for s in self._shape):
            raise ValueError("negative dimension")
        self._device = device if device is not None else "cpu"
        self._kind, self._dev_id = parse_device(self._device)
        if _storage is not None:
            self._st = _storage
        else:
            self._st = _Storage()
            self._allocate(_zero)

    # ---- storage ---------------------------------------------------------------------------
    def _allocate(self, zero: bool = True) -> None:
        nbytes = self.num_bytes
        if self._kind == "cpu":
            self._st.host = np.zeros(nbytes, np.uint8) if zero else np.empty(nbytes, np.uint8)
            self._st.dev = None
        else:
            if not hip_available():
                raise RuntimeError("no HIP device available for device '%s'" % self._device)
            n = _lib.device_count()
            if self._dev_id >= n:
                raise IndexError(f"HIP device {self._dev_id} out of range (0-{n - 1})")
            check(_lib.load().axhip_set_device(self._dev_id), "set_device")
            self._st.dev = DeviceBuffer(nbytes, zero=zero) if nbytes else None
            self._st.host = None

    @property
    def data_ptr(self) -> int:
        """Device pointer (hip) or host address (cpu); 0 for an empty tensor."""
        if self._kind == "hip":
            return self._st.dev.ptr if self._st.dev is not None else 0
        return self._st.host.ctypes.data if self._st.host is not None and self._st.host.size else 0

    # ---- metadata --------------------------------------------------------------------------
    @property
    def dtype(self) -> DataType:
        return self._dtype

    @property
    def shape(self):
        return list(self._shape)

    @property
    def ndim(self) -> int:
        return len(self._shape)

    @property
    def device(self) -> str:
        return self._device

    @property
    def is_hip(self) -> bool:
        return self._kind == "hip"

    @property
    def is_cuda(self) -> bool:  # there is no CUDA path in this build
        return False

    @property
    def num_elements(self) -> int:
        return _numel(self._shape)

    @property
    def num_bytes(self) -> int:
        return self.num_elements * DTYPE_SIZE[self._dtype]

    def is_same_shape(self, other: "Tensor") -> bool:
        return self._shape == other._shape

    def __repr__(self) -> str:
        return f"Tensor(dtype={self._dtype.name}, shape={self._shape}, device='{self._device}')"

    # ---- aliasing / copies -----------------------------------------------------------------
    def __copy__(self):
        return Tensor(self._dtype, self._shape, self._device, _storage=self._st)

    def __deepcopy__(self, memo):
        t = Tensor(self._dtype, self._shape, self._device, _zero=False)
        t.copy_from(self)
        return t

    @staticmethod
    def create_like(other: "Tensor") -> "Tensor":
        return Tensor(other._dtype, other._shape, other._device)

    def copy_from(self, src: "Tensor") -> "Tensor":
        """In-place data copy; element counts and dtypes must match (Tensor::CopyFrom,
        tensor.cpp:186-215).  Any device pair."""
        if src.num_elements != self.num_elements or src._dtype != self._dtype:
            raise AxhipError("copy_from", Status.SHAPE_MISMATCH)
        n = self.num_bytes
        if n == 0:
            return self
        self._st.version += 1
        lib = _lib.load()
        if self._kind == "cpu" and src._kind == "cpu":
            self._st.host[:n] = src._st.host[:n]
        elif self._kind == "hip" and src._kind == "cpu":
            check(lib.axhip_memcpy_h2d(self.data_ptr, src._st.host.ctypes.data, n), "copy_from")
        elif self._kind == "cpu" and src._kind == "hip":
            check(lib.axhip_memcpy_d2h(self._st.host.ctypes.data, src.data_ptr, n), "copy_from")
        else:
            check(lib.axhip_memcpy_d2d(self.data_ptr, src.data_ptr, n), "copy_from")
        return self

    def to(self, device: str) -> "Tensor":
        if device == self._device:
            return self
        kind, dev_id = parse_device(device)
        if kind == self._kind and (kind == "cpu" or dev_id == self._dev_id):
            return self  # "hip" and "hip:0" name the same device
        t = Tensor(self._dtype, self._shape, device, _zero=False)
        t.copy_from(self)
        return t

    def to_(self, device: str) -> Status:
        moved = self.to(device)
        if moved is not self:
            self._device, self._kind, self._dev_id, self._st = moved._device, moved._kind, moved._dev_id, moved._st
        return Status.OK

    # ---- shape ops -------------------------------------------------------------------------
    def reshape(self, new_shape) -> "Tensor":
        shape = [int(s) for s in new_shape]
        if any(s < 0 for s in shape):
            if sum(1 for s in shape if s < 0) > 1:
                raise ValueError("reshape: 至多一个 -1")
            known = 1
            for s in shape:
                if s >= 0:
                    known *= s
            total = self.num_elements
            if known == 0 or total % known != 0:
                raise ValueError(f"reshape: 无法解析 -1 (known={known})")
            shape = [total // known if s < 0 else s for s in shape]
        if _numel(shape) != self.num_elements:
            raise RuntimeError(f"Reshape failed with status: {Status.INVALID_ARGUMENT!r}")
        self._shape = shape
        return self

    def resize(self, new_shape) -> "Tensor":
        shape = [int(s) for s in new_shape]
        if _numel(shape) != self.num_elements:
            self._shape = shape
            self._st = _Storage()
            self._allocate(True)
        else:
            self._shape = shape
        return self

    def transpose(self, dim0: int = -2, dim1: int = -1) -> "Tensor":
        """A new tensor with two dimensions exchanged (a copy: tensors carry no strides).  Negative
        indices count from the end; equal dims return an alias (Tensor::Transpose,
        src/core/tensor.cpp:386-424; device kernel src/core/cuda/tensor/transpose.cu)."""
        nd = self.ndim
        d0 = dim0 + nd if dim0 < 0 else dim0
        d1 = dim1 + nd if dim1 < 0 else dim1
        if not (0 <= d0 < nd and 0 <= d1 < nd):
            raise ValueError(f"Transpose: invalid dims, ndim={nd}, dim0={dim0}, dim1={dim1}")
        if d0 == d1:
            return self.__copy__()
        if d0 > d1:
            d0, d1 = d1, d0
        shape = list(self._shape)
        shape[d0], shape[d1] = shape[d1], shape[d0]
        out = Tensor(self._dtype, shape, self._device, _zero=False)
        if self.num_elements == 0:
            return out
        if self._kind == "cpu":
            src = self._as_numpy(raw_f16=True)
            out._st.host[:] = np.ascontiguousarray(np.swapaxes(src, d0, d1)).reshape(-1).view(np.uint8)
            return out
        outer, mid, inner = _numel(self._shape[:d0]) if d0 else 1, 1, 1
        for s_ in self._shape[d0 + 1:d1]:
            mid *= s_
        for s_ in self._shape[d1 + 1:]:
            inner *= s_
        from ..device import current_stream
        check(_lib.load().axhip_transpose(self.data_ptr, out.data_ptr, DTYPE_SIZE[self._dtype], outer, self._shape[d0],
                                          mid, self._shape[d1], inner, current_stream()), "transpose")
        return out

    @property
    def T(self) -> "Tensor":  # noqa: N802 - the reference's name (core/tensor.py:281-290)
        return self.transpose()

    # ---- arithmetic: only what the decode path has a kernel for --------------------------------
    def __add__(self, other) -> "Tensor":
        """Same-shape elementwise sum on the device (the residual add of a decoder layer); the
        reference's `+` also broadcasts a bias row and takes scalars through its generic elementwise
        family, which this build does not carry."""
        from .. import libaxono
        if not isinstance(other, Tensor):
            return NotImplemented
        return libaxono.add(self, other)

    __radd__ = __add__

    def _no_operator(self, *_):
        raise NotImplementedError("this build carries the decode path only: of the arithmetic operators, "
                                  "`+` on equal shapes has a kernel; use NumPy on to_numpy() for the rest")

    __sub__ = __mul__ = __truediv__ = __matmul__ = __neg__ = __abs__ = _no_operator

    def fill_zero(self) -> "Tensor":
        self._st.version += 1
        if self._kind == "cpu":
            self._st.host[:] = 0
        elif self.num_bytes:
            check(_lib.load().axhip_fill_zero(self.data_ptr, self.num_bytes), "fill_zero")
        return self

    def fill(self, value) -> "Tensor":
        host = np.full(self._shape, value, dtype=DTYPE_TO_NUMPY[self._dtype])
        return self.copy_from_numpy(host)

    # ---- numpy interop -----------------------------------------------------------------------
    @classmethod
    def from_numpy(cls, array: np.ndarray) -> "Tensor":
        """Copies a NumPy array into a new tensor on the default device.  float16 arrays keep their
        bit patterns (the reference cannot take them here, core/tensor.py:115-117)."""
        array = np.ascontiguousarray(array)
        dt = NUMPY_TO_DTYPE.get(array.dtype)
        if dt is None:
            array = array.astype(np.float32)
            dt = DataType.FLOAT32
        t = cls(dt, list(array.shape), "cpu", _zero=False)
        if array.nbytes:
            t._st.host[:] = array.reshape(-1).view(np.uint8)
        default = get_default_device()
        return t.to(default) if default != "cpu" else t

    @classmethod
    def from_numpy_ref(cls, array: np.ndarray) -> "Tensor":
        """Borrows a C-contiguous NumPy array without copying (host tensor sharing its memory)."""
        arr = np.asarray(array)
        if not arr.flags["C_CONTIGUOUS"]:
            raise ValueError("from_numpy_ref needs a C-contiguous array")
        dt = NUMPY_TO_DTYPE.get(arr.dtype)
        if dt is None:
            raise ValueError(f"unsupported dtype {arr.dtype}")
        st = _Storage(host=arr.reshape(-1).view(np.uint8), keep=array)
        return cls(dt, list(arr.shape), "cpu", _storage=st)

    @classmethod
    def from_borrowed(cls, array: np.ndarray) -> "Tensor":
        """Zero-copy host tensor over a C-contiguous float32 array, or over a uint16 array holding
        FLOAT16 bit patterns (nanobind_module.cpp:218-236); the array is kept alive by the tensor."""
        arr = np.asarray(array)
        if not arr.flags["C_CONTIGUOUS"]:
            raise ValueError("from_borrowed needs a C-contiguous array")
        if arr.dtype == np.float32:
            dt = DataType.FLOAT32
        elif arr.dtype in (np.uint16, np.float16):
            dt = DataType.FLOAT16
        else:
            raise RuntimeError("from_borrowed: only FLOAT32 / FLOAT16 (as uint16 bit patterns)")
        return cls(dt, list(arr.shape), "cpu", _storage=_Storage(host=arr.reshape(-1).view(np.uint8), keep=array))

    @classmethod
    def from_borrowed_i64(cls, array: np.ndarray) -> "Tensor":
        """Zero-copy host tensor over a C-contiguous int64 array (nanobind_module.cpp:237-250)."""
        arr = np.asarray(array)
        if arr.dtype != np.int64 or not arr.flags["C_CONTIGUOUS"]:
            raise RuntimeError("from_borrowed_i64: a C-contiguous INT64 array is required")
        return cls(DataType.INT64, list(arr.shape), "cpu", _storage=_Storage(host=arr.reshape(-1).view(np.uint8), keep=array))

    # data_<dtype>() accessors of the binding (nanobind_module.cpp:325-372): a host tensor gives a view
    # sharing its memory, a device tensor a host copy; the element type is not checked against the
    # tensor's dtype except for data_float16, which returns int16 bit patterns of a FLOAT16 tensor.
    def _data_as(self, npdt) -> np.ndarray:
        npdt = np.dtype(npdt)
        if self.num_bytes % npdt.itemsize or DTYPE_SIZE[self._dtype] != npdt.itemsize:
            raise RuntimeError(f"data accessor: {self._dtype.name} elements are not {npdt.itemsize} bytes wide")
        if self._kind == "cpu":
            return self._st.host[:self.num_bytes].view(npdt).reshape(self._shape)
        out = np.empty(self._shape, dtype=npdt)
        if self.num_bytes:
            check(_lib.load().axhip_memcpy_d2h(out.ctypes.data, self.data_ptr, self.num_bytes), "data")
        return out

    def data_int8(self):
        return self._data_as(np.int8)

    def data_int16(self):
        return self._data_as(np.int16)

    def data_int32(self):
        return self._data_as(np.int32)

    def data_int64(self):
        return self._data_as(np.int64)

    def data_float16(self):
        if self._dtype != DataType.FLOAT16:
            raise RuntimeError("data_float16: the tensor is not FLOAT16")
        return self._data_as(np.int16)

    def data_float32(self):
        return self._data_as(np.float32)

    def data_float64(self):
        return self._data_as(np.float64)

    def data_bool(self):
        return self._data_as(np.bool_)

    def _host_typed(self, raw_f16: bool):
        npdt = DTYPE_TO_NUMPY[self._dtype]
        if raw_f16 and self._dtype == DataType.FLOAT16:
            npdt = np.int16
        return npdt

    def to_numpy(self) -> np.ndarray:
        """Host tensors: a view sharing memory.  Device tensors: a host copy.  FLOAT16 is returned as
        int16 bit patterns, as the reference does; use `numpy()` for typed values."""
        return self._as_numpy(raw_f16=True)

    def numpy(self) -> np.ndarray:
        """Like to_numpy() with FLOAT16 returned as np.float16."""
        return self._as_numpy(raw_f16=False)

    def _as_numpy(self, raw_f16: bool) -> np.ndarray:
        npdt = self._host_typed(raw_f16)
        n = self.num_bytes
        if self._kind == "cpu":
            return self._st.host[:n].view(npdt).reshape(self._shape)
        out = np.empty(self._shape, dtype=npdt)
        if n:
            check(_lib.load().axhip_memcpy_d2h(out.ctypes.data, self.data_ptr, n), "to_numpy")
        return out

    def copy_from_numpy(self, array: np.ndarray) -> "Tensor":
        if list(array.shape) != self._shape:
            raise ValueError(f"copy_from_numpy: 形状不匹配 {list(array.shape)} vs {self._shape}")
        array = np.ascontiguousarray(array)
        if NUMPY_TO_DTYPE.get(array.dtype) != self._dtype:
            raise ValueError(f"copy_from_numpy: dtype 不匹配 {array.dtype} vs {self._dtype.name}")
        n = self.num_bytes
        if n == 0:
            return self
        self._st.version += 1
        if self._kind == "cpu":
            self._st.host[:n] = array.reshape(-1).view(np.uint8)
        else:
            check(_lib.load().axhip_memcpy_h2d(self.data_ptr, array.ctypes.data, n), "copy_from_numpy")
        return self

    # ---- dtype conversion ----------------------------------------------------------------------
    def cast_to(self, target: DataType) -> "Tensor":
        """FLOAT16 <-> FLOAT32, IEEE round-to-nearest-even on both devices (Tensor::CastTo,
        tensor.cpp:437-489; the device kernels it stands for are kernel.cu:175-223).  Same dtype: an
        alias sharing storage."""
        target = DataType(target)
        if target == self._dtype:
            return self.__copy__()
        pair = {self._dtype, target}
        if pair != {DataType.FLOAT16, DataType.FLOAT32}:
            if self._kind == "cpu":
                return Tensor.from_numpy_ref(np.ascontiguousarray(self.numpy().astype(DTYPE_TO_NUMPY[target])))
            raise AxhipError("cast_to", Status.UNSUPPORTED_TYPE)
        out = Tensor(target, self._shape, self._device, _zero=False)
        if self._kind == "cpu":
            out._st.host[:] = self.numpy().astype(DTYPE_TO_NUMPY[target]).reshape(-1).view(np.uint8)
        elif self.num_elements:
            from ..device import current_stream
            check(_lib.load().axhip_cast(self.data_ptr, int(self._dtype), out.data_ptr, int(target),
                                         self.num_elements, current_stream()), "cast_to")
        return out

    _orig_cast_to = cast_to

    # ---- factories -----------------------------------------------------------------------------
    @classmethod
    def zeros(cls, shape, dtype: DataType = DataType.FLOAT32, device: str | None = None) -> "Tensor":
        return cls(dtype, list(shape), device or get_default_device())

    @classmethod
    def ones(cls, shape, dtype: DataType = DataType.FLOAT32, device: str | None = None) -> "Tensor":
        return cls.full(shape, 1, dtype, device)

    @classmethod
    def full(cls, shape, value, dtype: DataType = DataType.FLOAT32, device: str | None = None) -> "Tensor":
        t = cls(dtype, list(shape), device or get_default_device(), _zero=False)
        return t.fill(value)

    @classmethod
    def randn(cls, shape, dtype: DataType = DataType.FLOAT32, device: str | None = None, mean: float = 0.0,
              stddev: float = 1.0) -> "Tensor":
        """Unseeded standard normal values, drawn on the host (the reference's randn is unseeded on
        both devices too, src/ops/cpu/randn.cpp:13); seeded inputs come from NumPy."""
        host = (np.random.standard_normal(list(shape)) * stddev + mean).astype(DTYPE_TO_NUMPY[DataType(dtype)])
        t = cls(dtype, list(shape), device or get_default_device(), _zero=False)
        return t.copy_from_numpy(host)
