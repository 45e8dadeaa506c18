"""AXM1 weight container, byte-compatible with the reference's (axono/python/axono/format/axm.py:19-33).

File layout (all little-endian):

    0   "AXM1"
    4   uint16 version (1)
    6   2 reserved bytes
    8   uint64 length L of the index
    16  index: UTF-8 JSON {"tensors": [{"name", "dtype", "shape", "offset", "size"}, ...], "meta": {...}}
    align64(16 + L)  tensor bytes; every tensor starts on a 64-byte boundary; `offset` / `size` are
                     relative to this point

`save_axm`, `load_axm`, `read_axm_index` and `AxmReader` keep the reference's signatures and error
behaviour (axm.py:50-109, 112-135, 138-171, 174-214).  `load_axm_to_device` is this build's addition:
tensors go from the file mapping to device memory one at a time (the mapping is the staging buffer),
optionally converted to fp16 on the way, which is how the decode model wants its Linear weights.
"""
from __future__ import annotations

import json
import struct

import numpy as np

MAGIC = b"AXM1"
VERSION = 1
_ALIGN = 64
_HEAD = struct.Struct("<4sHHQ")

__all__ = ["save_axm", "load_axm", "read_axm_index", "AxmReader", "load_axm_to_device"]


def _pad(n: int) -> int:
    return -n % _ALIGN


def write_axm(specs, path: str, meta: dict | None = None) -> None:
    """Writes an AXM1 file from `specs`, an iterable of (name, numpy dtype, shape, produce) where
    produce() returns the array: the index is laid out from dtype and shape alone, and the arrays are
    produced and written one at a time, so a converter never holds more than one tensor."""
    specs = list(specs)
    tensors, cursor = [], 0
    for name, dt, shape, _ in specs:
        nbytes = int(np.dtype(dt).itemsize * int(np.prod(shape, dtype=np.int64)))
        tensors.append({"name": name, "dtype": str(np.dtype(dt)), "shape": [int(d) for d in shape], "offset": cursor,
                        "size": nbytes})
        cursor += nbytes + _pad(nbytes)
    index = json.dumps({"tensors": tensors, "meta": meta or {}}).encode("utf-8")
    with open(path, "wb") as f:
        f.write(_HEAD.pack(MAGIC, VERSION, 0, len(index)))
        f.write(index)
        f.write(bytes(_pad(_HEAD.size + len(index))))
        for (name, dt, shape, produce), t in zip(specs, tensors):
            a = np.ascontiguousarray(produce(), dtype=dt)
            if a.nbytes != t["size"] or tuple(a.shape) != tuple(shape):
                raise ValueError(f"tensor {name}: produced {a.shape} {a.dtype}, announced {tuple(shape)} {np.dtype(dt)}")
            f.write(memoryview(a).cast("B") if a.nbytes else b"")
            f.write(bytes(_pad(a.nbytes)))


def save_axm(state_dict: dict, path: str, meta: dict | None = None, dtype=None) -> None:
    """Writes {name: ndarray} to `path`.  `dtype` (e.g. "float16") converts every tensor; None keeps
    each array's dtype.  `meta` is stored verbatim in the index.  (Reference: axm.py:50-109.)"""
    def spec(name, value):
        a = np.asarray(value)
        return name, (a.dtype if dtype is None else np.dtype(dtype)), a.shape, lambda: a
    write_axm((spec(n, v) for n, v in state_dict.items()), path, meta)


def read_axm_index(path: str):
    """Header and index only.  Returns (index dict, byte offset where tensor data starts).
    ValueError for a short file, a wrong magic or an unknown version (axm.py:112-135)."""
    with open(path, "rb") as f:
        head = f.read(_HEAD.size)
        if len(head) < _HEAD.size:
            raise ValueError(f"{path} is not an .axm file (too short)")
        magic, version, _, n = _HEAD.unpack(head)
        if magic != MAGIC:
            raise ValueError(f"{path} is not an .axm file (magic={magic!r})")
        if version != VERSION:
            raise ValueError(f"unsupported .axm version: {version}")
        index = json.loads(f.read(n).decode("utf-8"))
    return index, _HEAD.size + n + _pad(_HEAD.size + n)


def _view(path: str, start: int, t: dict, mode="r") -> np.ndarray:
    shape = tuple(t["shape"])
    if int(np.prod(shape, dtype=np.int64)) == 0:  # memmap cannot map zero bytes
        return np.empty(shape, dtype=t["dtype"])
    return np.memmap(path, dtype=t["dtype"], mode=mode, offset=start + t["offset"], shape=shape)


def load_axm(path: str, mmap: bool = True) -> dict:
    """{name: read-only memmap view} of every tensor; data is paged in on access (axm.py:138-171).
    mmap=False returns independent in-memory copies."""
    index, start = read_axm_index(path)
    out = {}
    for t in index["tensors"]:
        v = _view(path, start, t)
        out[t["name"]] = v if mmap else np.array(v)
    return out


class AxmReader:
    """Parses the index once, then maps single tensors by name: read one layer, upload it, drop it
    (axm.py:174-214)."""

    def __init__(self, path: str):
        self.path = path
        self.index, self.data_start = read_axm_index(path)
        self._by_name = {t["name"]: t for t in self.index["tensors"]}

    def names(self):
        return list(self._by_name)

    def meta(self):
        return self.index.get("meta", {})

    def entry(self, name: str) -> dict:
        return dict(self._by_name[name])

    def get(self, name: str) -> np.ndarray:
        return _view(self.path, self.data_start, self._by_name[name])


def load_axm_to_device(path: str, device: str = "hip", dtype=None, names=None, convert=None) -> dict:
    """{name: Tensor on `device`}.  Each tensor is copied from its file mapping straight into a device
    allocation.  `dtype` ("float16" / "float32" / None) converts floating tensors on the host side of
    the copy; `convert(name, array) -> array` overrides it per tensor; `names` restricts the set."""
    from ..core.tensor import Tensor

    reader = AxmReader(path)
    out = {}
    for name in (names if names is not None else reader.names()):
        a = reader.get(name)
        if convert is not None:
            a = convert(name, a)
        elif dtype is not None and np.issubdtype(a.dtype, np.floating):
            a = a.astype(dtype, copy=False)
        out[name] = Tensor.from_numpy_ref(np.ascontiguousarray(a)).to(device)
    return out
