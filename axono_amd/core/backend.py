"""Global backend switch: "cpu" | "hip" | "hip:<id>" (the reference's set_backend accepts
"cpu" | "cuda" | "cuda:<id>", axono/python/axono/core/backend.py:37-61)."""
from __future__ import annotations

from .tensor import get_default_device, hip_available, parse_device, set_default_device

_VALID_BACKENDS = ("cpu", "hip")


def set_backend(device: str) -> None:
    if not isinstance(device, str) or not device:
        raise ValueError("backend 必须是非空字符串, 如 'cpu' / 'hip' / 'hip:0'")
    name = device.split(":")[0].lower()
    if name not in _VALID_BACKENDS:
        raise ValueError(f"未知后端 '{device}', 可选: cpu / hip / hip:<id>")
    parse_device(device)
    if name == "hip" and not hip_available():
        raise RuntimeError("no HIP device available, cannot switch to the hip backend")
    set_default_device(device)


def get_backend() -> str:
    return get_default_device()
