"""axono_amd: the LLM decode path of Axono on MI355X (gfx950).

Hand-written HIP kernels behind a C ABI (include/axhip.h, built into axono_amd/lib/libaxhip.so) and
the host-side mirror of the reference's Python surface for that path: the same names as
`axono` (axono/python/axono/__init__.py:46-113) for the operators, `nn`, `fused`, `gqa`, `compile`
and graph capture, on the device strings "hip" / "hip:<id>".
"""
from . import format, fused, gqa, nn  # noqa: F401,A004
from .core import DataType, Status, Tensor, cuda_available, get_default_device, hip_available, set_default_device
from .core.backend import get_backend, set_backend
from .core.compile import compile  # noqa: A004
from .core.hip_graph import CUDAGraph, HIPGraph, cuda_graph, hip_graph
from .core.ops import (add, argmax, concat, embedding, linear, linear_nobias, mrope_cos_sin, rms_norm, rope,
                       rope_thd, rope_with_cos_sin, scaled_dot_product_attention, slice_)
from .fused import add_rms_norm, silu_mul
from .gqa import gqa_decode_attention, gqa_decode_attention_cache

__version__ = "0.2.0"

__all__ = [
    "DataType", "Status", "Tensor", "add", "rms_norm", "linear", "linear_nobias", "mrope_cos_sin", "embedding", "rope",
    "rope_with_cos_sin", "rope_thd", "scaled_dot_product_attention", "concat", "slice_", "argmax", "cuda_available",
    "hip_available", "get_default_device", "set_default_device", "set_backend", "get_backend", "CUDAGraph",
    "cuda_graph", "HIPGraph", "hip_graph", "compile", "silu_mul", "add_rms_norm", "gqa_decode_attention",
    "gqa_decode_attention_cache", "nn", "fused", "gqa",
]
