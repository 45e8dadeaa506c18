"""The LLM operators of the decode path under the names of axono/python/axono/core/ops/llm.py; each
hands its arguments to the function table in `axono_amd.libaxono`."""
from ... import libaxono as _table

__all__ = ["rms_norm", "linear", "linear_nobias", "add"]


def rms_norm(x, weight, eps: float = 1e-5):
    """x * rsqrt(mean(x^2) + eps) * weight over the last axis (an empty weight: no scaling)."""
    return _table.rms_norm(x, weight, eps)


def linear(x, weight, bias):
    """x (M, K) . weight (N, K)^T + bias (N,); FLOAT16 weights with FLOAT32 or FLOAT16 x."""
    return _table.linear(x, weight, bias)


def linear_nobias(x, weight):
    return _table.linear_nobias(x, weight)


def add(a, b):
    """Elementwise sum of two tensors of one shape and dtype."""
    return _table.add(a, b)
