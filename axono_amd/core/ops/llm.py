"""LLM operators on the decode path (rms_norm, linear, linear_nobias, add): thin forwards, as in
axono/python/axono/core/ops/llm.py."""
from ... import libaxono as _l


def rms_norm(x, weight, eps: float = 1e-5):
    return _l.rms_norm(x, weight, eps)


def linear(x, weight, bias):
    return _l.linear(x, weight, bias)


def linear_nobias(x, weight):
    return _l.linear_nobias(x, weight)


def add(a, b):
    return _l.add(a, b)


__all__ = ["rms_norm", "linear", "linear_nobias", "add"]
