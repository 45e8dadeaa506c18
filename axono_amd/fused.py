"""Fused operators (axono/python/axono/fused.py): silu_mul and add_rms_norm, one kernel each."""
from . import libaxono as _l

__all__ = ["silu_mul", "add_rms_norm"]


def silu_mul(gate, up):
    """y = silu(gate) * up, elementwise; gate and up have the same shape."""
    return _l.silu_mul(gate, up)


def add_rms_norm(x, residual, weight, eps: float = 1e-6):
    """y = x + residual; out = y * rsqrt(mean(y^2) + eps) * weight.  Returns (y, out)."""
    return _l.add_rms_norm(x, residual, weight, eps)
