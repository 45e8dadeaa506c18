"""Sequence / position operators: thin forwards to the native function table, as in
axono/python/axono/core/ops/sequence.py."""
from ... import libaxono as _l


def rope(x, pos_ids, theta: float = 10000.0):
    return _l.rope(x, pos_ids, theta)


def rope_with_cos_sin(x, cos, sin):
    return _l.rope_with_cos_sin(x, cos, sin)


def rope_thd(x, pos, inv_freq, mrope_section):
    t_sec, h_sec, w_sec = (list(mrope_section) + [0, 0, 0])[:3]
    return _l.rope_thd(x, pos, inv_freq, int(t_sec), int(h_sec), int(w_sec))


def mrope_cos_sin(pos, inv_freq, h_sec: int, w_sec: int):
    return _l.mrope_cos_sin(pos, inv_freq, h_sec, w_sec)


def scaled_dot_product_attention(q, k, v, is_causal: bool = False):
    return _l.scaled_dot_product_attention(q, k, v, is_causal)


def embedding(ids, table):
    return _l.embedding(ids, table)


def concat(a, b, axis: int):
    return _l.concat(a, b, axis)


def slice_(x, axis: int, start: int, length: int):
    if axis < 0:
        axis = x.ndim + axis
    return _l.slice(x, axis, start, length)


def argmax(x):
    return _l.argmax(x)


__all__ = ["rope", "rope_with_cos_sin", "rope_thd", "mrope_cos_sin", "scaled_dot_product_attention", "embedding",
           "concat", "slice_", "argmax"]
