"""Sequence and position operators of the Python surface (the names of
axono/python/axono/core/ops/sequence.py); each one hands its arguments to the function table in
`axono_amd.libaxono`, which checks them and launches the HIP kernel."""
from ... import libaxono as _table

__all__ = ["rope", "rope_with_cos_sin", "rope_thd", "mrope_cos_sin", "scaled_dot_product_attention", "embedding",
           "concat", "slice_", "argmax"]


def rope(x, pos_ids, theta: float = 10000.0):
    """x (rows, heads, d) rotated by rotate-half RoPE at INT64 positions `pos_ids` (rows,)."""
    return _table.rope(x, pos_ids, theta)


def rope_with_cos_sin(x, cos, sin):
    """Rotate-half RoPE with given tables: cos / sin (rows, d), shared by the heads of a row."""
    return _table.rope_with_cos_sin(x, cos, sin)


def rope_thd(x, pos, inv_freq, mrope_section):
    """Interleaved M-RoPE: pos INT64 (3, rows) for the T / H / W axes, inv_freq (d/2,), mrope_section
    the three section sizes (missing entries count as 0)."""
    sizes = [int(s) for s in mrope_section][:3]
    sizes += [0] * (3 - len(sizes))
    return _table.rope_thd(x, pos, inv_freq, *sizes)


def mrope_cos_sin(pos, inv_freq, h_sec: int, w_sec: int):
    """The (cos, sin) tables that rope_with_cos_sin needs to do what rope_thd does."""
    return _table.mrope_cos_sin(pos, inv_freq, h_sec, w_sec)


def scaled_dot_product_attention(q, k, v, is_causal: bool = False):
    """q (Sq, Hq, d), k / v (Skv, Hkv, d) with Hq a multiple of Hkv."""
    return _table.scaled_dot_product_attention(q, k, v, is_causal)


def embedding(ids, table):
    """Rows of `table` picked by INT64 `ids` of any shape."""
    return _table.embedding(ids, table)


def concat(a, b, axis: int):
    return _table.concat(a, b, axis)


def slice_(x, axis: int, start: int, length: int):
    """The `length` entries from `start` along `axis` (negative axes count from the end)."""
    return _table.slice(x, axis + x.ndim if axis < 0 else axis, start, length)


def argmax(x):
    """Index of the first maximum of every row (last axis), INT64."""
    return _table.argmax(x)
