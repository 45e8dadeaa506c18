"""The operator function table of the decode path, name for name as the reference's native module
`libaxono` exposes it (axono/python/src/nanobind_module.cpp), re-stated over the C ABI of
libaxhip.so.  Every function allocates its result like the reference binding does, forwards to one
`axhip_*` entry point on the current stream, and turns a non-OK status into
`RuntimeError("<op> 失败, 错误代码: <int>")` (nanobind_module.cpp:1022-1024).

Operators run on hip tensors.  A host tensor is refused with DEVICE_MISMATCH: this build has no CPU
operator implementation to fall back to.
"""
from __future__ import annotations

import ctypes as C

from . import _lib
from .core.tensor import Tensor, hip_available
from .core.types import DataType, Status
from .device import AxhipError, check, current_stream

__version__ = "0.2.0"

_FLOATS = (DataType.FLOAT16, DataType.FLOAT32)


def _lib_():
    return _lib.load()


def _need_hip(op: str, *tensors) -> None:
    dev = None
    for t in tensors:
        if t is None or t.num_elements == 0:
            continue
        if not t.is_hip:
            raise AxhipError(op, Status.DEVICE_MISMATCH)
        if dev is None:
            dev = t._dev_id
        elif t._dev_id != dev:
            raise AxhipError(op, Status.DEVICE_MISMATCH)


def _new(dtype, shape, like: Tensor) -> Tensor:
    # results are fully overwritten by their kernels: no zero fill
    return Tensor(dtype, shape, like.device, _zero=False)


def cuda_available() -> bool:
    """Always False: this build has no CUDA path (the reference gates on a CUDA build,
    nanobind_module.cpp:1211-1217).  See hip_available()."""
    return False


def cached_bytes() -> int:
    return int(_lib_().axhip_cached_bytes())


def set_cache_budget(nbytes: int) -> None:
    check(_lib_().axhip_set_cache_budget(int(nbytes)), "set_cache_budget")


def empty_cache() -> None:
    check(_lib_().axhip_empty_cache(), "empty_cache")


def synchronize() -> None:
    check(_lib_().axhip_synchronize(), "synchronize")


# ---- decode attention ------------------------------------------------------------------------
def _workspace(nbytes: int, like: Tensor) -> Tensor:
    return Tensor(DataType.INT8, [max(int(nbytes), 256)], like.device, _zero=False)


def gqa_decode_attention(q: Tensor, k: Tensor, v: Tensor) -> Tensor:
    """q (1,Hq,D), k/v (L,Hkv,D) -> (1,Hq,D).  nanobind_module.cpp:1016-1028 -> GqaDecodeAttention
    (src/ops/cuda/gqa.cu:139-182).  FLOAT32 as in the reference, or FLOAT16."""
    op = "gqa_decode_attention"
    _need_hip(op, q, k, v)
    if q.ndim != 3 or k.ndim != 3 or v.ndim != 3 or q.dtype not in _FLOATS:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    sq, hq, d = q.shape
    L, hkv, dk = k.shape
    if sq != 1:
        raise AxhipError(op, Status.INVALID_ARGUMENT)
    if dk != d or v.shape != k.shape or hkv == 0 or hq % hkv != 0:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    out = _new(q.dtype, [1, hq, d], q)
    lib = _lib_()
    wsb = lib.axhip_gqa_decode_workspace_bytes(1, hq, hkv, d, L)
    ws = _workspace(wsb, q)
    check(lib.axhip_gqa_decode(q.data_ptr, k.data_ptr, v.data_ptr, None, out.data_ptr, ws.data_ptr, wsb,
                               int(q.dtype), 1, hq, hkv, d, L, 0, d, hkv * d, current_stream()), op)
    return out


def gqa_decode_attention_cache(q: Tensor, k_cache: Tensor, v_cache: Tensor, seq_lens: Tensor | None = None,
                               max_len: int | None = None, out: Tensor | None = None,
                               workspace: Tensor | None = None) -> Tensor:
    """Batched form over a static cache: q (B,Hq,D), caches (B,Hkv,Lmax,D), seq_lens INT32 (B,) on
    the device (read by the kernel, so a captured graph follows it).  No reference counterpart: the
    reference calls the single-sequence op once per sequence."""
    op = "gqa_decode_attention_cache"
    _need_hip(op, q, k_cache, v_cache, seq_lens)
    if q.ndim != 3 or k_cache.ndim != 4 or q.dtype not in _FLOATS or k_cache.dtype != q.dtype or v_cache.dtype != q.dtype:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    B, hq, d = q.shape
    Bc, hkv, lmax, dk = k_cache.shape
    if Bc != B or dk != d or v_cache.shape != k_cache.shape or hkv == 0 or hq % hkv != 0:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    if seq_lens is not None and (seq_lens.dtype != DataType.INT32 or seq_lens.num_elements != B):
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    max_len = lmax if max_len is None else min(int(max_len), lmax)
    if out is None:
        out = _new(q.dtype, [B, hq, d], q)
    lib = _lib_()
    wsb = lib.axhip_gqa_decode_workspace_bytes(B, hq, hkv, d, max_len)
    ws = workspace if workspace is not None else _workspace(wsb, q)
    check(lib.axhip_gqa_decode(q.data_ptr, k_cache.data_ptr, v_cache.data_ptr,
                               seq_lens.data_ptr if seq_lens is not None else None, out.data_ptr, ws.data_ptr,
                               ws.num_bytes, int(q.dtype), B, hq, hkv, d, max_len, hkv * lmax * d, lmax * d, d,
                               current_stream()), op)
    return out


PAGE_KEYS = 128  # keys per page of a paged KV cache (AXHIP_PAGE_KEYS)


def gqa_decode_attention_paged(q: Tensor, k_pool: Tensor, v_pool: Tensor, page_table: Tensor, seq_lens: Tensor | None,
                               max_len: int, out: Tensor | None = None, workspace: Tensor | None = None) -> Tensor:
    """Decode attention over a paged cache: q (B,Hq,D), pools (n_pages,Hkv,128,D), page_table INT32
    (B,max_pages), seq_lens INT32 (B,), both on the device; max_len bounds every length.  Same result, bit
    for bit, as gqa_decode_attention_cache on a dense cache holding the same keys."""
    op = "gqa_decode_attention_paged"
    _need_hip(op, q, k_pool, v_pool, page_table, seq_lens)
    if q.ndim != 3 or k_pool.ndim != 4 or q.dtype not in _FLOATS or k_pool.dtype != q.dtype or v_pool.dtype != q.dtype:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    B, hq, d = q.shape
    n_pages, hkv, pk, dk = k_pool.shape
    if pk != PAGE_KEYS or dk != d or v_pool.shape != k_pool.shape or hkv == 0 or hq % hkv != 0:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    if page_table.dtype != DataType.INT32 or page_table.ndim != 2 or page_table.shape[0] != B:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    if seq_lens is not None and (seq_lens.dtype != DataType.INT32 or seq_lens.num_elements != B):
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    max_pages = page_table.shape[1]
    max_len = int(max_len)
    if out is None:
        out = _new(q.dtype, [B, hq, d], q)
    lib = _lib_()
    wsb = lib.axhip_gqa_decode_workspace_bytes(B, hq, hkv, d, max(max_len, 1))
    ws = workspace if workspace is not None else _workspace(wsb, q)
    check(lib.axhip_gqa_decode_paged(q.data_ptr, k_pool.data_ptr, v_pool.data_ptr, page_table.data_ptr,
                                     seq_lens.data_ptr if seq_lens is not None else None, out.data_ptr, ws.data_ptr,
                                     ws.num_bytes, int(q.dtype), B, hq, hkv, d, max_len, max_pages, n_pages,
                                     current_stream()), op)
    return out


def kv_append_paged(k_new: Tensor, v_new: Tensor, k_pool: Tensor, v_pool: Tensor, page_table: Tensor,
                    start: Tensor | None, tokens_per_sequence: int = 1, table_row: int | None = None) -> None:
    """In place: token t of sequence b (rows [B, S, Hkv, D], S = tokens_per_sequence) is written at key
    position start[b] + t of the paged cache.  table_row: treat the rows as ONE sequence, the one of that
    row of the page table (start is then that sequence's entry of a per-sequence tensor)."""
    op = "kv_append_paged"
    _need_hip(op, k_new, v_new, k_pool, v_pool, page_table, start)
    if k_pool.ndim != 4 or k_new.dtype != k_pool.dtype or v_new.dtype != v_pool.dtype or k_pool.dtype != v_pool.dtype:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    n_pages, hkv, pk, d = k_pool.shape
    B, max_pages = page_table.shape
    S = int(tokens_per_sequence)
    tbl, st_ptr = page_table.data_ptr, (start.data_ptr if start is not None else None)
    if table_row is not None:
        if not 0 <= table_row < B:
            raise AxhipError(op, Status.INVALID_ARGUMENT)
        tbl += table_row * max_pages * 4
        if start is not None:
            st_ptr += table_row * (4 if start.dtype == DataType.INT32 else 8)
        B = 1
    if pk != PAGE_KEYS or v_pool.shape != k_pool.shape or k_new.num_elements != B * S * hkv * d or v_new.num_elements != k_new.num_elements:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    if start is not None and start.dtype not in (DataType.INT32, DataType.INT64):
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    check(_lib_().axhip_kv_append_paged(k_new.data_ptr, v_new.data_ptr, k_pool.data_ptr, v_pool.data_ptr, tbl, st_ptr,
                                        int(start.dtype) if start is not None else int(DataType.INT32),
                                        k_pool.num_bytes // max(k_pool.num_elements, 1), B, S, hkv, d, max_pages, n_pages,
                                        current_stream()), op)


def scaled_dot_product_attention(q: Tensor, k: Tensor, v: Tensor, is_causal: bool = False) -> Tensor:
    """q (Sq,Hq,D), k/v (Skv,Hkv,D).  nanobind_module.cpp:1107-1135."""
    op = "scaled_dot_product_attention"
    _need_hip(op, q, k, v)
    if q.ndim != 3 or k.ndim != 3 or v.ndim != 3:
        raise AxhipError(op, Status.INVALID_ARGUMENT)
    if q.dtype not in _FLOATS or k.dtype != q.dtype or v.dtype != q.dtype:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    sq, hq, d = q.shape
    skv, hkv, dk = k.shape
    if dk != d or v.shape != k.shape or hkv == 0 or hq % hkv != 0:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    out = _new(q.dtype, [sq, hq, d], q)
    check(_lib_().axhip_sdpa(q.data_ptr, k.data_ptr, v.data_ptr, out.data_ptr, int(q.dtype), sq, hq, hkv, d, skv,
                             1 if is_causal else 0, current_stream()), op)
    return out


# ---- KV cache movement -----------------------------------------------------------------------
def concat(a: Tensor, b: Tensor, axis: int) -> Tensor:
    """nanobind_module.cpp:1137-1160 -> Concat (src/ops/cpu/sequence.cpp:303-338)."""
    op = "concat"
    _need_hip(op, a, b)
    if a.ndim < 1 or a.ndim != b.ndim or a.dtype != b.dtype:
        raise AxhipError(op, Status.INVALID_ARGUMENT)
    nd = a.ndim
    ax = axis + nd if axis < 0 else axis
    if ax < 0 or ax >= nd:
        raise AxhipError(op, Status.INVALID_ARGUMENT)
    sa, sb = a.shape, b.shape
    if any(i != ax and sa[i] != sb[i] for i in range(nd)):
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    shape = list(sa)
    shape[ax] += sb[ax]
    out = _new(a.dtype, shape, a)
    outer = 1
    for i in range(ax):
        outer *= sa[i]
    if outer and (a.num_bytes or b.num_bytes):
        check(_lib_().axhip_concat(a.data_ptr, b.data_ptr, out.data_ptr, outer, a.num_bytes // outer,
                                   b.num_bytes // outer, current_stream()), op)
    return out


def slice(x: Tensor, axis: int, start: int, length: int) -> Tensor:  # noqa: A001 - the reference's name
    """Contiguous slice along an axis (nanobind_module.cpp:1162-1180 -> Slice, sequence.cpp:340-370)."""
    op = "slice"
    _need_hip(op, x)
    if x.ndim < 1 or axis < 0 or axis >= x.ndim or start < 0 or length < 0 or start + length > x.shape[axis]:
        raise AxhipError(op, Status.INVALID_ARGUMENT)
    shape = x.shape
    outer = 1
    for i in range(axis):
        outer *= shape[i]
    src_len = shape[axis]
    shape[axis] = length
    out = _new(x.dtype, shape, x)
    if out.num_bytes:
        seg = x.num_bytes // outer // src_len  # bytes of one index of the axis
        lib = _lib_()
        for o in range(outer):
            check(lib.axhip_memcpy_d2d(out.data_ptr + o * length * seg, x.data_ptr + (o * src_len + start) * seg,
                                       length * seg), op)
    return out


def copy_bytes(dst: Tensor, dst_offset: int, src: Tensor, src_offset: int, nbytes: int) -> None:
    """dst bytes [dst_offset, +nbytes) = src bytes [src_offset, +nbytes), device to device on the current
    stream (the axis-0 copy Concat is made of, src/ops/cuda/sequence.cu:500-518).  Used by the KV-cache
    components to append rows in place."""
    op = "copy_bytes"
    _need_hip(op, dst, src)
    if min(dst_offset, src_offset, nbytes) < 0 or dst_offset + nbytes > dst.num_bytes or src_offset + nbytes > src.num_bytes:
        raise AxhipError(op, Status.INVALID_ARGUMENT)
    if nbytes:
        check(_lib_().axhip_memcpy_d2d(dst.data_ptr + dst_offset, src.data_ptr + src_offset, nbytes), op)


def kv_append(k_new: Tensor, v_new: Tensor, k_cache: Tensor, v_cache: Tensor, pos: Tensor) -> None:
    """In place: cache[b,h,pos[b],:] = new[b,h,:] for K and V.  Replaces the concat-append of
    DynamicKVCache.update (axono/python/axono/nn/kv_cache.py:96-102) for a static cache."""
    op = "kv_append"
    _need_hip(op, k_new, v_new, k_cache, v_cache, pos)
    if k_cache.ndim != 4 or k_new.dtype != k_cache.dtype or v_new.dtype != v_cache.dtype or k_cache.dtype != v_cache.dtype:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    B, hkv, lmax, d = k_cache.shape
    if v_cache.shape != k_cache.shape or k_new.num_elements != B * hkv * d or v_new.num_elements != B * hkv * d:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    if pos.dtype not in (DataType.INT32, DataType.INT64) or pos.num_elements != B:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    check(_lib_().axhip_kv_append(k_new.data_ptr, v_new.data_ptr, k_cache.data_ptr, v_cache.data_ptr, pos.data_ptr,
                                  int(pos.dtype), k_cache.num_bytes // max(k_cache.num_elements, 1), B, hkv, lmax, d,
                                  current_stream()), op)


# ---- fused / row-wise --------------------------------------------------------------------------
def silu_mul(gate: Tensor, up: Tensor) -> Tensor:
    """nanobind_module.cpp:1031-1051 -> SiluMul (src/ops/cuda/fused.cu:76-89)."""
    op = "silu_mul"
    _need_hip(op, gate, up)
    if gate.dtype not in _FLOATS or up.dtype != gate.dtype or gate.shape != up.shape:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    out = _new(gate.dtype, gate.shape, gate)
    check(_lib_().axhip_silu_mul(gate.data_ptr, up.data_ptr, out.data_ptr, int(gate.dtype), gate.num_elements,
                                 current_stream()), op)
    return out


def add_rms_norm(x: Tensor, residual: Tensor, weight: Tensor, eps: float = 1e-6, out_dtype: DataType | None = None):
    """Returns (y, out).  nanobind_module.cpp:1053-1078 -> AddRmsNorm (src/ops/cuda/fused.cu:91-110).
    out_dtype FLOAT16 (FLOAT32 inputs only) stores the normalised result as fp16."""
    op = "add_rms_norm"
    _need_hip(op, x, residual, weight)
    if x.dtype not in _FLOATS or residual.dtype != x.dtype or x.shape != residual.shape:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    if x.ndim < 1:
        raise AxhipError(op, Status.INVALID_ARGUMENT)
    hidden = x.shape[-1]
    if weight.ndim != 1 or weight.shape[0] != hidden or weight.dtype not in _FLOATS:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    odt = DataType(out_dtype) if out_dtype is not None else x.dtype
    y, out = _new(x.dtype, x.shape, x), _new(odt, x.shape, x)
    rows = x.num_elements // hidden if hidden else 0
    check(_lib_().axhip_add_rms_norm_ex(x.data_ptr, residual.data_ptr, weight.data_ptr, float(eps), y.data_ptr,
                                        out.data_ptr, int(x.dtype), int(weight.dtype), int(odt), rows, hidden,
                                        current_stream()), op)
    return y, out


def rms_norm(x: Tensor, weight: Tensor | None, eps: float = 1e-5, out_dtype: DataType | None = None) -> Tensor:
    """nanobind_module.cpp:909-942 (llm ops) -> RmsNorm (src/ops/cpu/llm.cpp:240-264).  An empty or
    missing weight means no scaling."""
    op = "rms_norm"
    has_w = weight is not None and weight.num_elements != 0
    _need_hip(op, x, weight if has_w else None)
    if x.dtype not in _FLOATS:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    if x.ndim < 1:
        raise AxhipError(op, Status.INVALID_ARGUMENT)
    cols = x.shape[-1]
    if has_w and (weight.ndim != 1 or weight.shape[0] != cols or weight.dtype not in _FLOATS):
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    odt = DataType(out_dtype) if out_dtype is not None else x.dtype
    out = _new(odt, x.shape, x)
    rows = x.num_elements // cols if cols else 0
    check(_lib_().axhip_rms_norm_ex(x.data_ptr, weight.data_ptr if has_w else None, float(eps), out.data_ptr,
                                    int(x.dtype), int(weight.dtype) if has_w else int(DataType.FLOAT32), int(odt),
                                    rows, cols, current_stream()), op)
    return out


def add(a: Tensor, b: Tensor) -> Tensor:
    """Same-shape add (the final residual of a decoder layer)."""
    op = "add"
    _need_hip(op, a, b)
    if a.dtype not in _FLOATS or b.dtype != a.dtype:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    if a.shape != b.shape:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    out = _new(a.dtype, a.shape, a)
    check(_lib_().axhip_add(a.data_ptr, b.data_ptr, out.data_ptr, int(a.dtype), a.num_elements, current_stream()), op)
    return out


# ---- rotary ------------------------------------------------------------------------------------
def _rope_check(op, x):
    if x.ndim != 3 or x.dtype not in _FLOATS:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    if x.shape[2] % 2 != 0:
        raise AxhipError(op, Status.INVALID_ARGUMENT)


def rope(x: Tensor, pos_ids: Tensor, theta: float = 10000.0) -> Tensor:
    """nanobind_module.cpp:944-966 -> Rope (src/ops/cpu/sequence.cpp:54-93)."""
    op = "rope"
    _need_hip(op, x, pos_ids)
    _rope_check(op, x)
    rows, heads, dim = x.shape
    if pos_ids.num_elements != rows or pos_ids.dtype != DataType.INT64:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    out = _new(x.dtype, x.shape, x)
    check(_lib_().axhip_rope(x.data_ptr, pos_ids.data_ptr, float(theta), out.data_ptr, int(x.dtype), rows, heads,
                             dim, current_stream()), op)
    return out


def rope_qk(q: Tensor, k: Tensor, pos_ids: Tensor, theta: float = 10000.0):
    """rope(q, pos_ids, theta) and rope(k, pos_ids, theta) in one launch (the two calls of a decoder layer,
    examples/vlm/qwen3vl/model.py:358-359, share the positions).  Returns (q_out, k_out); same bits as the
    two separate calls."""
    op = "rope"
    _need_hip(op, q, k, pos_ids)
    _rope_check(op, q)
    _rope_check(op, k)
    rows, hq, dim = q.shape
    if k.shape[0] != rows or k.shape[2] != dim or k.dtype != q.dtype:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    if pos_ids.num_elements != rows or pos_ids.dtype != DataType.INT64:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    qo, ko = _new(q.dtype, q.shape, q), _new(k.dtype, k.shape, k)
    check(_lib_().axhip_rope_qk(q.data_ptr, k.data_ptr, pos_ids.data_ptr, float(theta), qo.data_ptr, ko.data_ptr,
                                int(q.dtype), rows, hq, k.shape[1], dim, current_stream()), op)
    return qo, ko


def rope_with_cos_sin(x: Tensor, cos: Tensor, sin: Tensor) -> Tensor:
    """nanobind_module.cpp:968-990 -> RopeWithCosSin (sequence.cpp:96-135)."""
    op = "rope_with_cos_sin"
    _need_hip(op, x, cos, sin)
    _rope_check(op, x)
    rows, heads, dim = x.shape
    for t in (cos, sin):
        if t.ndim != 2 or t.shape != [rows, dim] or t.dtype != DataType.FLOAT32:
            raise AxhipError(op, Status.SHAPE_MISMATCH)
    out = _new(x.dtype, x.shape, x)
    check(_lib_().axhip_rope_with_cos_sin(x.data_ptr, cos.data_ptr, sin.data_ptr, out.data_ptr, int(x.dtype), rows,
                                          heads, dim, current_stream()), op)
    return out


def rope_thd(x: Tensor, pos: Tensor, inv_freq: Tensor, t_sec: int, h_sec: int, w_sec: int) -> Tensor:
    """nanobind_module.cpp:992-1013 -> RopeThd (sequence.cpp:184-234)."""
    op = "rope_thd"
    _need_hip(op, x, pos, inv_freq)
    _rope_check(op, x)
    rows, heads, dim = x.shape
    if pos.ndim != 2 or pos.shape != [3, rows] or pos.dtype != DataType.INT64:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    if inv_freq.ndim != 1 or inv_freq.shape[0] != dim // 2 or inv_freq.dtype != DataType.FLOAT32:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    out = _new(x.dtype, x.shape, x)
    check(_lib_().axhip_rope_thd(x.data_ptr, pos.data_ptr, inv_freq.data_ptr, int(t_sec), int(h_sec), int(w_sec),
                                 out.data_ptr, int(x.dtype), rows, heads, dim, current_stream()), op)
    return out


def mrope_cos_sin(pos: Tensor, inv_freq: Tensor, h_sec: int, w_sec: int):
    """Returns (cos, sin), each (rows, 2*half) FLOAT32.  nanobind_module.cpp:1080-1105 -> MropeCosSin
    (sequence.cpp:140-182)."""
    op = "mrope_cos_sin"
    _need_hip(op, pos, inv_freq)
    if pos.ndim != 2 or pos.shape[0] != 3 or pos.dtype != DataType.INT64:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    if inv_freq.dtype != DataType.FLOAT32 or inv_freq.ndim != 1:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    rows, half = pos.shape[1], inv_freq.shape[0]
    if half == 0:
        raise AxhipError(op, Status.INVALID_ARGUMENT)
    cos = _new(DataType.FLOAT32, [rows, 2 * half], pos)
    sin = _new(DataType.FLOAT32, [rows, 2 * half], pos)
    check(_lib_().axhip_mrope_cos_sin(pos.data_ptr, inv_freq.data_ptr, int(h_sec), int(w_sec), cos.data_ptr,
                                      sin.data_ptr, rows, half, current_stream()), op)
    return cos, sin


# ---- linear ------------------------------------------------------------------------------------
def _linear_impl(x: Tensor, weight: Tensor, bias: Tensor | None, out_dtype: DataType | None = None) -> Tensor:
    """nanobind_module.cpp:746-791 (linear_impl) -> the fp16 branch of cuda::Linear
    (src/ops/cuda/linear.cu:105-176).  Weight (and bias) FLOAT16; x FLOAT32 (the reference's mixed
    case: result FLOAT32) or FLOAT16 (result FLOAT32 unless out_dtype says FLOAT16)."""
    op = "linear"
    has_b = bias is not None and bias.num_elements != 0
    if x.is_hip != weight.is_hip or (has_b and bias.is_hip != x.is_hip):
        raise RuntimeError("linear: 输入张量不在同一设备上")
    _need_hip(op, x, weight, bias if has_b else None)
    if x.ndim < 1 or weight.ndim != 2:
        raise AxhipError(op, Status.INVALID_ARGUMENT)
    k = x.shape[-1]
    n = weight.shape[0]
    if weight.shape[1] != k or (has_b and (bias.ndim != 1 or bias.shape[0] != n)):
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    rows = x.num_elements // k if k else 0
    if weight.dtype == DataType.FLOAT32:
        # a Linear that has not been cast to fp16: the reference's FLOAT32 branch (linear.cu:178-251), x and bias
        # FLOAT32 like the weight (linear.cu:178-181)
        if x.dtype != DataType.FLOAT32 or (has_b and bias.dtype != DataType.FLOAT32) or \
                (out_dtype is not None and DataType(out_dtype) != DataType.FLOAT32):
            raise RuntimeError("linear: 数据类型不一致")
        out = _new(DataType.FLOAT32, x.shape[:-1] + [n], x)
        check(_lib_().axhip_linear_f32(x.data_ptr, weight.data_ptr, bias.data_ptr if has_b else None, out.data_ptr,
                                       rows, k, n, current_stream()), op)
        return out
    if weight.dtype != DataType.FLOAT16 or x.dtype not in _FLOATS or (has_b and bias.dtype != DataType.FLOAT16):
        # FLOAT64 weights (the reference's third branch) are not provided on hip
        raise RuntimeError("linear: 数据类型不一致")
    odt = DataType(out_dtype) if out_dtype is not None else DataType.FLOAT32
    out = _new(odt, x.shape[:-1] + [n], x)
    lib = _lib_()
    wsb = lib.axhip_linear_f16_workspace_bytes(rows, k, n)
    ws = _workspace(wsb, x) if wsb else None
    check(lib.axhip_linear_f16(x.data_ptr, int(x.dtype), weight.data_ptr, bias.data_ptr if has_b else None,
                               out.data_ptr, int(odt), rows, k, n, ws.data_ptr if ws else None, wsb,
                               current_stream()), op)
    return out


def pack_linear_weight(weight: Tensor, glu: bool = False) -> Tensor:
    """FLOAT16 W [N,K] -> the packed (MFMA fragment order) copy that linear_packed reads.  Done once,
    when a Linear's weights become resident fp16 (the build's extension of cast_linear_fp16)."""
    op = "pack_linear_weight"
    _need_hip(op, weight)
    if weight.dtype != DataType.FLOAT16 or weight.ndim != 2:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    n, k = weight.shape
    lib = _lib_()
    nbytes = lib.axhip_linear_f16_packed_bytes(n, k)
    packed = Tensor(DataType.FLOAT16, [nbytes // 2], weight.device, _zero=False)
    check(lib.axhip_linear_f16_pack(weight.data_ptr, packed.data_ptr, n, k, 1 if glu else 0, current_stream()), op)
    return packed


def linear_packed(x: Tensor, packed: Tensor, n: int, bias: Tensor | None = None,
                  out_dtype: DataType | None = None, glu: bool = False) -> Tensor:
    """x (..., K) . packed W [n, K]^T (+ bias): the HBM-bound skinny kernels up to 32 rows, the
    packed-weight MFMA GEMM above.  glu: W was packed as a fused [gate ; up] projection and the result
    is silu(gate) * up, (..., n/2)."""
    op = "linear"
    has_b = bias is not None and bias.num_elements != 0
    _need_hip(op, x, packed, bias if has_b else None)
    if x.dtype not in _FLOATS or packed.dtype != DataType.FLOAT16 or x.ndim < 1:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    k = x.shape[-1]
    rows = x.num_elements // k if k else 0
    lib = _lib_()
    if packed.num_bytes != lib.axhip_linear_f16_packed_bytes(n, k) or (has_b and bias.num_elements != n):
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    odt = DataType(out_dtype) if out_dtype is not None else DataType.FLOAT32
    out = _new(odt, x.shape[:-1] + [n // 2 if glu else n], x)
    check(lib.axhip_linear_f16_packed(x.data_ptr, int(x.dtype), packed.data_ptr, bias.data_ptr if has_b else None,
                                      out.data_ptr, int(odt), rows, k, n, 1 if glu else 0, current_stream()), op)
    return out


PACKED_MAX_ROWS = 32


def linear(x: Tensor, weight: Tensor, bias: Tensor) -> Tensor:
    return _linear_impl(x, weight, bias)


def linear_nobias(x: Tensor, weight: Tensor) -> Tensor:
    return _linear_impl(x, weight, None)


# ---- index ops ---------------------------------------------------------------------------------
def embedding(ids: Tensor, table: Tensor) -> Tensor:
    """nanobind_module.cpp:1182-1200 -> Embedding (sequence.cpp:18-52); table FLOAT32 or FLOAT16."""
    op = "embedding"
    _need_hip(op, ids, table)
    if ids.ndim < 1 or table.ndim != 2:
        raise AxhipError(op, Status.INVALID_ARGUMENT)
    if table.dtype not in _FLOATS or ids.dtype not in (DataType.INT32, DataType.INT64):
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    vocab, hidden = table.shape
    out = _new(table.dtype, ids.shape + [hidden], table)
    check(_lib_().axhip_embedding(ids.data_ptr, int(ids.dtype), table.data_ptr, out.data_ptr, int(table.dtype),
                                  ids.num_elements, vocab, hidden, current_stream()), op)
    return out


def argmax(x: Tensor) -> Tensor:
    """INT64 index of the first maximum over the last dim (nanobind_module.cpp:1202-1208)."""
    op = "argmax"
    _need_hip(op, x)
    if x.ndim < 1:
        raise AxhipError(op, Status.INVALID_ARGUMENT)
    if x.dtype not in _FLOATS:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    cols = x.shape[-1]
    rows = x.num_elements // cols if cols else 0
    out = _new(DataType.INT64, [rows], x)
    check(_lib_().axhip_argmax(x.data_ptr, out.data_ptr, int(x.dtype), rows, cols, current_stream()), op)
    return out


# ---- glue of the captured decode step -------------------------------------------------------------
def index_add(x: Tensor, delta: int) -> Tensor:
    """x += delta in place (INT32 / INT64), on the device."""
    op = "index_add"
    _need_hip(op, x)
    if x.dtype not in (DataType.INT32, DataType.INT64):
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    check(_lib_().axhip_index_add(x.data_ptr, int(x.dtype), x.num_elements, int(delta), current_stream()), op)
    return x


def embedding_rms_norm(ids: Tensor, table: Tensor, weight: Tensor, eps: float):
    """The opening of a decode step in one launch: (h, xn) with h = embedding(ids, table) widened to FLOAT32 and
    xn = rms_norm(h, weight, eps) stored as FLOAT16 - bit for bit what the three operators give."""
    op = "embedding_rms_norm"
    _need_hip(op, ids, table, weight)
    if ids.ndim < 1 or table.ndim != 2 or weight.ndim != 1 or weight.shape[0] != table.shape[1]:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    if table.dtype != DataType.FLOAT16 or weight.dtype not in _FLOATS or ids.dtype not in (DataType.INT32, DataType.INT64):
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    vocab, hidden = table.shape
    h = _new(DataType.FLOAT32, ids.shape + [hidden], table)
    xn = _new(DataType.FLOAT16, ids.shape + [hidden], table)
    check(_lib_().axhip_embedding_rms_norm(ids.data_ptr, int(ids.dtype), table.data_ptr, weight.data_ptr, int(weight.dtype),
                                           float(eps), h.data_ptr, xn.data_ptr, ids.num_elements, vocab, hidden,
                                           current_stream()), op)
    return h, xn


def decode_layer_tail_supported(m: int, hidden: int, k1: int, inter: int, n_next: int) -> bool:
    """Whether decode_layer_tail is built for these widths on the current device (the 2B text tower's on a device
    with 256 compute units, and a small set for tests)."""
    return hip_available() and bool(_lib_().axhip_decode_layer_tail_supported(m, hidden, k1, inter, n_next))


def decode_layer_tail(attn: Tensor, h_in: Tensor, w_o: Tensor, w_post: Tensor, w_gate_up: Tensor, w_down: Tensor,
                      w_next: Tensor, w_next_linear: Tensor, n_next: int, eps: float, workspace: Tensor,
                      h_out: Tensor | None = None):
    """Everything of a decoder layer behind the attention plus the next layer's fused q/k/v projection, for at
    most 16 rows, as one persistent launch: returns (h_out FLOAT32 [M,H], y FLOAT32 [M,n_next]).  The weights are
    the packed copies (pack_linear_weight; gate+up with glu=True).  h_out, if given, must not be h_in."""
    op = "decode_layer_tail"
    _need_hip(op, attn, h_in, w_o, w_post, w_gate_up, w_down, w_next, w_next_linear, workspace)
    if attn.dtype != DataType.FLOAT16 or h_in.dtype != DataType.FLOAT32 or w_post.dtype != DataType.FLOAT32 or \
            w_next.dtype != DataType.FLOAT32:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    m, hidden = h_in.shape
    k1 = attn.num_elements // m
    inter = w_down.num_elements // hidden
    lib = _lib_()
    need = lib.axhip_decode_layer_tail_workspace_bytes(hidden, inter)
    if workspace.num_bytes < need or w_post.num_elements != hidden or w_next.num_elements != hidden:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    if h_out is None:
        h_out = _new(DataType.FLOAT32, [m, hidden], h_in)
    y = _new(DataType.FLOAT32, [m, n_next], h_in)
    check(lib.axhip_decode_layer_tail(attn.data_ptr, h_in.data_ptr, w_o.data_ptr, w_post.data_ptr, w_gate_up.data_ptr,
                                      w_down.data_ptr, w_next.data_ptr, w_next_linear.data_ptr, h_out.data_ptr, y.data_ptr,
                                      workspace.data_ptr, workspace.num_bytes, m, hidden, k1, inter, n_next, float(eps),
                                      current_stream()), op)
    return h_out, y


def decode_layer_tail_last(attn: Tensor, h_in: Tensor, w_o: Tensor, w_post: Tensor, w_gate_up: Tensor, w_down: Tensor,
                           w_final_norm: Tensor, eps: float, workspace: Tensor, h_out: Tensor | None = None):
    """decode_layer_tail for a model's last layer: ends with the final norm instead of a next projection.  Returns
    (h_out FLOAT32 [M,H], xn FLOAT16 [M,H] = rms_norm(h_out, w_final_norm), the rows the lm_head reads)."""
    op = "decode_layer_tail_last"
    _need_hip(op, attn, h_in, w_o, w_post, w_gate_up, w_down, w_final_norm, workspace)
    if attn.dtype != DataType.FLOAT16 or h_in.dtype != DataType.FLOAT32 or w_post.dtype != DataType.FLOAT32 or \
            w_final_norm.dtype != DataType.FLOAT32:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    m, hidden = h_in.shape
    k1 = attn.num_elements // m
    inter = w_down.num_elements // hidden
    lib = _lib_()
    need = lib.axhip_decode_layer_tail_workspace_bytes(hidden, inter)
    if workspace.num_bytes < need or w_post.num_elements != hidden or w_final_norm.num_elements != hidden:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    if h_out is None:
        h_out = _new(DataType.FLOAT32, [m, hidden], h_in)
    xn = _new(DataType.FLOAT16, [m, hidden], h_in)
    check(lib.axhip_decode_layer_tail_last(attn.data_ptr, h_in.data_ptr, w_o.data_ptr, w_post.data_ptr, w_gate_up.data_ptr,
                                           w_down.data_ptr, w_final_norm.data_ptr, h_out.data_ptr, xn.data_ptr,
                                           workspace.data_ptr, workspace.num_bytes, m, hidden, k1, inter, float(eps),
                                           current_stream()), op)
    return h_out, xn


def decode_layer_tail_failed_waits(reset: bool = False) -> int:
    """Barrier waits of decode_layer_tail that ran out since the last reset (0 in a healthy process)."""
    n = C.c_uint(0)
    check(_lib_().axhip_decode_layer_tail_status(0, C.byref(n)), "decode_layer_tail_status")
    if reset and n.value:   # (resetting moves the counters: only when something went wrong, with the device idle)
        check(_lib_().axhip_decode_layer_tail_status(1, None), "decode_layer_tail_status")
    return int(n.value)


def decode_advance(next_ids: Tensor, ids: Tensor | None = None, pos: Tensor | None = None, seq_lens: Tensor | None = None,
                   log: Tensor | None = None, counter: Tensor | None = None) -> None:
    """The closing of a greedy decode step in one launch: ids = next_ids, pos += 1 (INT64 [rows, B]),
    seq_lens += 1 (INT32 [B]), log[counter] = next_ids (INT64 [steps, B]), counter += 1 (INT64 [1])."""
    op = "decode_advance"
    _need_hip(op, next_ids)
    B = next_ids.num_elements
    if next_ids.dtype != DataType.INT64 or (ids is not None and ids.dtype != DataType.INT64) or \
            (pos is not None and pos.dtype != DataType.INT64) or (seq_lens is not None and seq_lens.dtype != DataType.INT32) or \
            (log is not None and log.dtype != DataType.INT64) or (counter is not None and counter.dtype != DataType.INT64):
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    for t in (ids, seq_lens):
        if t is not None and t.num_elements != B:
            raise AxhipError(op, Status.SHAPE_MISMATCH)
    if (pos is not None and pos.num_elements % B) or (log is not None and log.num_elements % B):
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    ptr = lambda t: t.data_ptr if t is not None else None
    check(_lib_().axhip_decode_advance(next_ids.data_ptr, ptr(ids), ptr(pos), pos.num_elements // B if pos is not None else 0,
                                       ptr(seq_lens), ptr(log), log.num_elements // B if log is not None else 0, ptr(counter),
                                       B, current_stream()), op)


def silu_mul_fused(gate_up: Tensor, out_dtype: DataType | None = None) -> Tensor:
    """[rows, 2*cols] = [gate | up] -> silu(gate) * up, [rows, cols]; out_dtype FLOAT16 for a FLOAT32
    input stores the result rounded once (for a result that only feeds an fp16 Linear)."""
    op = "silu_mul_fused"
    _need_hip(op, gate_up)
    if gate_up.dtype not in _FLOATS or gate_up.ndim < 1 or gate_up.shape[-1] % 2 != 0:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    cols = gate_up.shape[-1] // 2
    rows = gate_up.num_elements // (2 * cols) if cols else 0
    odt = DataType(out_dtype) if out_dtype is not None else gate_up.dtype
    out = _new(odt, gate_up.shape[:-1] + [cols], gate_up)
    check(_lib_().axhip_silu_mul_fused(gate_up.data_ptr, out.data_ptr, int(gate_up.dtype), int(odt), rows, cols,
                                       current_stream()), op)
    return out


def qkv_norm_rope_append(qkv: Tensor, q_weight: Tensor, k_weight: Tensor, eps: float, pos: Tensor, inv_freq: Tensor,
                         mrope_section, seq_lens: Tensor, k_cache: Tensor, v_cache: Tensor, n_q_heads: int) -> Tensor:
    """qkv FLOAT32 [B, (Hq + 2*Hkv) * D] (fused projection) -> q [B,Hq,D] in the cache dtype; k and v
    are normalised / rotated / converted and appended to the caches at seq_lens[b]."""
    op = "qkv_norm_rope_append"
    _need_hip(op, qkv, q_weight, k_weight, pos, inv_freq, seq_lens, k_cache, v_cache)
    if qkv.dtype != DataType.FLOAT32 or k_cache.ndim != 4 or k_cache.dtype not in _FLOATS or v_cache.dtype != k_cache.dtype:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    B, hkv, lmax, d = k_cache.shape
    hq = int(n_q_heads)
    width = (hq + 2 * hkv) * d
    if qkv.num_elements != B * width or v_cache.shape != k_cache.shape:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    if pos.dtype != DataType.INT64 or pos.shape != [3, B] or seq_lens.dtype != DataType.INT32 or seq_lens.num_elements != B:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    if inv_freq.dtype != DataType.FLOAT32 or inv_freq.num_elements != d // 2:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    for w in (q_weight, k_weight):
        if w is not None and (w.num_elements != d or w.dtype not in _FLOATS):
            raise AxhipError(op, Status.SHAPE_MISMATCH)
    if q_weight is not None and k_weight is not None and q_weight.dtype != k_weight.dtype:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    _, h_sec, w_sec = (list(mrope_section) + [0, 0, 0])[:3]
    q_out = _new(k_cache.dtype, [B, hq, d], qkv)
    base = qkv.data_ptr
    wdt = int(q_weight.dtype) if q_weight is not None else int(DataType.FLOAT32)
    check(_lib_().axhip_qkv_norm_rope_append(
        base, width, base + hq * d * 4, width, base + (hq + hkv) * d * 4, width,
        q_weight.data_ptr if q_weight is not None else None, k_weight.data_ptr if k_weight is not None else None,
        wdt, float(eps), pos.data_ptr, inv_freq.data_ptr, int(h_sec), int(w_sec), seq_lens.data_ptr, q_out.data_ptr,
        k_cache.data_ptr, v_cache.data_ptr, int(k_cache.dtype), B, 1, hq, hkv, d, lmax, current_stream()), op)
    return q_out


TAIL_MAX_ROWS = 16


def prefill_attention(q: Tensor, k_cache: Tensor, v_cache: Tensor, start: Tensor | None = None) -> Tensor:
    """Causal attention of S new tokens per sequence over a static cache that already holds their
    keys / values: q FLOAT16 [B,S,Hq,D], caches FLOAT16 [B,Hkv,rows,D], start INT32 [B] = absolute
    position of query 0 (None: 0).  Returns FLOAT16 [B,S,Hq,D]."""
    op = "scaled_dot_product_attention"
    _need_hip(op, q, k_cache, v_cache, start)
    if q.dtype != DataType.FLOAT16 or k_cache.dtype != DataType.FLOAT16 or v_cache.dtype != DataType.FLOAT16:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    if q.ndim != 4 or k_cache.ndim != 4 or v_cache.shape != k_cache.shape:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    B, S, hq, d = q.shape
    if k_cache.shape[0] != B or k_cache.shape[3] != d:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    if start is not None and (start.dtype != DataType.INT32 or start.num_elements != B):
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    out = _new(DataType.FLOAT16, [B, S, hq, d], q)
    check(_lib_().axhip_prefill_attention(q.data_ptr, k_cache.data_ptr, v_cache.data_ptr,
                                          start.data_ptr if start is not None else None, out.data_ptr,
                                          int(DataType.FLOAT16), B, S, hq, k_cache.shape[1], d, k_cache.shape[2],
                                          current_stream()), op)
    return out


def gqa_decode_attention_qkv(qkv: Tensor, q_weight: Tensor, k_weight: Tensor, eps: float, pos: Tensor, inv_freq: Tensor,
                             mrope_section, seq_lens: Tensor, k_cache: Tensor, v_cache: Tensor, n_q_heads: int,
                             max_len: int | None = None, workspace: Tensor | None = None) -> Tensor:
    """The attention block of one decode step in one launch: qkv FLOAT32 [B, (Hq + 2*Hkv) * D] (fused
    projection) is normalised per head, rotated, its k / v rows appended to the caches at seq_lens[b],
    and the query attends over seq_lens[b] + 1 keys.  Equals qkv_norm_rope_append followed by
    gqa_decode_attention_cache.  Returns [B, Hq, D] in the cache dtype."""
    op = "gqa_decode_attention"
    _need_hip(op, qkv, q_weight, k_weight, pos, inv_freq, seq_lens, k_cache, v_cache, workspace)
    if qkv.dtype != DataType.FLOAT32 or k_cache.ndim != 4 or k_cache.dtype not in _FLOATS or v_cache.dtype != k_cache.dtype:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    B, hkv, rows, d = k_cache.shape
    hq = int(n_q_heads)
    width = (hq + 2 * hkv) * d
    if qkv.num_elements != B * width or v_cache.shape != k_cache.shape:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    if pos.dtype != DataType.INT64 or pos.shape != [3, B] or seq_lens.dtype != DataType.INT32 or seq_lens.num_elements != B:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    if inv_freq.dtype != DataType.FLOAT32 or inv_freq.num_elements != d // 2:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    for w in (q_weight, k_weight):
        if w is not None and (w.num_elements != d or w.dtype not in _FLOATS):
            raise AxhipError(op, Status.SHAPE_MISMATCH)
    if q_weight is not None and k_weight is not None and q_weight.dtype != k_weight.dtype:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    _, h_sec, w_sec = (list(mrope_section) + [0, 0, 0])[:3]
    bound = int(max_len) if max_len else rows
    lib = _lib_()
    wsb = lib.axhip_gqa_decode_workspace_bytes(B, hq, hkv, d, bound)
    if workspace is None:
        workspace = _new(DataType.INT8, [max(wsb, 256)], qkv)
    out = _new(k_cache.dtype, [B, hq, d], qkv)
    base = qkv.data_ptr
    wdt = int(q_weight.dtype) if q_weight is not None else int(DataType.FLOAT32)
    check(lib.axhip_gqa_decode_qkv(
        base, width, base + hq * d * 4, width, base + (hq + hkv) * d * 4, width,
        q_weight.data_ptr if q_weight is not None else None, k_weight.data_ptr if k_weight is not None else None,
        wdt, float(eps), pos.data_ptr, inv_freq.data_ptr, int(h_sec), int(w_sec), seq_lens.data_ptr,
        k_cache.data_ptr, v_cache.data_ptr, out.data_ptr, workspace.data_ptr, workspace.num_bytes, int(k_cache.dtype),
        B, hq, hkv, d, rows, bound, current_stream()), op)
    return out


def gqa_decode_attention_qkv_paged(qkv: Tensor, q_weight: Tensor, k_weight: Tensor, eps: float, pos: Tensor, inv_freq: Tensor,
                                   mrope_section, seq_lens: Tensor, k_pool: Tensor, v_pool: Tensor, page_table: Tensor,
                                   n_q_heads: int, max_len: int, workspace: Tensor | None = None) -> Tensor:
    """gqa_decode_attention_qkv over a paged cache (pools (n_pages,Hkv,128,D) FLOAT16, page_table INT32
    (B,max_pages)): the new token's k / v row is written through the table at position seq_lens[b] (its page
    must be reserved) and the query attends over seq_lens[b] + 1 keys.  Same bits as the dense form."""
    op = "gqa_decode_attention"
    _need_hip(op, qkv, q_weight, k_weight, pos, inv_freq, seq_lens, k_pool, v_pool, page_table, workspace)
    if qkv.dtype != DataType.FLOAT32 or k_pool.ndim != 4 or k_pool.dtype != DataType.FLOAT16 or v_pool.dtype != k_pool.dtype:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    n_pages, hkv, pk, d = k_pool.shape
    B = seq_lens.num_elements
    hq = int(n_q_heads)
    width = (hq + 2 * hkv) * d
    if pk != PAGE_KEYS or qkv.num_elements != B * width or v_pool.shape != k_pool.shape:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    if pos.dtype != DataType.INT64 or pos.shape != [3, B] or seq_lens.dtype != DataType.INT32:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    if page_table.dtype != DataType.INT32 or page_table.ndim != 2 or page_table.shape[0] != B:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    if inv_freq.dtype != DataType.FLOAT32 or inv_freq.num_elements != d // 2:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    for w in (q_weight, k_weight):
        if w is not None and (w.num_elements != d or w.dtype not in _FLOATS):
            raise AxhipError(op, Status.SHAPE_MISMATCH)
    if q_weight is not None and k_weight is not None and q_weight.dtype != k_weight.dtype:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    _, h_sec, w_sec = (list(mrope_section) + [0, 0, 0])[:3]
    bound = int(max_len)
    lib = _lib_()
    wsb = lib.axhip_gqa_decode_workspace_bytes(B, hq, hkv, d, bound)
    if workspace is None:
        workspace = _new(DataType.INT8, [max(wsb, 256)], qkv)
    out = _new(k_pool.dtype, [B, hq, d], qkv)
    base = qkv.data_ptr
    wdt = int(q_weight.dtype) if q_weight is not None else int(DataType.FLOAT32)
    check(lib.axhip_gqa_decode_qkv_paged(
        base, width, base + hq * d * 4, width, base + (hq + hkv) * d * 4, width,
        q_weight.data_ptr if q_weight is not None else None, k_weight.data_ptr if k_weight is not None else None,
        wdt, float(eps), pos.data_ptr, inv_freq.data_ptr, int(h_sec), int(w_sec), seq_lens.data_ptr,
        k_pool.data_ptr, v_pool.data_ptr, page_table.data_ptr, out.data_ptr, workspace.data_ptr, workspace.num_bytes,
        int(k_pool.dtype), B, hq, hkv, d, bound, page_table.shape[1], n_pages, current_stream()), op)
    return out


def kv_dense_to_paged(k_dense: Tensor, v_dense: Tensor, k_pool: Tensor, v_pool: Tensor, page_table: Tensor,
                      lens: Tensor | None = None, table_row: int | None = None) -> None:
    """Copies the first lens[b] key positions (all rows when lens is None) of dense caches [B,Hkv,rows,D] into
    the pages the table names.  table_row: the dense caches hold ONE sequence, the one of that table row."""
    op = "kv_dense_to_paged"
    _need_hip(op, k_dense, v_dense, k_pool, v_pool, page_table, lens)
    if k_dense.ndim != 4 or k_pool.ndim != 4 or k_dense.dtype != k_pool.dtype or v_dense.dtype != k_pool.dtype or v_pool.dtype != k_pool.dtype:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    B, hkv, rows, d = k_dense.shape
    n_pages, hkv_p, pk, d_p = k_pool.shape
    tb, max_pages = page_table.shape
    tbl = page_table.data_ptr
    lens_ptr = lens.data_ptr if lens is not None else None
    if table_row is not None:
        if B != 1 or not 0 <= table_row < tb:
            raise AxhipError(op, Status.INVALID_ARGUMENT)
        tbl += table_row * max_pages * 4
        if lens is not None:
            lens_ptr += table_row * 4
    elif tb != B:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    if pk != PAGE_KEYS or hkv_p != hkv or d_p != d or v_dense.shape != k_dense.shape or v_pool.shape != k_pool.shape:
        raise AxhipError(op, Status.SHAPE_MISMATCH)
    if lens is not None and lens.dtype != DataType.INT32:
        raise AxhipError(op, Status.UNSUPPORTED_TYPE)
    check(_lib_().axhip_kv_dense_to_paged(k_dense.data_ptr, v_dense.data_ptr, k_pool.data_ptr, v_pool.data_ptr, tbl, lens_ptr,
                                          k_pool.num_bytes // max(k_pool.num_elements, 1), B, hkv, rows, d, max_pages, n_pages,
                                          current_stream()), op)


# ---- graph capture -------------------------------------------------------------------------------
def set_ticket_lane(lane: int) -> None:
    """Attention and wide argmax launches issued (or captured) from now on by this thread use the
    ticket counters of `lane` (0..7); launches that overlap in time on the device need different lanes."""
    check(_lib_().axhip_set_ticket_lane(int(lane)), "set_ticket_lane")


def set_plan_reuse(mode: int) -> None:
    """The attention launches of one decode step deal the same lengths the same way: mode 1 makes the next
    gqa_decode_qkv launches of this thread leave what they dealt in a device table, mode 2 makes them take it
    from there, mode 0 (default) is every launch for itself.  A mode-2 launch must follow a mode-1 launch of the
    same lengths (same seq_lens tensor and contents) and shape on the same stream."""
    check(_lib_().axhip_set_plan_reuse(int(mode)), "set_plan_reuse")


class HIPGraph:
    """The binding-level graph object (the reference's CUDAGraph class, nanobind_module.cpp:1228-1324):
    capture(fn) = reset the capture pool, run fn once with pool recording on, begin capture, run fn
    again (allocations pop the recorded blocks), end capture and instantiate."""

    def __init__(self):
        self._graph = None
        self._nodes = 0

    def capture(self, fn) -> None:
        lib = _lib_()
        self.reset()
        check(lib.axhip_capture_pool_reset(), "capture")
        check(lib.axhip_capture_pool_set_recording(1), "capture")
        try:
            fn()  # warm-up: registers every allocation size -> block
        finally:
            lib.axhip_capture_pool_set_recording(0)
        stream = C.c_void_p()
        check(lib.axhip_graph_begin_capture(C.byref(stream)), "capture")
        try:
            fn()
        except BaseException:
            lib.axhip_graph_abort_capture(stream)
            lib.axhip_capture_pool_reset()
            raise
        self._finalize(stream)
        lib.axhip_capture_pool_reset()

    def _finalize(self, stream) -> None:
        lib = _lib_()
        g, n = C.c_void_p(), C.c_size_t(0)
        rc = lib.axhip_graph_end_capture(stream, C.byref(g), C.byref(n))
        if rc == Status.INVALID_ARGUMENT:
            raise RuntimeError("CUDAGraph: 捕获到空图 (capture 体内没有任何设备算子)")
        check(rc, "capture")
        self._graph, self._nodes = g, int(n.value)

    def replay(self) -> None:
        if self._graph is None:
            raise RuntimeError("replay() 之前必须先 capture()")
        check(_lib_().axhip_graph_replay(self._graph), "replay")

    def launch(self) -> None:
        """Enqueue one replay without waiting (a serving loop syncs once per many steps)."""
        if self._graph is None:
            raise RuntimeError("launch() 之前必须先 capture()")
        check(_lib_().axhip_graph_launch(self._graph), "launch")

    def launch_async(self) -> None:
        """Enqueue one replay on the graph's own stream, unordered against the default stream: replays
        of different graphs run side by side.  Such graphs are captured under different ticket lanes
        (set_ticket_lane) and ordered with sync()."""
        if self._graph is None:
            raise RuntimeError("launch_async() 之前必须先 capture()")
        check(_lib_().axhip_graph_launch_async(self._graph), "launch")

    def sync(self) -> None:
        if self._graph is not None:
            check(_lib_().axhip_graph_sync(self._graph), "sync")

    def reset(self) -> None:
        if self._graph is not None:
            _lib_().axhip_graph_destroy(self._graph)
            self._graph, self._nodes = None, 0

    @property
    def is_captured(self) -> bool:
        return self._graph is not None

    @property
    def num_nodes(self) -> int:
        return self._nodes

    def __del__(self):
        try:
            self.reset()
        except Exception:
            pass


CUDAGraph = HIPGraph  # the name the reference's Python layer asks its native module for


def _graph_begin_capture():
    stream = C.c_void_p()
    check(_lib_().axhip_graph_begin_capture(C.byref(stream)), "_graph_begin_capture")
    return stream


def _graph_end_capture(stream, graph: HIPGraph) -> None:
    graph.reset()
    graph._finalize(stream)


def _graph_abort_capture(stream) -> None:
    _lib_().axhip_graph_abort_capture(stream)


__all__ = [n for n in dir() if not n.startswith("_")] + ["_graph_begin_capture", "_graph_end_capture",
                                                         "_graph_abort_capture"]
# keep `hip_available` importable from here as the counterpart of cuda_available
hip_available = hip_available
