"""ctypes binding of libaxhip.so (the C ABI declared in include/axhip.h).

The library is the product: if it cannot be loaded this module raises, there is no fallback path.
It is built in-tree by `python -m axono_amd.build`; when no built library exists at all, loading
builds it once.
"""
from __future__ import annotations

import ctypes as C
import os

from . import build as _build

LIB_PATH = _build.LIB_PATH

c_vp = C.c_void_p
c_i = C.c_int
c_i64 = C.c_int64
c_sz = C.c_size_t
c_f = C.c_float

# name -> (restype, argtypes); mirrors include/axhip.h declaration by declaration
PROTOTYPES = {
    "axhip_version": (C.c_char_p, []),
    "axhip_device_count": (c_i, [C.POINTER(c_i)]),
    "axhip_set_device": (c_i, [c_i]),
    "axhip_device_info": (c_i, [c_i, C.c_char_p, c_sz, C.POINTER(c_i), C.POINTER(c_sz), C.POINTER(c_i)]),
    "axhip_alloc": (c_i, [c_sz, c_i, C.POINTER(c_vp)]),
    "axhip_free": (c_i, [c_vp]),
    "axhip_block_is_capture_owned": (c_i, [c_vp, C.POINTER(c_i)]),
    "axhip_cached_bytes": (c_sz, []),
    "axhip_set_cache_budget": (c_i, [c_sz]),
    "axhip_cache_budget": (c_sz, []),
    "axhip_empty_cache": (c_i, []),
    "axhip_allocated_bytes": (c_sz, []),
    "axhip_memcpy_h2d": (c_i, [c_vp, c_vp, c_sz]),
    "axhip_memcpy_d2h": (c_i, [c_vp, c_vp, c_sz]),
    "axhip_memcpy_d2d": (c_i, [c_vp, c_vp, c_sz]),
    "axhip_fill_zero": (c_i, [c_vp, c_sz]),
    "axhip_current_stream": (c_vp, []),
    "axhip_is_capturing": (c_i, []),
    "axhip_synchronize": (c_i, []),
    "axhip_graph_begin_capture": (c_i, [C.POINTER(c_vp)]),
    "axhip_graph_end_capture": (c_i, [c_vp, C.POINTER(c_vp), C.POINTER(c_sz)]),
    "axhip_graph_abort_capture": (c_i, [c_vp]),
    "axhip_graph_launch": (c_i, [c_vp]),
    "axhip_graph_launch_async": (c_i, [c_vp]),
    "axhip_graph_replay": (c_i, [c_vp]),
    "axhip_set_ticket_lane": (c_i, [c_i]),
    "axhip_ticket_lane": (c_i, []),
    "axhip_set_plan_reuse": (c_i, [c_i]),
    "axhip_plan_reuse": (c_i, []),
    "axhip_reset_tickets": (c_i, []),
    "axhip_graph_sync": (c_i, [c_vp]),
    "axhip_graph_destroy": (c_i, [c_vp]),
    "axhip_capture_pool_reset": (c_i, []),
    "axhip_capture_pool_set_recording": (c_i, [c_i]),
    "axhip_event_create": (c_i, [C.POINTER(c_vp)]),
    "axhip_event_record": (c_i, [c_vp, c_vp]),
    "axhip_event_elapsed_ms": (c_i, [c_vp, c_vp, C.POINTER(c_f)]),
    "axhip_event_destroy": (c_i, [c_vp]),
    "axhip_gqa_decode_workspace_bytes": (c_sz, [c_i, c_i, c_i, c_i, c_i]),
    "axhip_gqa_decode_plan": (None, [c_i, c_i, c_i, c_i, C.POINTER(c_i), C.POINTER(c_i)]),
    "axhip_gqa_decode_tune": (None, [c_i, c_i]),
    "axhip_gqa_decode": (c_i, [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_sz, c_i, c_i, c_i, c_i, c_i, c_i,
                               c_i64, c_i64, c_i64, c_vp]),
    "axhip_gqa_decode_static": (c_i, [c_vp, c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i, c_i, c_i, c_i,
                                      c_i64, c_i64, c_i64, c_vp]),
    "axhip_gqa_decode_paged": (c_i, [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_sz, c_i, c_i, c_i, c_i, c_i, c_i, c_i, c_i,
                                     c_vp]),
    "axhip_kv_append_paged": (c_i, [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i, c_i, c_i, c_i, c_i, c_i, c_vp]),
    "axhip_kv_dense_to_paged": (c_i, [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i, c_i, c_i, c_i, c_i, c_vp]),
    "axhip_sdpa": (c_i, [c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i, c_i, c_i, c_i, c_i, c_vp]),
    "axhip_kv_append": (c_i, [c_vp, c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i, c_i, c_i, c_i, c_vp]),
    "axhip_concat": (c_i, [c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_vp]),
    "axhip_add_rms_norm": (c_i, [c_vp, c_vp, c_vp, c_f, c_vp, c_vp, c_i, c_i, c_i64, c_i64, c_vp]),
    "axhip_add_rms_norm_ex": (c_i, [c_vp, c_vp, c_vp, c_f, c_vp, c_vp, c_i, c_i, c_i, c_i64, c_i64, c_vp]),
    "axhip_rms_norm_ex": (c_i, [c_vp, c_vp, c_f, c_vp, c_i, c_i, c_i, c_i64, c_i64, c_vp]),
    "axhip_silu_mul": (c_i, [c_vp, c_vp, c_vp, c_i, c_i64, c_vp]),
    "axhip_rms_norm": (c_i, [c_vp, c_vp, c_f, c_vp, c_i, c_i, c_i64, c_i64, c_vp]),
    "axhip_add": (c_i, [c_vp, c_vp, c_vp, c_i, c_i64, c_vp]),
    "axhip_transpose": (c_i, [c_vp, c_vp, c_i, c_i64, c_i64, c_i64, c_i64, c_i64, c_vp]),
    "axhip_cast": (c_i, [c_vp, c_i, c_vp, c_i, c_i64, c_vp]),
    "axhip_rope": (c_i, [c_vp, c_vp, c_f, c_vp, c_i, c_i64, c_i64, c_i64, c_vp]),
    "axhip_rope_qk": (c_i, [c_vp, c_vp, c_vp, c_f, c_vp, c_vp, c_i, c_i64, c_i64, c_i64, c_i64, c_vp]),
    "axhip_rope_thd": (c_i, [c_vp, c_vp, c_vp, c_i, c_i, c_i, c_vp, c_i, c_i64, c_i64, c_i64, c_vp]),
    "axhip_mrope_cos_sin": (c_i, [c_vp, c_vp, c_i, c_i, c_vp, c_vp, c_i64, c_i64, c_vp]),
    "axhip_rope_with_cos_sin": (c_i, [c_vp, c_vp, c_vp, c_vp, c_i, c_i64, c_i64, c_i64, c_vp]),
    "axhip_linear_f16_workspace_bytes": (c_sz, [c_i64, c_i64, c_i64]),
    "axhip_linear_f16_tune": (None, [c_i, c_i, c_i, c_i]),
    "axhip_linear_f16": (c_i, [c_vp, c_i, c_vp, c_vp, c_vp, c_i, c_i64, c_i64, c_i64, c_vp, c_sz, c_vp]),
    "axhip_linear_f32": (c_i, [c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_vp]),
    "axhip_linear_f16_packed_bytes": (c_sz, [c_i64, c_i64]),
    "axhip_linear_f16_pack": (c_i, [c_vp, c_vp, c_i64, c_i64, c_i, c_vp]),
    "axhip_linear_f16_packed": (c_i, [c_vp, c_i, c_vp, c_vp, c_vp, c_i, c_i64, c_i64, c_i64, c_i, c_vp]),
    "axhip_embedding": (c_i, [c_vp, c_i, c_vp, c_vp, c_i, c_i64, c_i64, c_i64, c_vp]),
    "axhip_argmax": (c_i, [c_vp, c_vp, c_i, c_i64, c_i64, c_vp]),
    "axhip_prefill_attention_tune": (None, [c_i]),
    "axhip_prefill_attention": (c_i, [c_vp, c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i, c_i, c_i, c_i, c_i, c_vp]),
    "axhip_gqa_decode_qkv": (c_i, [c_vp, c_i64, c_vp, c_i64, c_vp, c_i64, c_vp, c_vp, c_i, c_f, c_vp, c_vp, c_i, c_i, c_vp,
                                   c_vp, c_vp, c_vp, c_vp, c_sz, c_i, c_i, c_i, c_i, c_i, c_i, c_i, c_vp]),
    "axhip_gqa_decode_qkv_paged": (c_i, [c_vp, c_i64, c_vp, c_i64, c_vp, c_i64, c_vp, c_vp, c_i, c_f, c_vp, c_vp, c_i, c_i, c_vp,
                                         c_vp, c_vp, c_vp, c_vp, c_vp, c_sz, c_i, c_i, c_i, c_i, c_i, c_i, c_i, c_i, c_vp]),
    "axhip_qkv_norm_rope_append": (c_i, [c_vp, c_i64, c_vp, c_i64, c_vp, c_i64, c_vp, c_vp, c_i, c_f, c_vp, c_vp,
                                         c_i, c_i, c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i, c_i, c_i, c_i, c_i, c_vp]),
    "axhip_silu_mul_fused": (c_i, [c_vp, c_vp, c_i, c_i, c_i64, c_i64, c_vp]),
    "axhip_index_add": (c_i, [c_vp, c_i, c_i64, c_i64, c_vp]),
    "axhip_embedding_rms_norm": (c_i, [c_vp, c_i, c_vp, c_vp, c_i, c_f, c_vp, c_vp, c_i64, c_i64, c_i64, c_vp]),
    "axhip_decode_advance": (c_i, [c_vp, c_vp, c_vp, c_i, c_vp, c_vp, c_i64, c_vp, c_i, c_vp]),
    "axhip_decode_layer_tail_supported": (c_i, [c_i, c_i, c_i, c_i, c_i]),
    "axhip_decode_layer_tail_workspace_bytes": (c_sz, [c_i, c_i]),
    "axhip_decode_layer_tail": (c_i, [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_sz,
                                      c_i, c_i, c_i, c_i, c_i, c_f, c_vp]),
    "axhip_decode_layer_tail_last": (c_i, [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_sz,
                                           c_i, c_i, c_i, c_i, c_f, c_vp]),
    "axhip_decode_layer_tail_status": (c_i, [c_i, c_vp]),
    "axhip_decode_layer_tail_tune": (None, [c_i]),
    "axhip_decode_layer_tail_trace": (None, [c_vp]),
}

_lib = None


def load() -> C.CDLL:
    """Loads libaxhip.so and types every entry point.  Raises if the library is unusable."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        _build.build_library()
    try:
        lib = C.CDLL(LIB_PATH)
    except OSError as e:  # pragma: no cover - depends on the machine
        raise RuntimeError(f"libaxhip.so could not be loaded from {LIB_PATH}: {e}") from e
    missing = []
    for name, (res, args) in PROTOTYPES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError:
            missing.append(name)
            continue
        fn.restype = res
        fn.argtypes = args
    if missing:
        raise RuntimeError(f"libaxhip.so at {LIB_PATH} lacks entry points: {missing}")
    _lib = lib
    return lib


def device_count() -> int:
    n = c_i(0)
    load().axhip_device_count(C.byref(n))
    return int(n.value)
