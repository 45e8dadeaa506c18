"""The C-ABI library loads on a machine without a GPU and exports every entry point that
include/axhip.h declares (no compute calls here)."""
import os
import re

from axono_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols(headers=("axhip.h", "axhip_experimental.h")):
    text = "".join(open(os.path.join(ROOT, "include", h)).read() for h in headers)
    return sorted(set(re.findall(r"AXHIP_API\s+[\w\s\*]+?\b(axhip_\w+)\s*\(", text)))


def test_measurement_hooks_are_not_part_of_the_boundary_header():
    boundary = declared_symbols(("axhip.h",))
    assert not [n for n in boundary if n.endswith("_tune")]
    assert not [n for n in boundary if n.endswith("_trace")]
    assert sorted(declared_symbols(("axhip_experimental.h",))) == ["axhip_decode_layer_tail_trace", "axhip_decode_layer_tail_tune",
                                                                   "axhip_gqa_decode_tune", "axhip_linear_f16_tune",
                                                                   "axhip_prefill_attention_tune"]


def test_header_declares_the_path():
    names = declared_symbols()
    for must in ("axhip_gqa_decode", "axhip_kv_append", "axhip_add_rms_norm", "axhip_silu_mul", "axhip_rope",
                 "axhip_rope_thd", "axhip_mrope_cos_sin", "axhip_rope_with_cos_sin", "axhip_linear_f16",
                 "axhip_alloc", "axhip_graph_begin_capture", "axhip_graph_launch"):
        assert must in names
    assert len(names) >= 45


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    for name in declared_symbols():
        assert hasattr(lib, name), name


def test_python_prototypes_cover_the_header():
    assert sorted(_lib.PROTOTYPES) == declared_symbols()


def test_version_and_device_count_without_gpu():
    lib = _lib.load()
    assert lib.axhip_version() == b"0.2.0-hip"
    assert _lib.device_count() >= 0


def test_argument_checks_run_without_a_device():
    """Status codes for malformed calls are decided on the host before anything is launched."""
    lib = _lib.load()
    assert lib.axhip_silu_mul(None, None, None, 2, 8, None) == 3       # UNSUPPORTED_TYPE (INT32)
    assert lib.axhip_silu_mul(None, None, None, 5, 8, None) == 7       # INVALID_PTR
    assert lib.axhip_silu_mul(None, None, None, 5, 0, None) == 0       # empty input is fine
    assert lib.axhip_rope(None, None, 1e4, None, 5, 4, 2, 7, None) == 1  # odd dim
    assert lib.axhip_gqa_decode(None, None, None, None, None, None, 0, 5, 1, 16, 5, 128, 16, 0, 0, 0, None) == 4
    assert lib.axhip_kv_append(None, None, None, None, None, 5, 2, 1, 1, 1, 8, None) == 3  # pos dtype
    assert lib.axhip_gqa_decode_workspace_bytes(32, 16, 8, 128, 8192) > 0
    # entry points added for paged caches, callers that cannot allocate, one-launch RoPE and transpose
    assert lib.axhip_gqa_decode_static(None, None, None, None, None, 5, 1, 16, 5, 128, 16, 0, 0, 0, None) == 4
    assert lib.axhip_gqa_decode_static(None, None, None, None, None, 5, 1, 16, 8, 128, 16, 0, 128, 1024, None) == 7
    assert lib.axhip_gqa_decode_paged(None, None, None, None, None, None, None, 0, 4, 1, 16, 8, 128, 300, 2, 4, None) == 1
    assert lib.axhip_gqa_decode_paged(None, None, None, None, None, None, None, 0, 4, 1, 16, 8, 128, 256, 2, 4, None) == 7
    assert lib.axhip_kv_append_paged(None, None, None, None, None, None, 2, 3, 1, 1, 1, 8, 1, 1, None) == 3   # 3-byte elements
    assert lib.axhip_kv_append_paged(None, None, None, None, None, None, 2, 2, 0, 1, 1, 8, 1, 1, None) == 0   # no sequences
    assert lib.axhip_rope_qk(None, None, None, 1e6, None, None, 5, 4, 2, 1, 7, None) == 1                      # odd head size
    assert lib.axhip_transpose(None, None, 3, 1, 2, 1, 2, 1, None) == 3
    assert lib.axhip_transpose(None, None, 4, 1, 2, 1, 0, 1, None) == 0                                        # no elements
    assert lib.axhip_reset_tickets() == 0                                                                      # no device: nothing to reset
