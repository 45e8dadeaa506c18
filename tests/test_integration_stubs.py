"""The operator stubs and the binding branch that INTEGRATION.md describes, compiled for real: plain g++ over
tests/integration_stubs/*.cpp with the reference's own headers (core::Tensor, core::Status, core::DataType) and this
repository's include/axhip.h.  A signature change in the C ABI, a misuse of core::Tensor or a drift of the
enumeration values fails here, on a machine without a GPU.  Needs the reference tree for its headers; skipped
without it (as oracle/Makefile skips the `ref` target)."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
STUBS = os.path.join(ROOT, "tests", "integration_stubs")
REF_INCLUDE = os.environ.get("AXONO_REFERENCE", "/root/reference") + "/include"
SOURCES = ("hip_ops.cpp", "binding_branch.cpp")

needs_reference = pytest.mark.skipif(not os.path.isfile(os.path.join(REF_INCLUDE, "axono", "core", "tensor.h")),
                                     reason="the reference's headers are not on this machine")
needs_gxx = pytest.mark.skipif(shutil.which("g++") is None, reason="no g++")


def _compile(src, out):
    cmd = ["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-fPIC", "-c", "-I" + REF_INCLUDE,
           "-I" + os.path.join(ROOT, "include"), "-I" + STUBS, os.path.join(STUBS, src), "-o", out]
    return subprocess.run(cmd, capture_output=True, text=True)


@needs_reference
@needs_gxx
@pytest.mark.parametrize("src", SOURCES)
def test_stub_compiles_against_the_reference_headers_and_the_c_abi(src, tmp_path):
    r = _compile(src, str(tmp_path / (src + ".o")))
    assert r.returncode == 0, r.stderr


@needs_reference
@needs_gxx
def test_every_entry_point_the_stubs_call_is_exported_by_the_library(tmp_path):
    from axono_amd import _lib

    lib = _lib.load()
    called = set()
    for src in SOURCES:
        obj = str(tmp_path / (src + ".o"))
        assert _compile(src, obj).returncode == 0
        nm = subprocess.run(["nm", "-u", obj], capture_output=True, text=True, check=True).stdout
        called |= set(re.findall(r"\b(axhip_\w+)\b", nm))
    # one C-ABI call per operator of the table in INTEGRATION.md, plus the runtime calls of the binding branch
    for must in ("axhip_gqa_decode", "axhip_sdpa", "axhip_silu_mul", "axhip_add_rms_norm", "axhip_rms_norm", "axhip_rope",
                 "axhip_rope_with_cos_sin", "axhip_rope_thd", "axhip_mrope_cos_sin", "axhip_concat", "axhip_linear_f16",
                 "axhip_embedding", "axhip_argmax", "axhip_add", "axhip_cast", "axhip_alloc", "axhip_free",
                 "axhip_graph_begin_capture", "axhip_graph_end_capture", "axhip_graph_replay", "axhip_graph_destroy",
                 "axhip_capture_pool_reset", "axhip_capture_pool_set_recording", "axhip_current_stream"):
        assert must in called, must
    for name in sorted(called):
        assert hasattr(lib, name), name


@needs_reference
@needs_gxx
def test_a_changed_signature_is_caught(tmp_path):
    """The check has teeth: the same stub against a header whose axhip_gqa_decode lost an argument does not compile."""
    inc = tmp_path / "include"
    inc.mkdir()
    text = open(os.path.join(ROOT, "include", "axhip.h")).read()
    broken = text.replace("int max_len, int64_t stride_b, int64_t stride_h, int64_t stride_s,\n                               axhip_stream stream);",
                          "int max_len, int64_t stride_b, int64_t stride_h,\n                               axhip_stream stream);", 1)
    assert broken != text
    (inc / "axhip.h").write_text(broken)
    cmd = ["g++", "-std=c++17", "-fsyntax-only", "-I" + REF_INCLUDE, "-I" + str(inc), "-I" + STUBS,
           os.path.join(STUBS, "hip_ops.cpp")]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode != 0 and "axhip_gqa_decode" in r.stderr
