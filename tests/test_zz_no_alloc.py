"""axhip_gqa_decode_static, the decode-attention entry point that allocates nothing: its split partials
live in a static device array of the library instead of a caller's workspace.  Through the C ABI it must
give the bits axhip_gqa_decode gives (same kernels, same plan), on two calls in a row that share the
array - the second with a smaller input - and against the CPU oracle to the fp16 bar; a plan that needs
more scratch than the array holds is refused before anything is launched."""
import ctypes as C

import numpy as np
import pytest

from axono_amd import _lib
from axono_amd.device import DeviceBuffer, check, synchronize
from oracle import port

pytestmark = pytest.mark.gpu

F16, F32 = 4, 5
STATIC_BYTES = 48 << 20


def _inputs(seed, B, Hq, Hkv, D, L, lens, dtype):
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((B, Hq, D)).astype(np.float32).astype(dtype)
    k = rng.standard_normal((B, Hkv, L, D)).astype(np.float32).astype(dtype)
    v = rng.standard_normal((B, Hkv, L, D)).astype(np.float32).astype(dtype)
    return q, k, v, np.asarray(lens, np.int32)


def _both(lib, q, k, v, lens):
    """(result of axhip_gqa_decode with a caller's workspace, result of axhip_gqa_decode_static)."""
    B, Hq, D = q.shape
    _, Hkv, L, _ = k.shape
    code = F16 if q.dtype == np.float16 else F32
    dq, dk, dv, dl = (DeviceBuffer.from_numpy(a) for a in (q, k, v, lens))
    out_ws, out_st = DeviceBuffer(q.nbytes, zero=True), DeviceBuffer(q.nbytes, zero=True)
    wsb = lib.axhip_gqa_decode_workspace_bytes(B, Hq, Hkv, D, L)
    ws = DeviceBuffer(max(wsb, 256))
    strides = (Hkv * L * D, L * D, D)
    check(lib.axhip_gqa_decode(dq.ptr, dk.ptr, dv.ptr, dl.ptr, out_ws.ptr, ws.ptr, wsb, code, B, Hq, Hkv, D, L,
                               *strides, None), "gqa_decode")
    # everything is allocated by now: the call under test gets pointers only
    check(lib.axhip_gqa_decode_static(dq.ptr, dk.ptr, dv.ptr, dl.ptr, out_st.ptr, code, B, Hq, Hkv, D, L,
                                      *strides, None), "gqa_decode_static")
    synchronize()
    return out_ws.download(q.dtype, q.shape), out_st.download(q.dtype, q.shape)


def test_static_scratch_entry_point_matches_the_workspace_one_twice_in_a_row():
    lib = _lib.load()
    # first call: ragged batch whose sequences are cut into several key ranges (partials + in-kernel merge)
    q, k, v, lens = _inputs(21, 4, 16, 8, 128, 3000, [3000, 1, 2049, 777], np.float16)
    n_splits, chunk = C.c_int(0), C.c_int(0)
    lib.axhip_gqa_decode_plan(4, 16, 8, 3000, C.byref(n_splits), C.byref(chunk))
    assert n_splits.value > 1, "the case must exercise the scratch"
    want_ws, got = _both(lib, q, k, v, lens)
    np.testing.assert_array_equal(got.view(np.uint16), want_ws.view(np.uint16))
    ref = port.gqa_decode_cache_native(q, k, v, lens)
    assert np.abs(got.astype(np.float32) - ref).max() <= 2e-3
    # second call, smaller: the array still holds the first call's partials
    q2, k2, v2, lens2 = _inputs(22, 2, 16, 8, 128, 700, [700, 513], np.float16)
    want2, got2 = _both(lib, q2, k2, v2, lens2)
    np.testing.assert_array_equal(got2.view(np.uint16), want2.view(np.uint16))
    ref2 = port.gqa_decode_cache_native(q2, k2, v2, lens2)
    assert np.abs(got2.astype(np.float32) - ref2).max() <= 2e-3
    # third: fp32, the reference's own shape (one sequence), again smaller
    q3, k3, v3, lens3 = _inputs(23, 1, 16, 8, 128, 1024, [1024], np.float32)
    want3, got3 = _both(lib, q3, k3, v3, lens3)
    np.testing.assert_array_equal(got3.view(np.uint32), want3.view(np.uint32))
    assert np.abs(got3 - port.gqa_decode_cache_native(q3, k3, v3, lens3)).max() <= 1e-5


def test_static_scratch_entry_point_refuses_what_does_not_fit():
    lib = _lib.load()
    # B = 64 sequences of Hq = 128 heads: 64 * 128 * 64 ranges * 130 floats = 273 MB of partials
    B, Hq, Hkv, D, L = 64, 128, 64, 128, 4096
    assert B * Hq * 64 * (D + 2) * 4 > STATIC_BYTES
    one = DeviceBuffer(256)
    rc = lib.axhip_gqa_decode_static(one.ptr, one.ptr, one.ptr, None, one.ptr, F16, B, Hq, Hkv, D, L,
                                     Hkv * L * D, L * D, D, None)
    assert rc == 2  # OUT_OF_MEMORY: refused on the host, nothing launched
    # and the same checks as the workspace form before that
    assert lib.axhip_gqa_decode_static(None, None, None, None, None, F16, 1, 16, 5, 128, 16, 0, 0, 0, None) == 4
    synchronize()


def _device_free_bytes():
    """Free device memory as the HIP runtime reports it (the runtime library this process already has loaded)."""
    hip = C.CDLL("libamdhip64.so")
    free_b, total_b = C.c_size_t(0), C.c_size_t(0)
    assert hip.hipMemGetInfo(C.byref(free_b), C.byref(total_b)) == 0
    return free_b.value


def test_static_scratch_entry_point_allocates_nothing_and_replays_from_a_graph():
    """What the entry point is for: no device memory is taken or returned across the call (driver's free bytes,
    the library's handed-out and cached byte counts), and it can be recorded into a hipGraph - with several key
    ranges per sequence, i.e. partials in the static array and the in-kernel merge - whose replays, with eager work
    between them that overwrites the array, give the eager bits every time."""
    lib = _lib.load()
    q, k, v, lens = _inputs(31, 3, 16, 8, 128, 2600, [2600, 1300, 2049], np.float16)
    B, Hq, D = q.shape
    _, Hkv, L, _ = k.shape
    dq, dk, dv, dl = (DeviceBuffer.from_numpy(a) for a in (q, k, v, lens))
    out_e, out_g = DeviceBuffer(q.nbytes, zero=True), DeviceBuffer(q.nbytes, zero=True)
    strides = (Hkv * L * D, L * D, D)

    def call(out, stream):
        check(lib.axhip_gqa_decode_static(dq.ptr, dk.ptr, dv.ptr, dl.ptr, out.ptr, F16, B, Hq, Hkv, D, L, *strides, stream),
              "gqa_decode_static")

    call(out_e, None)        # first call on this device (symbol address looked up) stays outside the measurement
    synchronize()
    before = (_device_free_bytes(), lib.axhip_allocated_bytes(), lib.axhip_cached_bytes())
    call(out_e, None)
    synchronize()
    after = (_device_free_bytes(), lib.axhip_allocated_bytes(), lib.axhip_cached_bytes())
    assert after == before, (before, after)
    eager = out_e.download(np.uint16, q.shape)
    ref = port.gqa_decode_cache_native(q, k, v, lens)
    assert np.abs(eager.view(np.float16).astype(np.float32) - ref).max() <= 2e-3

    stream, graph, nodes = C.c_void_p(), C.c_void_p(), C.c_size_t(0)
    check(lib.axhip_graph_begin_capture(C.byref(stream)), "begin_capture")
    try:
        call(out_g, stream)
    except Exception:
        lib.axhip_graph_abort_capture(stream)
        raise
    check(lib.axhip_graph_end_capture(stream, C.byref(graph), C.byref(nodes)), "end_capture")
    assert nodes.value >= 1
    # (the graph object and its stream take driver memory of their own; the library's allocator hands out nothing)
    assert (lib.axhip_allocated_bytes(), lib.axhip_cached_bytes()) == (before[1], before[2])
    # a different, smaller problem between replays leaves other partials in the static array
    q2, k2, v2, lens2 = _inputs(32, 2, 16, 8, 128, 900, [900, 514], np.float16)
    try:
        for _ in range(3):
            check(lib.axhip_fill_zero(out_g.ptr, q.nbytes), "fill_zero")
            check(lib.axhip_graph_replay(graph), "replay")
            np.testing.assert_array_equal(out_g.download(np.uint16, q.shape), eager)
            want2, got2 = _both(lib, q2, k2, v2, lens2)
            np.testing.assert_array_equal(got2.view(np.uint16), want2.view(np.uint16))
    finally:
        check(lib.axhip_graph_destroy(graph), "graph_destroy")
