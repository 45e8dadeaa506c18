"""Per-operator micro-benchmarks of the decode path (HIP-event timing, through the C ABI).

    python -m axono_amd.benchmarks.microbench gqa   [--B 32 --L 8192 --steps 100 --ragged]
    python -m axono_amd.benchmarks.microbench gqa-sweep
    python -m axono_amd.benchmarks.microbench gqa-paged
    python -m axono_amd.benchmarks.microbench copy  [--mib 1024 --steps 20]
    python -m axono_amd.benchmarks.microbench rowops
    python -m axono_amd.benchmarks.microbench linear

Each line reports algorithmic bytes (or flops) over the average launch time and the fraction of
the MI355X peak (HBM 8 TB/s; fp16 dense MFMA 2.5 PFLOP/s).  `copy` is the plain device-to-device
copy kernel of known size that counter readings (FETCH_SIZE / WRITE_SIZE) are scaled against.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import sys

import numpy as np

from axono_amd import _lib
from axono_amd.device import DeviceBuffer, check

HBM_PEAK = 8000.0      # GB/s
MFMA_F16_PEAK = 2500.0  # TFLOP/s dense
F16, F32, I64 = 4, 5, 3


def _time(lib, fn, steps, warmup=5):
    for _ in range(warmup):
        fn()
    check(lib.axhip_synchronize(), "sync")
    e0, e1 = C.c_void_p(), C.c_void_p()
    lib.axhip_event_create(C.byref(e0))
    lib.axhip_event_create(C.byref(e1))
    lib.axhip_event_record(e0, None)
    for _ in range(steps):
        fn()
    lib.axhip_event_record(e1, None)
    ms = C.c_float(0)
    check(lib.axhip_event_elapsed_ms(e0, e1, C.byref(ms)), "elapsed")
    lib.axhip_event_destroy(e0)
    lib.axhip_event_destroy(e1)
    return ms.value / steps * 1e3  # us


ZERO_DATA = False   # --zero-data: operands of all zeros (the same instructions on data that toggles nothing)


def _rand_fill(buf, nbytes, seed):
    rng = np.random.default_rng(seed)
    block = rng.standard_normal(8 * 1024 * 1024).astype(np.float32).astype(np.float16)
    if ZERO_DATA:
        block[:] = 0
    off = 0
    while off < nbytes:
        n = min(block.nbytes, nbytes - off)
        buf.upload(block[: n // 2], off)
        off += n


# When a list is put here, records are appended to it instead of being printed (bench.py collects the
# per-configuration tables of its JSON line this way).
SINK = None


def _emit(rec):
    if SINK is not None:
        SINK.append(rec)
    else:
        print(json.dumps(rec), flush=True)


def collect(fn, *args, **kwargs):
    """Runs one of the bench_* functions and returns the records it would have printed."""
    global SINK
    prev, SINK = SINK, []
    try:
        fn(*args, **kwargs)
        return SINK
    finally:
        SINK = prev


def bench_gqa(lib, B, L, steps, lens=None, n_rot=None, Hq=16, Hkv=8, D=128, tag="gqa", fp32=False,
              token_major=False):
    """token_major: K/V as [B, L, Hkv, D] (the layout of the reference's single-sequence call) instead
    of the cache layout [B, Hkv, L, D]; fp32: FLOAT32 q / K / V / out."""
    elems = B * Hkv * L * D
    esz = 4 if fp32 else 2
    if n_rot is None:  # enough distinct buffers to exceed the 256 MB Infinity Cache several times
        n_rot = max(2, min(8, int(2**30 // (elems * 2 * esz)) + 1))
    kv = []
    for r in range(n_rot):
        kb, vb = DeviceBuffer(elems * esz), DeviceBuffer(elems * esz)
        if fp32:
            blk = np.random.default_rng(r).standard_normal(min(elems, 1 << 22)).astype(np.float32)
            for buf in (kb, vb):
                for off in range(0, elems, blk.size):
                    n = min(blk.size, elems - off)
                    check(lib.axhip_memcpy_h2d(buf.ptr + off * 4, blk.ctypes.data, n * 4), "h2d")
        else:
            _rand_fill(kb, elems * 2, 2 * r)
            _rand_fill(vb, elems * 2, 2 * r + 1)
        kv.append((kb, vb))
    qh = np.random.default_rng(9).standard_normal((B, Hq, D)).astype(np.float32)
    q = DeviceBuffer.from_numpy(qh if fp32 else qh.astype(np.float16))
    out = DeviceBuffer(B * Hq * D * esz)
    wsb = lib.axhip_gqa_decode_workspace_bytes(B, Hq, Hkv, D, L)
    ws = DeviceBuffer(max(wsb, 256))
    dl = DeviceBuffer.from_numpy(np.asarray(lens, np.int32)) if lens is not None else None
    state = {"i": 0}

    def step():
        kb, vb = kv[state["i"] % n_rot]
        state["i"] += 1
        check(lib.axhip_gqa_decode(q.ptr, kb.ptr, vb.ptr, dl.ptr if dl else None, out.ptr, ws.ptr, wsb,
                                   F32 if fp32 else F16, B, Hq, Hkv, D, L, Hkv * L * D,
                                   D if token_major else L * D, Hkv * D if token_major else D, None), "gqa_decode")

    us = _time(lib, step, steps)
    L_sum = int(np.sum(lens)) if lens is not None else B * L
    nbytes = 2 * Hkv * D * esz * L_sum + 2 * Hq * D * esz * B
    s, c = C.c_int(0), C.c_int(0)
    lib.axhip_gqa_decode_plan(B, Hq, Hkv, L, C.byref(s), C.byref(c))
    gbs = nbytes / us / 1e3
    _emit({"op": tag, "B": B, "L": L, "dtype": "f32" if fp32 else "f16", "token_major": token_major,
           "ragged": lens is not None, "us": round(us, 2), "bytes": nbytes,
           "GBps": round(gbs, 1), "pct_hbm_peak": round(100 * gbs / HBM_PEAK, 1), "splits": s.value,
           "chunk": c.value, "kv_buffers": n_rot})
    return us


def bench_gqa_paged(lib, B, L, steps, lens=None, Hq=16, Hkv=8, D=128, n_rot=None, seed=0):
    """Decode attention over a paged cache (pools [n_pages, Hkv, 128, D] fp16) whose pages were handed out in a
    random order, beside the dense cache of the same size."""
    P = 128
    pages_per_seq = (L + P - 1) // P
    n_pages = B * pages_per_seq
    elems = n_pages * Hkv * P * D
    if n_rot is None:
        n_rot = max(2, min(8, int(2**30 // (elems * 4)) + 1))
    pools = []
    for r in range(n_rot):
        kb, vb = DeviceBuffer(elems * 2), DeviceBuffer(elems * 2)
        _rand_fill(kb, elems * 2, 2 * r)
        _rand_fill(vb, elems * 2, 2 * r + 1)
        pools.append((kb, vb))
    rng = np.random.default_rng(seed)
    table = rng.permutation(n_pages).astype(np.int32).reshape(B, pages_per_seq)
    dt_ = DeviceBuffer.from_numpy(table)
    q = DeviceBuffer.from_numpy(rng.standard_normal((B, Hq, D)).astype(np.float32).astype(np.float16))
    out = DeviceBuffer(B * Hq * D * 2)
    wsb = lib.axhip_gqa_decode_workspace_bytes(B, Hq, Hkv, D, L)
    ws = DeviceBuffer(max(wsb, 256))
    dl = DeviceBuffer.from_numpy(np.asarray(lens, np.int32)) if lens is not None else None
    state = {"i": 0}

    def paged():
        kb, vb = pools[state["i"] % n_rot]
        state["i"] += 1
        check(lib.axhip_gqa_decode_paged(q.ptr, kb.ptr, vb.ptr, dt_.ptr, dl.ptr if dl else None, out.ptr, ws.ptr, wsb, F16,
                                         B, Hq, Hkv, D, L, pages_per_seq, n_pages, None), "gqa_decode_paged")

    def dense():  # the same buffers read as a dense [B, Hkv, pages_per_seq * 128, D] cache
        kb, vb = pools[state["i"] % n_rot]
        state["i"] += 1
        rows = pages_per_seq * P
        check(lib.axhip_gqa_decode(q.ptr, kb.ptr, vb.ptr, dl.ptr if dl else None, out.ptr, ws.ptr, wsb, F16, B, Hq, Hkv, D, L,
                                   Hkv * rows * D, rows * D, D, None), "gqa_decode")

    L_sum = int(np.sum(lens)) if lens is not None else B * L
    nbytes = 2 * Hkv * D * 2 * L_sum + 2 * Hq * D * 2 * B
    for name, fn in (("gqa_dense", dense), ("gqa_paged_random_pages", paged)):
        us = _time(lib, fn, steps)
        _emit({"op": name, "B": B, "L": L, "ragged": lens is not None, "pages": n_pages, "us": round(us, 2), "bytes": nbytes,
               "GBps": round(nbytes / us / 1e3, 1), "pct_hbm_peak": round(100 * nbytes / us / 1e3 / HBM_PEAK, 1),
               "kv_buffers": n_rot})


def bench_gqa_step_form(lib, B, L, steps, Hq=16, Hkv=8, D=128, rows=None, n_rot=4):
    """The attention launch of a decode step (q/k RMSNorm, M-RoPE and the KV append in its prologue)
    beside plain attention over the same L + 1 keys of the same caches."""
    rows = rows or (L + 128) // 128 * 128
    elems = B * Hkv * rows * D
    kv = []
    for r in range(n_rot):
        kb, vb = DeviceBuffer(elems * 2), DeviceBuffer(elems * 2)
        _rand_fill(kb, elems * 2, 2 * r)
        _rand_fill(vb, elems * 2, 2 * r + 1)
        kv.append((kb, vb))
    rng = np.random.default_rng(5)
    width = (Hq + 2 * Hkv) * D
    qkv = DeviceBuffer.from_numpy(rng.standard_normal((B, width)).astype(np.float32))
    qh = DeviceBuffer.from_numpy(rng.standard_normal((B, Hq, D)).astype(np.float16))
    wq = DeviceBuffer.from_numpy(np.ones(D, np.float32))
    wk = DeviceBuffer.from_numpy(np.ones(D, np.float32))
    pos = DeviceBuffer.from_numpy(np.full((3, B), L, np.int64))
    inv = DeviceBuffer.from_numpy((1.0 / (1e6 ** (np.arange(0, D, 2, dtype=np.float32) / D))).astype(np.float32))
    lens = DeviceBuffer.from_numpy(np.full(B, L, np.int32))
    lens1 = DeviceBuffer.from_numpy(np.full(B, L + 1, np.int32))
    out = DeviceBuffer(B * Hq * D * 2)
    wsb = lib.axhip_gqa_decode_workspace_bytes(B, Hq, Hkv, D, rows)
    ws = DeviceBuffer(max(wsb, 256))
    state = {"i": 0}

    def step_form():
        kb, vb = kv[state["i"] % n_rot]
        state["i"] += 1
        check(lib.axhip_gqa_decode_qkv(qkv.ptr, width, qkv.ptr + Hq * D * 4, width, qkv.ptr + (Hq + Hkv) * D * 4, width,
                                       wq.ptr, wk.ptr, F32, 1e-6, pos.ptr, inv.ptr, 20, 20, lens.ptr, kb.ptr, vb.ptr,
                                       out.ptr, ws.ptr, wsb, F16, B, Hq, Hkv, D, rows, rows, None), "gqa_decode_qkv")

    def plain():
        kb, vb = kv[state["i"] % n_rot]
        state["i"] += 1
        check(lib.axhip_gqa_decode(qh.ptr, kb.ptr, vb.ptr, lens1.ptr, out.ptr, ws.ptr, wsb, F16, B, Hq, Hkv, D, rows,
                                   Hkv * rows * D, rows * D, D, None), "gqa_decode")

    nbytes = 2 * Hkv * D * 2 * (L + 1) * B + 2 * Hq * D * 2 * B
    for name, fn in (("gqa_plain", plain), ("gqa_decode_step_form", step_form)):
        us = _time(lib, fn, steps)
        _emit({"op": name, "B": B, "L": L + 1, "cache_rows": rows, "us": round(us, 2), "bytes": nbytes,
               "GBps": round(nbytes / us / 1e3, 1), "pct_hbm_peak": round(100 * nbytes / us / 1e3 / HBM_PEAK, 1)})


def bench_prefill_attn(lib, B, S, steps, Hq=16, Hkv=8, D=128):
    """Causal prefill attention: 4*D flops per visible (query, key) pair and query head."""
    n = B * Hkv * S * D
    q = DeviceBuffer(B * S * Hq * D * 2)
    k, v, out = DeviceBuffer(n * 2), DeviceBuffer(n * 2), DeviceBuffer(B * S * Hq * D * 2)
    for i, buf in enumerate((q, k, v)):
        _rand_fill(buf, buf.nbytes, 100 + i)

    def step():
        check(lib.axhip_prefill_attention(q.ptr, k.ptr, v.ptr, None, out.ptr, F16, B, S, Hq, Hkv, D, S, None), "prefill")

    us = _time(lib, step, steps)
    fl = 4.0 * D * Hq * B * (S * (S + 1) / 2)
    _emit({"op": "prefill_attention", "B": B, "S": S, "Hq": Hq, "Hkv": Hkv, "D": D, "us": round(us, 1),
           "TFLOPs": round(fl / us / 1e6, 1), "pct_mfma_f16_peak": round(100 * fl / us / 1e6 / MFMA_F16_PEAK, 2)})


def bench_sdpa(lib, S, steps, causal, Hq=16, Hkv=8, D=128):
    """The general attention entry on token-major q [S,Hq,D] and k/v [S,Hkv,D]."""
    q, out = DeviceBuffer(S * Hq * D * 2), DeviceBuffer(S * Hq * D * 2)
    k, v = DeviceBuffer(S * Hkv * D * 2), DeviceBuffer(S * Hkv * D * 2)
    for i, buf in enumerate((q, k, v)):
        _rand_fill(buf, buf.nbytes, 200 + i)

    def step():
        check(lib.axhip_sdpa(q.ptr, k.ptr, v.ptr, out.ptr, F16, S, Hq, Hkv, D, S, int(causal), None), "sdpa")

    us = _time(lib, step, steps)
    fl = 4.0 * D * Hq * (S * (S + 1) / 2 if causal else S * S)
    _emit({"op": "sdpa", "S": S, "Hq": Hq, "Hkv": Hkv, "D": D, "causal": bool(causal), "us": round(us, 1),
           "TFLOPs": round(fl / us / 1e6, 1), "pct_mfma_f16_peak": round(100 * fl / us / 1e6 / MFMA_F16_PEAK, 2)})


def bench_copy(lib, mib, steps):
    n = mib * 2**20
    a, b = DeviceBuffer(n), DeviceBuffer(n)
    _rand_fill(a, n, 1)
    us = _time(lib, lambda: check(lib.axhip_memcpy_d2d(b.ptr, a.ptr, n), "copy"), steps)
    gbs = 2 * n / us / 1e3
    _emit({"op": "copy_bytes_kernel", "bytes_read": n, "bytes_written": n, "us": round(us, 2),
           "GBps_read_plus_write": round(gbs, 1), "pct_hbm_peak": round(100 * gbs / HBM_PEAK, 1)})


def bench_rowops(lib, steps=200, row_counts=(32, 4096, 65536)):
    rng = np.random.default_rng(0)

    def h(shape, scale=1.0):
        return DeviceBuffer.from_numpy((scale * rng.standard_normal(shape)).astype(np.float32).astype(np.float16))

    for rows in row_counts:
        x, r, w = h((rows, 2048)), h((rows, 2048)), h((2048,))
        y, o = DeviceBuffer(rows * 4096), DeviceBuffer(rows * 4096)
        us = _time(lib, lambda: check(lib.axhip_add_rms_norm(x.ptr, r.ptr, w.ptr, 1e-6, y.ptr, o.ptr, F16, F16,
                                                              rows, 2048, None), "arn"), steps)
        nb = 4 * rows * 4096 + 4096
        _emit({"op": "add_rms_norm", "rows": rows, "hidden": 2048, "us": round(us, 2), "bytes": nb,
               "GBps": round(nb / us / 1e3, 1), "pct_hbm_peak": round(100 * nb / us / 1e3 / HBM_PEAK, 2)})
        g, u = h((rows, 6144)), h((rows, 6144))
        so = DeviceBuffer(rows * 6144 * 2)
        us = _time(lib, lambda: check(lib.axhip_silu_mul(g.ptr, u.ptr, so.ptr, F16, rows * 6144, None), "silu"), steps)
        nb = 3 * rows * 6144 * 2
        _emit({"op": "silu_mul", "rows": rows, "cols": 6144, "us": round(us, 2), "bytes": nb,
               "GBps": round(nb / us / 1e3, 1), "pct_hbm_peak": round(100 * nb / us / 1e3 / HBM_PEAK, 2)})
        qx, kx = h((rows, 16, 128)), h((rows, 8, 128))
        qo, ko = DeviceBuffer(rows * 16 * 256), DeviceBuffer(rows * 8 * 256)
        pos = DeviceBuffer.from_numpy(rng.integers(0, 8192, rows).astype(np.int64))

        def rope_qk():
            check(lib.axhip_rope_qk(qx.ptr, kx.ptr, pos.ptr, 1e6, qo.ptr, ko.ptr, F16, rows, 16, 8, 128, None), "rope")

        us = _time(lib, rope_qk, steps)
        nb = 2 * rows * 24 * 128 * 2
        _emit({"op": "rope q+k (one launch)", "rows": rows, "us": round(us, 2), "bytes": nb,
               "GBps": round(nb / us / 1e3, 1), "pct_hbm_peak": round(100 * nb / us / 1e3 / HBM_PEAK, 2)})
    B, Hkv, Lmax, D = 32, 8, 8192, 128
    kc, vc = DeviceBuffer(B * Hkv * Lmax * D * 2), DeviceBuffer(B * Hkv * Lmax * D * 2)
    kn, vn = h((B, Hkv, D)), h((B, Hkv, D))
    pos = DeviceBuffer.from_numpy(rng.integers(0, Lmax, B).astype(np.int64))
    us = _time(lib, lambda: check(lib.axhip_kv_append(kn.ptr, vn.ptr, kc.ptr, vc.ptr, pos.ptr, I64, 2, B, Hkv, Lmax,
                                                       D, None), "append"), steps)
    nb = 4 * B * Hkv * D * 2
    _emit({"op": "kv_append", "B": B, "us": round(us, 2), "bytes": nb, "GBps": round(nb / us / 1e3, 2),
           "pct_hbm_peak": round(100 * nb / us / 1e3 / HBM_PEAK, 3)})


def bench_linear(lib, steps=50, shapes=None, Ms=(1, 16, 32, 512), packed=False, rot=0):
    rng = np.random.default_rng(0)
    shapes = shapes or [(2048, 2048), (2048, 12288), (6144, 2048), (2048, 151936)]
    for K, N in shapes:
        w_host = (0.02 * rng.standard_normal((min(N, 4096), K))).astype(np.float32).astype(np.float16)
        if ZERO_DATA:
            w_host[:] = 0
        # several weight copies are rotated when one is smaller than the Infinity Cache
        n_rot = rot or max(1, min(8, int(600e6 // (2 * K * N)) + 1))
        ws_ = []
        for r in range(n_rot):
            wb = DeviceBuffer(N * K * 2)
            off = 0
            while off < N * K * 2:
                n = min(w_host.nbytes, N * K * 2 - off)
                wb.upload(w_host.reshape(-1)[: n // 2], off)
                off += n
            if packed:
                pb = DeviceBuffer(lib.axhip_linear_f16_packed_bytes(N, K))
                check(lib.axhip_linear_f16_pack(wb.ptr, pb.ptr, N, K, 0, None), "pack")
                check(lib.axhip_synchronize(), "sync")
                wb = pb
            ws_.append(wb)
        for M in Ms:
            x_host = rng.standard_normal((M, K)).astype(np.float32).astype(np.float16)
            if ZERO_DATA:
                x_host[:] = 0
            x = DeviceBuffer.from_numpy(x_host)
            out = DeviceBuffer(M * N * 4)
            wsb = lib.axhip_linear_f16_workspace_bytes(M, K, N)
            ws = DeviceBuffer(max(wsb, 256))
            st = {"i": 0}

            def step():
                wb = ws_[st["i"] % n_rot]
                st["i"] += 1
                if packed:
                    check(lib.axhip_linear_f16_packed(x.ptr, F16, wb.ptr, None, out.ptr, F32, M, K, N, 0, None), "linear")
                else:
                    check(lib.axhip_linear_f16(x.ptr, F16, wb.ptr, None, out.ptr, F32, M, K, N, ws.ptr, wsb, None), "linear")

            us = _time(lib, step, steps)
            nb = 2 * K * N + 2 * M * K + 4 * M * N
            fl = 2.0 * M * K * N
            _emit({"op": "linear_f16_packed" if packed else "linear_f16", "M": M, "K": K, "N": N, "us": round(us, 2), "bytes": nb,
                   "GBps": round(nb / us / 1e3, 1), "pct_hbm_peak": round(100 * nb / us / 1e3 / HBM_PEAK, 1),
                   "TFLOPs": round(fl / us / 1e6, 1), "pct_mfma_f16_peak": round(100 * fl / us / 1e6 / MFMA_F16_PEAK, 2),
                   "weight_copies": n_rot})


def bench_layer_tail(lib, steps, layers=28, M=16, H=2048, K1=2048, I=6144, N=4096):
    """The part of a decoder layer behind its attention plus the next q/k/v projection, over `layers` different
    weight sets (nothing comes from the memory-side cache): six launches against the one persistent launch, each
    as a captured graph of all layers replayed back to back; then where the time goes inside one launch in the
    middle of such a chain (axhip_decode_layer_tail_trace)."""
    import time
    from axono_amd import libaxono as L
    from axono_amd.core.hip_graph import HIPGraph
    from axono_amd.core.tensor import Tensor
    from axono_amd.core.types import DataType
    rng = np.random.default_rng(0)

    def dev(a):
        return Tensor.from_numpy_ref(np.ascontiguousarray(a)).to("hip")

    def lin(n, k):
        return (0.02 * rng.standard_normal((n, k), dtype=np.float32)).astype(np.float16)

    base = {"o": lin(H, K1), "gu": lin(2 * I, H), "d": lin(H, I), "q": lin(N, H)}
    W = [{k: L.pack_linear_weight(dev(v), glu=(k == "gu")) for k, v in base.items()} for _ in range(layers)]
    wn = dev(np.ones(H, np.float32))
    attn = dev(rng.standard_normal((M, K1)).astype(np.float16))
    h0 = dev(rng.standard_normal((M, H)).astype(np.float32))
    ws = Tensor(DataType.INT8, [lib.axhip_decode_layer_tail_workspace_bytes(H, I)], "hip")
    L.synchronize()

    def tails():
        h = h0
        for w in W:
            h, _ = L.decode_layer_tail(attn, h, w["o"], wn, w["gu"], w["d"], wn, w["q"], N, 1e-6, ws)

    def singles():
        h = h0
        for w in W:
            o = L.linear_packed(attn, w["o"], H)
            h, xn = L.add_rms_norm(o, h, wn, 1e-6, DataType.FLOAT16)
            act = L.linear_packed(xn, w["gu"], 2 * I, out_dtype=DataType.FLOAT16, glu=True)
            d = L.linear_packed(act, w["d"], H)
            h, xn = L.add_rms_norm(d, h, wn, 1e-6, DataType.FLOAT16)
            L.linear_packed(xn, w["q"], N)

    nbytes = 2 * (H * K1 + 2 * I * H + H * I + N * H)
    for name, fn in (("layer_tail_six_launches", singles), ("layer_tail_one_launch", tails)):
        g = HIPGraph()
        g.capture(fn)
        g.replay()
        L.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            g.launch_async()
        g.sync()
        us = (time.perf_counter() - t0) * 1e6 / (steps * layers)
        g.reset()
        _emit({"op": name, "M": M, "H": H, "I": I, "N_next": N, "us": round(us, 2), "bytes": nbytes,
               "GBps": round(nbytes / us / 1e3, 1), "pct_hbm_peak": round(nbytes / us / 1e3 / 80.0, 1), "weight_sets": layers})
    # the timeline of one launch in the middle of a chain
    stamps = DeviceBuffer(256 * 32 * 8)
    for rep in range(3):
        for i, w in enumerate(W):
            lib.axhip_decode_layer_tail_trace(stamps.ptr if (rep == 2 and i == layers // 2) else None)
            L.decode_layer_tail(attn, h0, w["o"], wn, w["gu"], w["d"], wn, w["q"], N, 1e-6, ws)
    L.synchronize()
    lib.axhip_decode_layer_tail_trace(None)
    t = stamps.download(np.uint64, (256, 2, 16)).astype(np.float64) / 100.0
    t -= t[:, 0, 0].min()
    points = ["start", "phase 1 matrix instructions done", "before barrier 1", "after barrier 1", "phase 2 row sums done",
              "phase 2 matrix instructions done", "before barrier 2", "after barrier 2", "phase 3 matrix instructions done",
              "before barrier 3", "after barrier 3", "phase 4 matrix instructions done", "end"]
    _emit({"op": "layer_tail_timeline", "unit": "us after the first workgroup started; median over the 256 workgroups (max)",
           "wavefront_0": {p: [round(float(np.median(t[:, 0, i])), 2), round(float(t[:, 0, i].max()), 2)] for i, p in enumerate(points)},
           "failed_barrier_waits": L.decode_layer_tail_failed_waits()})


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("what", choices=["gqa", "gqa-sweep", "gqa-shapes", "gqa-single", "gqa-step", "gqa-paged", "copy", "rowops", "linear", "linear-packed", "prefill-attn", "layer-tail"])
    ap.add_argument("--zero-data", action="store_true",
                    help="prefill-attn, linear-packed: all-zero operands (how much of the time is the power the data costs)")
    ap.add_argument("--tile-order", default="", help="linear-packed: 'plain' or 'A:B' rectangles of 256 x 128 GEMM tiles per XCD")
    ap.add_argument("--by-xcd", type=int, default=-1, help="prefill-attn: 1 / 0 force the workgroup order over the XCDs")
    ap.add_argument("--B", type=int, default=32)
    ap.add_argument("--L", type=int, default=8192)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--mib", type=int, default=1024)
    ap.add_argument("--ragged", action="store_true")
    ap.add_argument("--rows", type=int, default=0, help="gqa-step: rows the caches are allocated for (default: L rounded up)")
    ap.add_argument("--splits", type=int, default=0)
    ap.add_argument("--target-wgs", type=int, default=0)
    ap.add_argument("--nt", type=int, default=0, help="linear: 16-row groups of W per wavefront (1, 2, 4)")
    ap.add_argument("--waves", type=int, default=0, help="linear: wavefronts (K slices) per workgroup (4, 8, 16)")
    ap.add_argument("--M", type=int, default=0, help="linear: only this row count")
    ap.add_argument("--gemm-rows", type=int, default=0, help="linear: rows of x per GEMM workgroup (64 or 128)")
    ap.add_argument("--rot", type=int, default=0, help="linear, gqa-step: number of weight / cache copies rotated through (1 = cache-hot)")
    args = ap.parse_args(argv)
    global ZERO_DATA
    ZERO_DATA = bool(args.zero_data)
    lib = _lib.load()
    if _lib.device_count() < 1:
        sys.exit("no HIP device")
    if args.what == "gqa":
        lib.axhip_gqa_decode_tune(args.target_wgs, args.splits)
        lens = None
        if args.ragged:
            lens = np.random.default_rng(0).integers(512, args.L + 1, args.B)
        bench_gqa(lib, args.B, args.L, args.steps, lens)
    elif args.what == "gqa-sweep":
        for B in (1, 8, 32, 64):
            for L in (1024, 8192, 32768):
                bench_gqa(lib, B, L, max(10, min(args.steps, int(2e9 // (B * L * 4096)) + 10)))
        lens = np.random.default_rng(0).integers(512, 32769, 32)
        bench_gqa(lib, 32, 32768, 20, lens, tag="gqa_ragged_512_32768")
    elif args.what == "gqa-shapes":
        # other head shapes: group sizes 1, 4 and 8 (four and more run on the matrix cores), D = 64 and 256
        for Hq, Hkv, D in ((8, 8, 128), (32, 8, 128), (64, 8, 128), (32, 4, 128), (32, 8, 64), (16, 8, 64), (16, 8, 256)):
            for B, L in ((32, 8192), (16, 4160), (4, 8192), (1, 32768)):
                bench_gqa(lib, B, L, min(args.steps, 50), Hq=Hq, Hkv=Hkv, D=D, tag=f"gqa_Hq{Hq}_Hkv{Hkv}_D{D}")
    elif args.what == "gqa-paged":
        for B, L in ((32, 8192), (16, 4160), (8, 8192), (64, 1024), (1, 32768)):
            bench_gqa_paged(lib, B, L, min(args.steps, 100))
        bench_gqa_paged(lib, 32, 32768, 20, np.random.default_rng(0).integers(512, 32769, 32))
    elif args.what == "gqa-step":
        bench_gqa_step_form(lib, args.B if args.B != 32 else 16, args.L if args.L != 8192 else 4160, args.steps,
                            rows=args.rows or None, n_rot=args.rot or 4)
    elif args.what == "gqa-single":
        # the reference's own call: one sequence, q (1,Hq,D), K/V (L,Hkv,D) token-major, fp32 (and the same in fp16)
        for fp32 in (True, False):
            for L in (1024, 2048, 8192, 32768, 131072):
                bench_gqa(lib, 1, L, min(args.steps, 100), fp32=fp32, token_major=True, tag="gqa_single_sequence")
    elif args.what == "prefill-attn":
        lib.axhip_prefill_attention_tune(args.by_xcd)
        for S in (1024, 4096, 16384):
            bench_prefill_attn(lib, max(1, min(args.B, 65536 // S)), S, max(5, min(args.steps, 20)))
        for S in (4096, 16384):
            for causal in (True, False):
                bench_sdpa(lib, S, max(5, min(args.steps, 20)), causal)
    elif args.what == "layer-tail":
        bench_layer_tail(lib, min(args.steps, 20))
    elif args.what == "copy":
        bench_copy(lib, args.mib, args.steps)
    elif args.what == "rowops":
        bench_rowops(lib)
    elif args.what == "linear":
        lib.axhip_linear_f16_tune(0, args.nt, args.waves, args.gemm_rows)
        bench_linear(lib, Ms=(args.M,) if args.M else (1, 16, 32, 512), rot=args.rot)
    elif args.what == "linear-packed":
        order = 0
        if args.tile_order:
            order = 100000 if args.tile_order == "plain" else 100000 + 256 * int(args.tile_order.split(":")[0]) + int(args.tile_order.split(":")[1])
        lib.axhip_linear_f16_tune(order, args.nt, args.waves, args.gemm_rows)
        bench_linear(lib, shapes=[(2048, 2048), (2048, 4096), (2048, 12288), (6144, 2048), (2048, 151936)],
                     Ms=(args.M,) if args.M else (1, 16, 32, 512, 4096), packed=True, rot=args.rot, steps=min(args.steps, 50))


if __name__ == "__main__":
    main()
