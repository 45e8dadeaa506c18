"""Helpers for the GPU parity tests: every call goes through the C ABI of libaxhip.so."""
import contextlib
import ctypes as C

import numpy as np

from axono_amd import _lib
from axono_amd.device import DeviceBuffer, check, synchronize

F16, F32, I32, I64 = 4, 5, 2, 3  # DataType values of the ABI


def dt(arr):
    return {np.dtype(np.float16): F16, np.dtype(np.float32): F32, np.dtype(np.int32): I32,
            np.dtype(np.int64): I64}[np.dtype(arr.dtype)]


def lib():
    return _lib.load()


def dev(arr):
    return DeviceBuffer.from_numpy(np.ascontiguousarray(arr))


def gqa_decode(q, k, v, seq_lens=None, layout="cache", max_len=None):
    """layout 'cache': k/v [B,Hkv,Lmax,D]; 'ref': q (1,Hq,D), k/v (L,Hkv,D) (the reference's call)."""
    l = lib()
    if layout == "cache":
        B, Hq, D = q.shape
        _, Hkv, Lmax, _ = k.shape
        sb, sh, ss = Hkv * Lmax * D, Lmax * D, D
    else:
        B, Hq, D = q.shape
        Lmax, Hkv, _ = k.shape
        sb, sh, ss = 0, D, Hkv * D
    if max_len is None:
        max_len = Lmax
    dq, dk, dv = dev(q), dev(k), dev(v)
    dout = DeviceBuffer(q.nbytes)
    wsb = l.axhip_gqa_decode_workspace_bytes(B, Hq, Hkv, D, max_len)
    ws = DeviceBuffer(max(wsb, 256))
    dl = dev(np.asarray(seq_lens, np.int32)) if seq_lens is not None else None
    check(l.axhip_gqa_decode(dq.ptr, dk.ptr, dv.ptr, dl.ptr if dl else None, dout.ptr, ws.ptr, wsb, dt(q),
                             B, Hq, Hkv, D, max_len, sb, sh, ss, None), "gqa_decode")
    synchronize()
    return dout.download(q.dtype, q.shape)


@contextlib.contextmanager
def gqa_tuned(target_workgroups, force_splits):
    """Forces a split plan of the decode attention for the body; the defaults come back on every exit path."""
    lib().axhip_gqa_decode_tune(target_workgroups, force_splits)
    try:
        yield
    finally:
        lib().axhip_gqa_decode_tune(0, 0)


@contextlib.contextmanager
def linear_tuned(target_waves=0, force_nt=0, force_waves=0, gemm_rows=0):
    lib().axhip_linear_f16_tune(target_waves, force_nt, force_waves, gemm_rows)
    try:
        yield
    finally:
        lib().axhip_linear_f16_tune(0, 0, 0, 0)


def _run(fn_name, *args):
    check(getattr(lib(), fn_name)(*args), fn_name)


def add_rms_norm(x, res, w, eps=1e-6):
    hidden = x.shape[-1]
    rows = x.size // hidden
    dx, dr, dw = dev(x), dev(res), dev(w)
    dy, do = DeviceBuffer(x.nbytes), DeviceBuffer(x.nbytes)
    _run("axhip_add_rms_norm", dx.ptr, dr.ptr, dw.ptr, eps, dy.ptr, do.ptr, dt(x), dt(w), rows, hidden, None)
    synchronize()
    return dy.download(x.dtype, x.shape), do.download(x.dtype, x.shape)


def rms_norm(x, w, eps=1e-5):
    cols = x.shape[-1]
    rows = x.size // cols
    dx = dev(x)
    dw = dev(w) if w is not None else None
    do = DeviceBuffer(x.nbytes)
    _run("axhip_rms_norm", dx.ptr, dw.ptr if dw else None, eps, do.ptr, dt(x), dt(w) if w is not None else F32,
         rows, cols, None)
    synchronize()
    return do.download(x.dtype, x.shape)


def silu_mul(g, u):
    dg, du, do = dev(g), dev(u), DeviceBuffer(g.nbytes)
    _run("axhip_silu_mul", dg.ptr, du.ptr, do.ptr, dt(g), g.size, None)
    synchronize()
    return do.download(g.dtype, g.shape)


def add(a, b):
    da, db, do = dev(a), dev(b), DeviceBuffer(a.nbytes)
    _run("axhip_add", da.ptr, db.ptr, do.ptr, dt(a), a.size, None)
    synchronize()
    return do.download(a.dtype, a.shape)


def cast(x, to):
    dx = dev(x)
    do = DeviceBuffer(x.size * np.dtype(to).itemsize)
    _run("axhip_cast", dx.ptr, dt(x), do.ptr, dt(np.empty(0, to)), x.size, None)
    synchronize()
    return do.download(to, x.shape)


def rope(x, pos, theta):
    rows, heads, dim = x.shape
    dx, dp, do = dev(x), dev(np.asarray(pos, np.int64)), DeviceBuffer(x.nbytes)
    _run("axhip_rope", dx.ptr, dp.ptr, theta, do.ptr, dt(x), rows, heads, dim, None)
    synchronize()
    return do.download(x.dtype, x.shape)


def rope_qk(q, k, pos, theta):
    rows, hq, dim = q.shape
    hk = k.shape[1]
    dq, dk, dp = dev(q), dev(k), dev(np.asarray(pos, np.int64))
    oq, ok = DeviceBuffer(q.nbytes), DeviceBuffer(k.nbytes)
    _run("axhip_rope_qk", dq.ptr, dk.ptr, dp.ptr, theta, oq.ptr, ok.ptr, dt(q), rows, hq, hk, dim, None)
    synchronize()
    return oq.download(q.dtype, q.shape), ok.download(k.dtype, k.shape)


def rope_thd(x, pos3, inv_freq, section):
    rows, heads, dim = x.shape
    dx, dp, df, do = dev(x), dev(np.asarray(pos3, np.int64)), dev(np.asarray(inv_freq, np.float32)), DeviceBuffer(x.nbytes)
    t, h, w = (list(section) + [0, 0, 0])[:3]
    _run("axhip_rope_thd", dx.ptr, dp.ptr, df.ptr, t, h, w, do.ptr, dt(x), rows, heads, dim, None)
    synchronize()
    return do.download(x.dtype, x.shape)


def mrope_cos_sin(pos3, inv_freq, h_sec, w_sec):
    rows, half = pos3.shape[1], inv_freq.shape[0]
    dp, df = dev(np.asarray(pos3, np.int64)), dev(np.asarray(inv_freq, np.float32))
    dc, ds = DeviceBuffer(rows * 2 * half * 4), DeviceBuffer(rows * 2 * half * 4)
    _run("axhip_mrope_cos_sin", dp.ptr, df.ptr, h_sec, w_sec, dc.ptr, ds.ptr, rows, half, None)
    synchronize()
    return dc.download(np.float32, (rows, 2 * half)), ds.download(np.float32, (rows, 2 * half))


def rope_with_cos_sin(x, c, s):
    rows, heads, dim = x.shape
    dx, dc, ds, do = dev(x), dev(np.asarray(c, np.float32)), dev(np.asarray(s, np.float32)), DeviceBuffer(x.nbytes)
    _run("axhip_rope_with_cos_sin", dx.ptr, dc.ptr, ds.ptr, do.ptr, dt(x), rows, heads, dim, None)
    synchronize()
    return do.download(x.dtype, x.shape)


def kv_append(k_new, v_new, k_cache, v_cache, pos):
    B, Hkv, Lmax, D = k_cache.shape
    dkn, dvn, dkc, dvc, dp = dev(k_new), dev(v_new), dev(k_cache), dev(v_cache), dev(pos)
    _run("axhip_kv_append", dkn.ptr, dvn.ptr, dkc.ptr, dvc.ptr, dp.ptr, dt(pos), k_cache.itemsize, B, Hkv, Lmax, D, None)
    synchronize()
    return dkc.download(k_cache.dtype, k_cache.shape), dvc.download(v_cache.dtype, v_cache.shape)


def concat_axis0(a, b):
    da, db = dev(a), dev(b)
    do = DeviceBuffer(a.nbytes + b.nbytes)
    _run("axhip_concat", da.ptr, db.ptr, do.ptr, 1, a.nbytes, b.nbytes, None)
    synchronize()
    return do.download(a.dtype, (a.shape[0] + b.shape[0],) + a.shape[1:])


def linear_f16(x, w, bias=None, out_dtype=np.float32):
    M, K = x.shape
    N = w.shape[0]
    l = lib()
    dx, dw = dev(x), dev(w)
    db = dev(bias) if bias is not None else None
    do = DeviceBuffer(M * N * np.dtype(out_dtype).itemsize)
    wsb = l.axhip_linear_f16_workspace_bytes(M, K, N)
    ws = DeviceBuffer(max(wsb, 256))
    _run("axhip_linear_f16", dx.ptr, dt(x), dw.ptr, db.ptr if db else None, do.ptr, dt(np.empty(0, out_dtype)),
         M, K, N, ws.ptr, wsb, None)
    synchronize()
    return do.download(out_dtype, (M, N))


def linear_f16_packed(x, w, bias=None, out_dtype=np.float32, glu=False):
    M, K = x.shape
    N = w.shape[0]
    l = lib()
    dx, dw = dev(x), dev(w)
    dp = DeviceBuffer(l.axhip_linear_f16_packed_bytes(N, K))
    _run("axhip_linear_f16_pack", dw.ptr, dp.ptr, N, K, int(glu), None)
    db = dev(bias) if bias is not None else None
    n_out = N // 2 if glu else N
    do = DeviceBuffer(M * n_out * np.dtype(out_dtype).itemsize)
    _run("axhip_linear_f16_packed", dx.ptr, dt(x), dp.ptr, db.ptr if db else None, do.ptr,
         dt(np.empty(0, out_dtype)), M, K, N, int(glu), None)
    synchronize()
    return do.download(out_dtype, (M, n_out))


def embedding(ids, table):
    di, dtb = dev(ids), dev(table)
    do = DeviceBuffer(ids.size * table.shape[1] * table.itemsize)
    _run("axhip_embedding", di.ptr, dt(ids), dtb.ptr, do.ptr, dt(table), ids.size, table.shape[0], table.shape[1], None)
    synchronize()
    return do.download(table.dtype, ids.shape + (table.shape[1],))


def argmax(x):
    cols = x.shape[-1]
    rows = x.size // cols
    dx, do = dev(x), DeviceBuffer(rows * 8)
    _run("axhip_argmax", dx.ptr, do.ptr, dt(x), rows, cols, None)
    synchronize()
    return do.download(np.int64, (rows,))


def sdpa(q, k, v, causal):
    Sq, Hq, D = q.shape
    Skv, Hkv, _ = k.shape
    dq, dk, dv, do = dev(q), dev(k), dev(v), DeviceBuffer(q.nbytes)
    _run("axhip_sdpa", dq.ptr, dk.ptr, dv.ptr, do.ptr, dt(q), Sq, Hq, Hkv, D, Skv, int(causal), None)
    synchronize()
    return do.download(q.dtype, q.shape)
