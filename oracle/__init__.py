"""NumPy-facing loader for the CPU oracle.

TEST INFRASTRUCTURE ONLY.  `oracle.port` wraps `liboracle.so` (the C restatement in
`axono_cpu_oracle.c`), `oracle.ref` wraps `_ref/libaxono_ref.so` (the reference's own CPU
operators compiled from its sources by `oracle/Makefile`) when that file exists.  Only the test
suite, the smoke check and the benchmark's CPU-baseline leg may import this package; the shipped
package `axono_amd` never does.

All arithmetic is fp32, as in the reference.  fp16 inputs are widened exactly with NumPy before
they come here (the reference's CPU `Half2Float` halves every subnormal, include/axono/core/half.h:61-69,
so it is not used for widening).
"""

from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
PORT_LIB = os.path.join(_HERE, "liboracle.so")
REF_LIB = os.path.join(_HERE, "_ref", "libaxono_ref.so")


def build(ref: bool = True) -> None:
    """Compile the restatement and, when the reference sources are present, the reference."""
    subprocess.run(["make", "-C", _HERE, "oracle"], check=True, capture_output=True)
    if ref:
        subprocess.run(["make", "-C", _HERE, "ref"], check=True, capture_output=True)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i64(a):
    return np.ascontiguousarray(a, dtype=np.int64)


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


class _Ops:
    """Same operator set over either library; `prefix` is `axo_` or `axref_`."""

    def __init__(self, path: str, prefix: str):
        self.path = path
        self.prefix = prefix
        self.lib = C.CDLL(path)

    def _fn(self, name):
        f = getattr(self.lib, self.prefix + name)
        f.restype = C.c_int
        return f

    @staticmethod
    def _check(st, what):
        if st != 0:
            raise RuntimeError(f"oracle {what} failed with status {st}")

    # -- attention -------------------------------------------------------------------------
    def sdpa(self, q, k, v, is_causal=False):
        """q (sq,hq,d), k/v (skv,hkv,d) -> (sq,hq,d).  sequence.cpp:236-301."""
        q, k, v = _f32(q), _f32(k), _f32(v)
        sq, hq, d = q.shape
        skv, hkv, _ = k.shape
        out = np.empty((sq, hq, d), np.float32)
        st = self._fn("sdpa")(_p(q), _p(k), _p(v), _p(out), C.c_int64(sq), C.c_int64(hq),
                              C.c_int64(hkv), C.c_int64(d), C.c_int64(skv), C.c_int(bool(is_causal)))
        self._check(st, "sdpa")
        return out

    def gqa_decode(self, q, k, v):
        """Reference-shaped decode: q (1,hq,d), k/v (L,hkv,d).  Equals sdpa(is_causal=False)
        (axono/python/axono/gqa.py:31)."""
        return self.sdpa(q, k, v, False)

    def gqa_decode_cache(self, q, k_cache, v_cache, seq_lens=None):
        """q (B,hq,d), caches (B,hkv,Lmax,d), seq_lens (B,) -> (B,hq,d): the reference op per
        sequence on that sequence's first seq_lens[b] cache rows."""
        q = _f32(q)
        B, hq, d = q.shape
        _, hkv, lmax, _ = k_cache.shape
        out = np.zeros((B, hq, d), np.float32)
        for b in range(B):
            L = int(lmax if seq_lens is None else seq_lens[b])
            if L <= 0:
                continue
            kb = np.ascontiguousarray(np.transpose(k_cache[b, :, :L, :], (1, 0, 2)), dtype=np.float32)
            vb = np.ascontiguousarray(np.transpose(v_cache[b, :, :L, :], (1, 0, 2)), dtype=np.float32)
            out[b] = self.sdpa(q[b:b + 1], kb, vb, False)[0]
        return out

    # -- fused / norm ----------------------------------------------------------------------
    def silu_mul(self, gate, up):
        gate, up = _f32(gate), _f32(up)
        y = np.empty_like(gate)
        self._check(self._fn("silu_mul")(_p(gate), _p(up), _p(y), C.c_int64(gate.size)), "silu_mul")
        return y

    def add_rms_norm(self, x, res, w, eps=1e-6):
        x, res, w = _f32(x), _f32(res), _f32(w)
        hidden = x.shape[-1]
        rows = x.size // hidden
        y, out = np.empty_like(x), np.empty_like(x)
        st = self._fn("add_rms_norm")(_p(x), _p(res), _p(w), C.c_float(eps), _p(y), _p(out),
                                      C.c_int64(rows), C.c_int64(hidden))
        self._check(st, "add_rms_norm")
        return y, out

    def rms_norm(self, x, w, eps=1e-5):
        x = _f32(x)
        cols = x.shape[-1]
        rows = x.size // cols
        out = np.empty_like(x)
        wk = _f32(w) if w is not None else None
        st = self._fn("rms_norm")(_p(x), _p(wk) if wk is not None else None, C.c_float(eps), _p(out),
                                  C.c_int64(rows), C.c_int64(cols))
        self._check(st, "rms_norm")
        return out

    # -- rotary ----------------------------------------------------------------------------
    def rope(self, x, pos, theta=10000.0):
        x, pos = _f32(x), _i64(pos)
        rows, heads, dim = x.shape
        out = np.empty_like(x)
        st = self._fn("rope")(_p(x), _p(pos), C.c_float(theta), _p(out), C.c_int64(rows),
                              C.c_int64(heads), C.c_int64(dim))
        self._check(st, "rope")
        return out

    def rope_with_cos_sin(self, x, cos, sin):
        x, cos, sin = _f32(x), _f32(cos), _f32(sin)
        rows, heads, dim = x.shape
        out = np.empty_like(x)
        st = self._fn("rope_with_cos_sin")(_p(x), _p(cos), _p(sin), _p(out), C.c_int64(rows),
                                           C.c_int64(heads), C.c_int64(dim))
        self._check(st, "rope_with_cos_sin")
        return out

    def mrope_cos_sin(self, pos, inv_freq, h_sec, w_sec):
        pos, inv_freq = _i64(pos), _f32(inv_freq)
        rows, half = pos.shape[1], inv_freq.shape[0]
        cs = np.empty((rows, 2 * half), np.float32)
        sn = np.empty((rows, 2 * half), np.float32)
        st = self._fn("mrope_cos_sin")(_p(pos), _p(inv_freq), C.c_int(h_sec), C.c_int(w_sec), _p(cs),
                                       _p(sn), C.c_int64(rows), C.c_int64(half))
        self._check(st, "mrope_cos_sin")
        return cs, sn

    def rope_thd(self, x, pos, inv_freq, mrope_section):
        x, pos, inv_freq = _f32(x), _i64(pos), _f32(inv_freq)
        rows, heads, dim = x.shape
        t, h, w = (list(mrope_section) + [0, 0, 0])[:3]
        out = np.empty_like(x)
        st = self._fn("rope_thd")(_p(x), _p(pos), _p(inv_freq), C.c_int(t), C.c_int(h), C.c_int(w),
                                  _p(out), C.c_int64(rows), C.c_int64(heads), C.c_int64(dim))
        self._check(st, "rope_thd")
        return out

    # -- linear ----------------------------------------------------------------------------
    def linear(self, x, w, bias=None):
        x, w = _f32(x), _f32(w)
        k = x.shape[-1]
        rows = x.size // k
        out_f = w.shape[0]
        b = _f32(bias) if bias is not None else None
        out = np.empty(x.shape[:-1] + (out_f,), np.float32)
        st = self._fn("linear")(_p(x), _p(w), _p(b) if b is not None else None, _p(out),
                                C.c_int64(rows), C.c_int64(k), C.c_int64(out_f))
        self._check(st, "linear")
        return out

    # -- index / byte ops ------------------------------------------------------------------
    def argmax(self, x):
        x = _f32(x)
        cols = x.shape[-1]
        rows = x.size // cols
        out = np.empty((rows,), np.int64)
        self._check(self._fn("argmax")(_p(x), _p(out), C.c_int64(rows), C.c_int64(cols)), "argmax")
        return out

    def embedding(self, ids, table):
        ids, table = _i64(ids), _f32(table)
        out = np.empty(ids.shape + (table.shape[1],), np.float32)
        if self.prefix == "axref_":
            st = self._fn("embedding")(_p(ids), _p(table), _p(out), C.c_int64(ids.size),
                                       C.c_int64(table.shape[0]), C.c_int64(table.shape[1]))
        else:
            st = self._fn("embedding")(_p(ids), _p(table), _p(out), C.c_int64(ids.size),
                                       C.c_int64(table.shape[1]))
        self._check(st, "embedding")
        return out

    def concat_axis0(self, a, b):
        """Byte-level concat along axis 0 (the reference's KV append, nn/kv_cache.py:96-102)."""
        a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
        assert a.dtype == b.dtype and a.shape[1:] == b.shape[1:]
        out = np.empty((a.shape[0] + b.shape[0],) + a.shape[1:], a.dtype)
        row_bytes = int(np.prod(a.shape[1:], dtype=np.int64)) * a.itemsize
        if self.prefix == "axref_":
            st = self._fn("concat_axis0")(_p(a), _p(b), _p(out), C.c_int64(a.shape[0]),
                                          C.c_int64(b.shape[0]), C.c_int64(row_bytes))
        else:
            st = self._fn("concat")(_p(a), _p(b), _p(out), C.c_int64(1),
                                    C.c_int64(a.shape[0] * row_bytes), C.c_int64(b.shape[0] * row_bytes))
        self._check(st, "concat")
        return out


class _Port(_Ops):
    """Extras only the restatement has (they have no single reference function)."""

    def num_threads(self):
        self.lib.axo_num_threads.restype = C.c_int
        return int(self.lib.axo_num_threads())

    def rope_inv_freq(self, theta, dim):
        out = np.empty((dim // 2,), np.float32)
        self.lib.axo_rope_inv_freq.restype = None
        self.lib.axo_rope_inv_freq(C.c_float(theta), C.c_int64(dim), _p(out))
        return out

    def gqa_decode_cache_native(self, q, k_cache, v_cache, seq_lens=None):
        """Same result as gqa_decode_cache, without the per-sequence transposes (used where the
        cache is large: the CPU-baseline timing)."""
        q, k_cache, v_cache = _f32(q), _f32(k_cache), _f32(v_cache)
        B, hq, d = q.shape
        _, hkv, lmax, _ = k_cache.shape
        sl = None if seq_lens is None else np.ascontiguousarray(seq_lens, dtype=np.int32)
        out = np.empty((B, hq, d), np.float32)
        st = self._fn("gqa_decode_cache")(_p(q), _p(k_cache), _p(v_cache),
                                          _p(sl) if sl is not None else None, _p(out), C.c_int64(B),
                                          C.c_int64(hq), C.c_int64(hkv), C.c_int64(d), C.c_int64(lmax))
        self._check(st, "gqa_decode_cache")
        return out

    def kv_append(self, k_new, v_new, k_cache, v_cache, pos):
        """In place: cache[b,h,pos[b],:] = new[b,h,:] for both caches (any dtype; byte copy)."""
        B, hkv, lmax, d = k_cache.shape
        assert k_cache.flags.c_contiguous and v_cache.flags.c_contiguous
        k_new, v_new = np.ascontiguousarray(k_new), np.ascontiguousarray(v_new)
        pos = _i64(pos)
        st = self._fn("kv_append")(_p(k_new), _p(v_new), _p(k_cache), _p(v_cache), _p(pos),
                                   C.c_int64(B), C.c_int64(hkv), C.c_int64(lmax),
                                   C.c_int64(d * k_cache.itemsize))
        self._check(st, "kv_append")

    def add(self, a, b):
        a, b = _f32(a), _f32(b)
        out = np.empty_like(a)
        self._check(self._fn("add")(_p(a), _p(b), _p(out), C.c_int64(a.size)), "add")
        return out


def _load_port():
    if not os.path.exists(PORT_LIB):
        build(ref=False)
    return _Port(PORT_LIB, "axo_")


port = _load_port()
ref = _Ops(REF_LIB, "axref_") if os.path.exists(REF_LIB) else None


def ref_float2half(x):
    """The reference's CPU Float2Half bit patterns (half.h:14-52); needs oracle/_ref."""
    x = _f32(x)
    out = np.empty(x.shape, np.uint16)
    ref.lib.axref_float2half(_p(x), _p(out), C.c_int64(x.size))
    return out


def ref_half2float(bits):
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    out = np.empty(bits.shape, np.float32)
    ref.lib.axref_half2float(_p(bits), _p(out), C.c_int64(bits.size))
    return out
