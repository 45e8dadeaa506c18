"""The decode-step operators evaluated in float64 with NumPy: what the mathematics gives for the same
inputs, free of fp32 rounding and of any particular summation order.

TEST INFRASTRUCTURE ONLY.  It is not a restatement of the reference (oracle.port is): it is the
yardstick both the fp32 restatement and the device are measured against where two correct fp32
pipelines legitimately drift apart (a decode step is 28 layers deep and re-rounds to fp16 at every
storage point, so a 1e-7 difference can land on the other side of an fp16 boundary and grow).  The
operator set and argument conventions are those of `oracle.port`, so `OracleDecoder(..., ops=F64Ops())`
runs the same op sequence.  Formulas: softmax(q K^T / sqrt(D)) V with the head -> kv-head map
h // group (tests/core/test_gqa.py:11-25 of the reference); x / sqrt(mean(x^2) + eps) * w
(tests/core/test_fused.py:50-53); g / (1 + exp(-g)) * u (test_fused.py:9-10); interleaved M-RoPE with
rotate-half pairs (examples/vlm/qwen3vl/model.py:37-46, tests/core/test_sequence_ops.py:252-259).
"""
from __future__ import annotations

import numpy as np

F = np.float64


class F64Ops:
    dtype = F

    # ---- attention -------------------------------------------------------------------------------
    def sdpa(self, q, k, v, is_causal=False):
        q, k, v = (np.asarray(a, F) for a in (q, k, v))
        sq, hq, d = q.shape
        skv, hkv, _ = k.shape
        group = hq // hkv
        out = np.empty((sq, hq, d), F)
        for h in range(hq):
            kk, vv = k[:, h // group], v[:, h // group]
            s = (q[:, h] @ kk.T) / np.sqrt(F(d))                      # [sq, skv]
            if is_causal:
                t = np.arange(sq)[:, None]
                s = np.where(np.arange(skv)[None, :] <= t, s, -np.inf)
            s = s - s.max(axis=1, keepdims=True)
            p = np.exp(s)
            out[:, h] = (p / p.sum(axis=1, keepdims=True)) @ vv
        return out

    # ---- norms and gates -------------------------------------------------------------------------
    def rms_norm(self, x, w, eps=1e-5):
        x = np.asarray(x, F)
        y = x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + F(np.float32(eps)))
        return y if w is None else y * np.asarray(w, F)

    def add_rms_norm(self, x, res, w, eps=1e-6):
        y = np.asarray(x, F) + np.asarray(res, F)
        return y, self.rms_norm(y, w, eps)

    def silu_mul(self, gate, up):
        g, u = np.asarray(gate, F), np.asarray(up, F)
        return g / (1.0 + np.exp(-g)) * u

    # ---- rotary ----------------------------------------------------------------------------------
    def rope_thd(self, x, pos, inv_freq, mrope_section):
        x = np.asarray(x, F)
        rows, heads, dim = x.shape
        half = dim // 2
        pos = np.asarray(pos, np.int64)                                # [3, rows]
        _, h_sec, w_sec = (list(mrope_section) + [0, 0, 0])[:3]
        i = np.arange(half)
        src = np.zeros(half, np.int64)                                 # 0: T, 1: H, 2: W
        src[(i % 3 == 1) & (i < 3 * h_sec)] = 1
        src[(i % 3 == 2) & (i < 3 * w_sec)] = 2
        # the angle is the product of an integer position and the given fp32 frequency, exactly
        ang = pos[src, :].T.astype(F) * np.asarray(inv_freq, np.float32).astype(F)[None, :]   # [rows, half]
        c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
        a, b = x[..., :half], x[..., half:]
        return np.concatenate([a * c - b * s, b * c + a * s], axis=-1)

    # ---- linear / index --------------------------------------------------------------------------
    def linear(self, x, w, bias=None):
        out = np.asarray(x, F) @ np.asarray(w, F).T
        return out if bias is None else out + np.asarray(bias, F)

    def embedding(self, ids, table):
        return np.asarray(table, F)[np.asarray(ids, np.int64)]

    def argmax(self, x):
        return np.argmax(np.asarray(x), axis=-1).astype(np.int64)
