"""CPU restatement of the text-tower decode step, built from the oracle's operators in the order
the reference's example model applies them (axono/python/examples/vlm/qwen3vl/model.py:330-373
attention, :384 MLP, :408-436 layer, :483-486 final norm + tied lm_head, :729-761 decode_step).

TEST INFRASTRUCTURE ONLY (parity tests and the benchmark's CPU-baseline leg).

All arithmetic is fp32 with the default operator set (`oracle.port`); `ops=F64Ops()`
(oracle/f64_ops.py) evaluates the same sequence in float64 with the same storage roundings.  Data formats are those of the build under test and are modelled as
roundings of stored values only: Linear weights and the embedding table are fp16; the activation
entering a Linear is rounded to fp16 (the reference's fp16 Linear does that, src/ops/cuda/linear.cu:110);
q after RoPE and the k / v rows written to the cache are fp16 (the cache format).
"""
from __future__ import annotations

import numpy as np

from . import port


def _h(x):
    """Round to fp16 (IEEE RNE, one rounding from the array's own precision) and widen back exactly."""
    return np.asarray(x).astype(np.float16).astype(np.float32)


class OracleDecoder:
    def __init__(self, cfg, weights: dict, batch: int, max_len: int, ops=port):
        self.cfg, self.w, self.B, self.max_len, self.ops = cfg, weights, batch, max_len, ops
        nkv, D = cfg.num_key_value_heads, cfg.head_dim
        self.k = [np.zeros((batch, nkv, max_len, D), np.float16) for _ in range(cfg.num_hidden_layers)]
        self.v = [np.zeros((batch, nkv, max_len, D), np.float16) for _ in range(cfg.num_hidden_layers)]
        self.lens = np.zeros(batch, np.int32)
        self.inv_freq = (1.0 / (cfg.rope_theta ** (np.arange(0, D, 2, dtype=np.float32) / D))).astype(np.float32)
        self._w32 = {}

    def W(self, name):
        """fp16 weight widened to fp32 (cached per name; dropped with drop_cache())."""
        if name not in self._w32:
            self._w32[name] = np.asarray(self.w[name], np.float32)
        return self._w32[name]

    def drop_cache(self):
        self._w32.clear()

    def _linear(self, x, name):
        return self.ops.linear(_h(x), self.W(name))

    def _layer(self, i, h, xn, pos3, rows_b, rows_t):
        """h, xn [R,H] for R token rows; rows_b / rows_t give each row's sequence and cache position."""
        cfg, ops = self.cfg, self.ops
        nq, nkv, D = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
        p = f"layers.{i}."
        R = h.shape[0]
        qkv = self._linear(xn, p + "self_attn.qkv_proj.weight")
        q = qkv[:, : nq * D].reshape(R, nq, D)
        k = qkv[:, nq * D: (nq + nkv) * D].reshape(R, nkv, D)
        v = qkv[:, (nq + nkv) * D:].reshape(R, nkv, D)
        q = ops.rms_norm(q, self.w[p + "self_attn.q_norm.weight"], cfg.rms_norm_eps)
        k = ops.rms_norm(k, self.w[p + "self_attn.k_norm.weight"], cfg.rms_norm_eps)
        q = _h(ops.rope_thd(q, pos3, self.inv_freq, cfg.mrope_section))
        k = ops.rope_thd(k, pos3, self.inv_freq, cfg.mrope_section)
        self.k[i][rows_b, :, rows_t] = k.astype(np.float16)
        self.v[i][rows_b, :, rows_t] = v.astype(np.float16)
        attn = np.empty((R, nq, D), getattr(ops, "dtype", np.float32))
        for b in np.unique(rows_b):
            sel = np.nonzero(rows_b == b)[0]
            for r in sel:  # each row attends over the keys up to and including its own position
                L = int(rows_t[r]) + 1
                kk = np.ascontiguousarray(np.transpose(self.k[i][b, :, :L], (1, 0, 2)), dtype=np.float32)
                vv = np.ascontiguousarray(np.transpose(self.v[i][b, :, :L], (1, 0, 2)), dtype=np.float32)
                attn[r] = ops.sdpa(q[r:r + 1], kk, vv, False)[0]
        attn_out = self._linear(attn.reshape(R, nq * D), p + "self_attn.o_proj.weight")
        h, xn2 = ops.add_rms_norm(attn_out, h, self.w[p + "post_attention_layernorm.weight"], cfg.rms_norm_eps)
        gu = self._linear(xn2, p + "mlp.gate_up_proj.weight")
        I = cfg.intermediate_size
        act = ops.silu_mul(np.ascontiguousarray(gu[:, :I]), np.ascontiguousarray(gu[:, I:]))
        mlp_out = self._linear(act, p + "mlp.down_proj.weight")
        nxt = f"layers.{i + 1}.input_layernorm.weight" if i + 1 < cfg.num_hidden_layers else "norm.weight"
        # h + mlp_out, then the next RMSNorm: the reference does add (model.py:435) then rms_norm (:420 / :485)
        return ops.add_rms_norm(mlp_out, h, self.w[nxt], cfg.rms_norm_eps)

    def decode_layers_teacher_forced(self, h_in, pos3):
        """Layer-wise check of one decode step: layer i is evaluated from the residual stream the
        build under test had at that layer's input (h_in[i], FLOAT32 [B,H]); returns the list of
        residual streams each layer produces (to compare with h_in[i+1]) and the logits computed from
        h_in[-1].  Each layer is then compared on identical inputs, so roundings that fall on
        different sides of an fp16 boundary cannot compound through the depth of the model."""
        cfg, ops = self.cfg, self.ops
        rows_b, rows_t = np.arange(self.B), self.lens.copy()
        outs = []
        for i in range(cfg.num_hidden_layers):
            h = np.asarray(h_in[i], np.float32)
            wname = f"layers.{i}.input_layernorm.weight"
            xn = ops.rms_norm(h, self.w[wname], cfg.rms_norm_eps)
            h_next, _ = self._layer(i, h, xn, np.ascontiguousarray(pos3, dtype=np.int64), rows_b, rows_t)
            outs.append(h_next)
        self.lens += 1
        xn = ops.rms_norm(np.asarray(h_in[-1], np.float32), self.w["norm.weight"], cfg.rms_norm_eps)
        return outs, self._linear(xn, "embed_tokens.weight")

    def forward_rows(self, ids, pos3, rows_b, rows_t):
        cfg, ops = self.cfg, self.ops
        h = ops.embedding(np.asarray(ids, np.int64), self.W("embed_tokens.weight"))
        xn = ops.rms_norm(h, self.w["layers.0.input_layernorm.weight"], cfg.rms_norm_eps)
        for i in range(cfg.num_hidden_layers):
            h, xn = self._layer(i, h, xn, pos3, rows_b, rows_t)
        return xn

    def prefill(self, ids):
        """ids int64 [B,S], text-only positions.  Returns last-position logits [B,V] and next ids."""
        B, S = ids.shape
        last = []
        for b in range(B):
            pos3 = np.broadcast_to(np.arange(S, dtype=np.int64), (3, S))
            xn = self.forward_rows(ids[b], np.ascontiguousarray(pos3), np.full(S, b), np.arange(S))
            last.append(xn[-1])
        self.lens[:] = S
        logits = self._linear(np.stack(last), "embed_tokens.weight")
        return logits, self.ops.argmax(logits)

    def decode_step(self, ids, pos3):
        """ids int64 [B], pos3 int64 [3,B].  Appends at lens[b], attends over lens[b]+1 keys, advances."""
        B = self.B
        xn = self.forward_rows(ids, np.ascontiguousarray(pos3, dtype=np.int64), np.arange(B), self.lens.copy())
        self.lens += 1
        logits = self._linear(xn, "embed_tokens.weight")
        return logits, self.ops.argmax(logits)
