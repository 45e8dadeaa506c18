"""Text tower of a Qwen3-VL-shaped decoder on the hip device: batched prefill into a static KV cache
and a decode step that is captured once into a hipGraph and replayed.

Follows the op sequence of the reference's example model
(axono/python/examples/vlm/qwen3vl/model.py:308-501 for the layers, :729-761 for decode_step):
input RMSNorm -> q/k/v projections -> per-head q/k RMSNorm (over head_dim) -> M-RoPE -> KV append ->
grouped-query attention -> o_proj -> fused add + RMSNorm -> gate/up projections -> SiLU-mul ->
down_proj -> residual add; final RMSNorm and the tied lm_head; greedy argmax.

What differs from the reference, by design of the captured step: the cache is pre-allocated
[B, n_kv, max_len, d_head] per layer with lengths on the device; q/k/v and gate/up are fused
projections (their weights are the row-wise concatenation of the separate matrices); the residual
add at the end of a layer is folded into the next layer's fused add + RMSNorm; next-token argmax,
the embedding lookup of that token and the position increment all run on the device, so a step has
no host <-> device traffic.  Linear weights and the embedding table are FLOAT16; the residual
stream and every Linear output are FLOAT32, as in the reference's fp16-Linear mode; a tensor that
only feeds a Linear (norm outputs, the SiLU-mul result) is stored as FLOAT16 by its producer, which
is the rounding the fp16 Linear applies to its input anyway.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field

import numpy as np

from .. import _lib
from .. import libaxono as L
from .. import nn
from ..core.hip_graph import HIPGraph
from ..core.tensor import Tensor
from ..core.types import DataType
from ..device import check, current_stream


@dataclass
class TextConfig:
    """Qwen3-VL-2B text tower by default."""
    num_hidden_layers: int = 28
    hidden_size: int = 2048
    num_attention_heads: int = 16
    num_key_value_heads: int = 8
    head_dim: int = 128
    intermediate_size: int = 6144
    vocab_size: int = 151936
    rms_norm_eps: float = 1e-6
    rope_theta: float = 1e6
    mrope_section: list = field(default_factory=lambda: [24, 20, 20])


def inv_freq_table(theta: float, d_head: int) -> np.ndarray:
    """1 / theta^(2i/d) in fp32, as the reference builds it (model.py:474-481)."""
    return (1.0 / (theta ** (np.arange(0, d_head, 2, dtype=np.float32) / d_head))).astype(np.float32)


def random_weights(cfg: TextConfig, seed: int = 0) -> dict:
    """Random-init weights of the architecture: Linear / embedding ~ N(0, 0.02) rounded to fp16, norm
    weights 1.  Names follow the reference's module tree; q/k/v and gate/up are stored fused."""
    rng = np.random.default_rng(seed)
    H, D = cfg.hidden_size, cfg.head_dim
    nq, nkv, I = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.intermediate_size

    def lin(n, k):
        return (0.02 * rng.standard_normal((n, k), dtype=np.float32)).astype(np.float16)

    w = {"embed_tokens.weight": lin(cfg.vocab_size, H), "norm.weight": np.ones(H, np.float32)}
    for i in range(cfg.num_hidden_layers):
        p = f"layers.{i}."
        w[p + "self_attn.qkv_proj.weight"] = lin((nq + 2 * nkv) * D, H)
        w[p + "self_attn.o_proj.weight"] = lin(H, nq * D)
        w[p + "self_attn.q_norm.weight"] = np.ones(D, np.float32)
        w[p + "self_attn.k_norm.weight"] = np.ones(D, np.float32)
        w[p + "mlp.gate_up_proj.weight"] = lin(2 * I, H)
        w[p + "mlp.down_proj.weight"] = lin(H, I)
        w[p + "input_layernorm.weight"] = np.ones(H, np.float32)
        w[p + "post_attention_layernorm.weight"] = np.ones(H, np.float32)
    return w


# ---- AXM1 weight files --------------------------------------------------------------------------
# The reference stores the text tower under "model.language_model." with separate q/k/v and gate/up
# projections (examples/vlm/qwen3vl/model.py:323-326,379-381,595-621); this model keeps them fused.
AXM_TEXT_PREFIX = "model.language_model."


def weights_to_axm(weights: dict, cfg: TextConfig, path: str, prefix: str = AXM_TEXT_PREFIX) -> None:
    """Writes `weights` (this module's fused naming) as an .axm file in the reference's naming."""
    from ..format import save_axm

    D, nq, nkv, I = cfg.head_dim, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.intermediate_size
    out = {}
    for name, arr in weights.items():
        if name.endswith("self_attn.qkv_proj.weight"):
            base = name[: -len("qkv_proj.weight")]
            out[prefix + base + "q_proj.weight"] = arr[: nq * D]
            out[prefix + base + "k_proj.weight"] = arr[nq * D: (nq + nkv) * D]
            out[prefix + base + "v_proj.weight"] = arr[(nq + nkv) * D:]
        elif name.endswith("mlp.gate_up_proj.weight"):
            base = name[: -len("gate_up_proj.weight")]
            out[prefix + base + "gate_proj.weight"] = arr[:I]
            out[prefix + base + "up_proj.weight"] = arr[I:]
        else:
            out[prefix + name] = arr
    save_axm(out, path, meta={"text_config": dict(cfg.__dict__)})


def weights_from_axm(path: str, cfg: TextConfig, prefix: str = AXM_TEXT_PREFIX) -> dict:
    """Reads the text tower of an .axm file into this module's naming and storage formats: Linear and
    embedding weights fp16 (what `cast_linear_fp16` makes of them, nn/module.py:158-184), norm weights
    fp32, q/k/v and gate/up concatenated along the output axis.  Tensors outside `prefix` are
    ignored (the vision tower); a missing tensor raises KeyError."""
    from ..format import AxmReader

    r = AxmReader(path)
    have = {n[len(prefix):]: n for n in r.names() if n.startswith(prefix)}

    def get(name, dtype):
        return np.asarray(r.get(have[name])).astype(dtype, copy=False)

    def fused(base, parts, whole):
        if base + whole in have:
            return get(base + whole, np.float16)
        return np.concatenate([get(base + p, np.float16) for p in parts], axis=0)

    w = {"embed_tokens.weight": get("embed_tokens.weight", np.float16), "norm.weight": get("norm.weight", np.float32)}
    for i in range(cfg.num_hidden_layers):
        p = f"layers.{i}."
        w[p + "self_attn.qkv_proj.weight"] = fused(p + "self_attn.", ["q_proj.weight", "k_proj.weight", "v_proj.weight"],
                                                   "qkv_proj.weight")
        w[p + "mlp.gate_up_proj.weight"] = fused(p + "mlp.", ["gate_proj.weight", "up_proj.weight"], "gate_up_proj.weight")
        for n in ("self_attn.o_proj.weight", "mlp.down_proj.weight"):
            w[p + n] = get(p + n, np.float16)
        for n in ("self_attn.q_norm.weight", "self_attn.k_norm.weight", "input_layernorm.weight",
                  "post_attention_layernorm.weight"):
            w[p + n] = get(p + n, np.float32)
    return w


def _dev(arr, device):
    return Tensor.from_numpy_ref(np.ascontiguousarray(arr)).to(device)


class Qwen3VLTextDecoder(nn.Module):
    """paged=True keeps the KV cache in pages of 128 keys (nn.PagedKVCache, `n_pages` per layer pool; default:
    enough for every sequence to reach max_len) instead of one [B, n_kv, max_len, d_head] block per layer; the
    prefill of a sequence then runs over one dense scratch block and is copied into the sequence's pages."""

    def __init__(self, cfg: TextConfig, weights: dict, batch: int, max_len: int, device: str = "hip", paged: bool = False,
                 n_pages: int | None = None, fused_tail: bool | None = None, plan_reuse: bool = True,
                 fused_last: bool = True):
        super().__init__()
        self._cfg = cfg
        self._device = device
        self._batch = batch
        self._lib = _lib.load()
        for name, arr in weights.items():
            self._parameters[name] = _dev(arr, device)
        # decode-sized Linear calls read packed copies of the weights (made once, here)
        # (gate+up weights are packed as alternating gate / up tiles: the kernel's epilogue applies SiLU-mul)
        self._packed = {name: L.pack_linear_weight(t, glu=name.endswith("gate_up_proj.weight"))
                        for name, t in self._parameters.items()
                        if name.endswith("_proj.weight") or name == "embed_tokens.weight"}
        self._inv_freq = _dev(inv_freq_table(cfg.rope_theta, cfg.head_dim), device)
        self._paged = bool(paged)
        if self._paged:
            per_seq = (max_len + nn.PagedKVCache.PAGE - 1) // nn.PagedKVCache.PAGE
            self._cache = nn.PagedKVCache(cfg.num_hidden_layers, batch, cfg.num_key_value_heads, cfg.head_dim,
                                          n_pages if n_pages is not None else batch * per_seq, max_len,
                                          DataType.FLOAT16, device)
            # prefill works on one sequence and one layer at a time over this dense block
            shape = [1, cfg.num_key_value_heads, per_seq * nn.PagedKVCache.PAGE, cfg.head_dim]
            self._scratch_kv = (Tensor(DataType.FLOAT16, shape, device), Tensor(DataType.FLOAT16, shape, device))
        else:
            self._cache = nn.StaticKVCache(cfg.num_hidden_layers, batch, cfg.num_key_value_heads, max_len, cfg.head_dim,
                                           DataType.FLOAT16, device)
        # static state of the captured step
        self._ids = Tensor(DataType.INT64, [batch], device)
        self._pos = Tensor(DataType.INT64, [3, batch], device)
        wsb = self._lib.axhip_gqa_decode_workspace_bytes(batch, cfg.num_attention_heads, cfg.num_key_value_heads,
                                                         cfg.head_dim, max_len)
        self._attn_ws = Tensor(DataType.INT8, [max(wsb, 256)], device)
        self._graph = None
        self._graph_out = None
        # decode step: everything of a layer behind its attention + the next layer's q/k/v projection as one
        # persistent launch, where the library is built for the widths (None: wherever it is)
        n_qkv = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * cfg.head_dim
        can = L.decode_layer_tail_supported(batch, cfg.hidden_size, cfg.num_attention_heads * cfg.head_dim,
                                            cfg.intermediate_size, n_qkv)
        if fused_tail and not can:
            raise ValueError("decode_layer_tail is not built for these widths")
        self._fused_tail = can if fused_tail is None else bool(fused_tail)
        # the attention launches of a step deal the same lengths: layer 0 deals, the others take its table
        self._plan_reuse = bool(plan_reuse)
        # the last layer through the same launch, closed by the final norm (False: as single operators)
        self._fused_last = bool(fused_last)
        if self._fused_tail:
            nbytes = self._lib.axhip_decode_layer_tail_workspace_bytes(cfg.hidden_size, cfg.intermediate_size)
            self._tail_ws = Tensor(DataType.INT8, [nbytes], device)

    # ---- pieces ----------------------------------------------------------------------------
    def _w(self, name):
        return self._parameters[name]

    @property
    def cache(self):
        return self._cache

    def _attention_step(self, qkv, p, i, pos, max_len):
        """q/k RMSNorm + M-RoPE + KV append + attention over seq_lens + 1 keys: one launch (+ the merge)."""
        cfg, cache = self._cfg, self._cache
        args = (qkv, self._w(p + "self_attn.q_norm.weight"), self._w(p + "self_attn.k_norm.weight"), cfg.rms_norm_eps, pos,
                self._inv_freq, cfg.mrope_section, cache.seq_lens, *cache.get(i))
        L.set_plan_reuse((1 if i == 0 else 2) if self._plan_reuse else 0)
        try:
            if self._paged:
                return L.gqa_decode_attention_qkv_paged(*args, cache.page_table, cfg.num_attention_heads, max_len,
                                                        workspace=self._attn_ws)
            return L.gqa_decode_attention_qkv(*args, cfg.num_attention_heads, max_len, workspace=self._attn_ws)
        finally:
            L.set_plan_reuse(0)

    def _linear(self, x, name):
        """x @ W^T over the packed copy of the weight (skinny kernels in decode, MFMA GEMM in prefill)."""
        return L.linear_packed(x, self._packed[name], self._w(name).shape[0])

    def _mlp(self, xn, p):
        name = p + "mlp.gate_up_proj.weight"
        # the gate+up Linear applies SiLU-mul in its epilogue and stores fp16
        act = L.linear_packed(xn, self._packed[name], self._w(name).shape[0], out_dtype=DataType.FLOAT16, glu=True)
        return self._linear(act, p + "mlp.down_proj.weight")

    def forward(self, ids: Tensor, pos: Tensor):
        """One decode step as a Module call, for `axono.compile(model)`: (logits, next ids).  Like
        decode_forward it leaves the lengths alone, so running it again for the same step (the warm-up
        and capture runs of compile) writes the same cache rows; the caller advances the cache
        (`model.cache.advance()`) and the positions after each step, as the reference's loop does
        (examples/vlm/qwen3vl/model.py:827-861)."""
        return self.decode_forward(ids, pos)

    def decode_forward(self, ids: Tensor, pos: Tensor, attn_max_len: int | None = None, trace: list | None = None):
        """One token per sequence.  ids INT64 [B]; pos INT64 [3,B]; appends to the cache at
        cache.seq_lens and attends over seq_lens + 1 keys.  Returns (logits FLOAT32 [B,V], next ids
        INT64 [B]).  Does not advance the lengths.  `trace`, if given, receives the residual stream
        entering every layer and the one leaving the last (FLOAT32 [B,H] tensors), for layer-wise
        comparison with a reference evaluation."""
        cfg = self._cfg
        B = self._batch
        cache = self._cache
        max_len = attn_max_len or cache.max_len
        # embedding row widened to the fp32 residual stream + the first RMSNorm: one launch
        h, xn = L.embedding_rms_norm(ids, self._w("embed_tokens.weight"), self._w("layers.0.input_layernorm.weight"),
                                     cfg.rms_norm_eps)  # [B,H] each
        nl = cfg.num_hidden_layers
        nqd = cfg.num_attention_heads * cfg.head_dim
        n_qkv = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * cfg.head_dim
        qkv = None
        for i in range(nl):
            p = f"layers.{i}."
            if trace is not None:
                trace.append(h)
            if qkv is None:
                qkv = self._linear(xn, p + "self_attn.qkv_proj.weight")
            attn = self._attention_step(qkv, p, i, pos, max_len)
            qkv = None
            if self._fused_tail and i + 1 < nl:
                # o_proj + residual, norm, gate/up + SiLU-mul, down + residual, the next layer's norm and q/k/v
                # projection: one launch
                n = f"layers.{i + 1}."
                h, qkv = L.decode_layer_tail(attn.reshape([B, nqd]), h, self._packed[p + "self_attn.o_proj.weight"],
                                             self._w(p + "post_attention_layernorm.weight"),
                                             self._packed[p + "mlp.gate_up_proj.weight"],
                                             self._packed[p + "mlp.down_proj.weight"],
                                             self._w(n + "input_layernorm.weight"),
                                             self._packed[n + "self_attn.qkv_proj.weight"], n_qkv, cfg.rms_norm_eps,
                                             self._tail_ws)
                continue
            if self._fused_tail and self._fused_last:
                # the last layer: the same launch, closed by the final norm (the rows the lm_head reads)
                h, xn = L.decode_layer_tail_last(attn.reshape([B, nqd]), h, self._packed[p + "self_attn.o_proj.weight"],
                                                 self._w(p + "post_attention_layernorm.weight"),
                                                 self._packed[p + "mlp.gate_up_proj.weight"],
                                                 self._packed[p + "mlp.down_proj.weight"], self._w("norm.weight"),
                                                 cfg.rms_norm_eps, self._tail_ws)
                continue
            attn_out = self._linear(attn.reshape([B, nqd]), p + "self_attn.o_proj.weight")
            h, xn2 = L.add_rms_norm(attn_out, h, self._w(p + "post_attention_layernorm.weight"), cfg.rms_norm_eps,
                                    DataType.FLOAT16)
            mlp_out = self._mlp(xn2, p)
            nxt = f"layers.{i + 1}.input_layernorm.weight" if i + 1 < nl else "norm.weight"
            # h = h + mlp_out folded into the following RMSNorm (next layer's input norm / final norm)
            h, xn = L.add_rms_norm(mlp_out, h, self._w(nxt), cfg.rms_norm_eps, DataType.FLOAT16)
        if trace is not None:
            trace.append(h)
        logits = self._linear(xn, "embed_tokens.weight")  # tied lm_head
        return logits, L.argmax(logits)

    # ---- prefill -----------------------------------------------------------------------------
    def prefill(self, ids: np.ndarray, positions: np.ndarray | None = None):
        """ids int64 [B, S] (host).  Fills the cache for every sequence (all S tokens of up to 65 536 / S
        sequences per pass) and returns (last-position logits FLOAT32 [B,V] as a Tensor, next ids [B]).
        Text-only positions by default: T = H = W = token index."""
        cfg = self._cfg
        B, S = ids.shape
        assert B == self._batch and S <= self._cache.max_len
        lib, dev = self._lib, self._device
        H, D, nq, nkv = cfg.hidden_size, cfg.head_dim, cfg.num_attention_heads, cfg.num_key_value_heads
        width = (nq + 2 * nkv) * D
        lmax = self._cache.max_len
        if positions is None:
            positions = np.broadcast_to(np.arange(S, dtype=np.int64), (3, S))
        pos_t = _dev(np.ascontiguousarray(positions, dtype=np.int64), dev)
        vis = _dev(np.arange(1, S + 1, dtype=np.int32), dev)  # causal: row t sees t+1 keys
        wsb = lib.axhip_gqa_decode_workspace_bytes(S, nq, nkv, D, S)
        ws = Tensor(DataType.INT8, [max(wsb, 256)], dev, _zero=False)
        last_h = Tensor(DataType.FLOAT16, [B, H], dev)  # normalised hidden state of each sequence's last token
        esz = 2
        if self._paged:
            self._cache.reserve(S)
            lmax = self._scratch_kv[0].shape[2]
            s_lens = _dev(np.full(B, S, np.int32), dev)
        # several sequences per pass (their tokens are the rows of every GEMM and one attention launch covers
        # them all): up to 65 536 tokens at a time; the paged cache fills one sequence's dense scratch block at a time
        per_pass = 1 if self._paged else max(1, min(B, 65536 // max(S, 1)))
        for b in range(0, B, per_pass):
            nb = min(per_pass, B - b)
            pos_c = pos_t if nb == 1 else _dev(np.ascontiguousarray(np.tile(positions, (1, nb)), dtype=np.int64), dev)
            h = L.embedding(_dev(ids[b:b + nb].astype(np.int64).reshape(-1), dev),
                            self._w("embed_tokens.weight")).cast_to(DataType.FLOAT32)
            xn = L.rms_norm(h, self._w("layers.0.input_layernorm.weight"), cfg.rms_norm_eps, DataType.FLOAT16)
            for i in range(cfg.num_hidden_layers):
                p = f"layers.{i}."
                qkv = self._linear(xn, p + "self_attn.qkv_proj.weight")  # [nb*S, width] fp32
                if self._paged:
                    kc, vc = self._scratch_kv   # this sequence's rows of this layer, dense; copied to its pages below
                    seq_off = 0
                else:
                    kc, vc = self._cache.get(i)
                    seq_off = b * nkv * lmax * D * esz
                q = Tensor(DataType.FLOAT16, [nb * S, nq, D], dev, _zero=False)
                base = qkv.data_ptr
                check(lib.axhip_qkv_norm_rope_append(
                    base, width, base + nq * D * 4, width, base + (nq + nkv) * D * 4, width,
                    self._w(p + "self_attn.q_norm.weight").data_ptr, self._w(p + "self_attn.k_norm.weight").data_ptr,
                    int(DataType.FLOAT32), cfg.rms_norm_eps, pos_c.data_ptr, self._inv_freq.data_ptr,
                    cfg.mrope_section[1], cfg.mrope_section[2], None, q.data_ptr, kc.data_ptr + seq_off,
                    vc.data_ptr + seq_off, int(DataType.FLOAT16), nb, S, nq, nkv, D, lmax, current_stream()),
                    "qkv_norm_rope_append")
                attn = Tensor(DataType.FLOAT16, [nb * S, nq * D], dev, _zero=False)
                if D in (64, 128):
                    # causal attention over the rows just appended, on the matrix cores
                    check(lib.axhip_prefill_attention(q.data_ptr, kc.data_ptr + seq_off, vc.data_ptr + seq_off, None,
                                                      attn.data_ptr, int(DataType.FLOAT16), nb, S, nq, nkv, D, lmax,
                                                      current_stream()), "prefill_attention")
                else:
                    # every query row is a "sequence" of the decode kernel over its sequence's cache rows
                    for j in range(nb):
                        off = seq_off + j * nkv * lmax * D * esz
                        check(lib.axhip_gqa_decode(q.data_ptr + j * S * nq * D * esz, kc.data_ptr + off, vc.data_ptr + off,
                                                   vis.data_ptr, attn.data_ptr + j * S * nq * D * esz, ws.data_ptr,
                                                   ws.num_bytes, int(DataType.FLOAT16), S, nq, nkv, D, S, 0, lmax * D, D,
                                                   current_stream()), "gqa_decode")
                if self._paged:
                    L.kv_dense_to_paged(kc, vc, *self._cache.get(i), self._cache.page_table, lens=s_lens, table_row=b)
                attn_out = self._linear(attn, p + "self_attn.o_proj.weight")
                h, xn2 = L.add_rms_norm(attn_out, h, self._w(p + "post_attention_layernorm.weight"), cfg.rms_norm_eps,
                                    DataType.FLOAT16)
                mlp_out = self._mlp(xn2, p)
                nxt = f"layers.{i + 1}.input_layernorm.weight" if i + 1 < cfg.num_hidden_layers else "norm.weight"
                h, xn = L.add_rms_norm(mlp_out, h, self._w(nxt), cfg.rms_norm_eps, DataType.FLOAT16)
            # keep the normalised hidden state of each sequence's last position for the lm_head
            for j in range(nb):
                check(lib.axhip_memcpy_d2d(last_h.data_ptr + (b + j) * H * 2, xn.data_ptr + (j * S + S - 1) * H * 2, H * 2),
                      "copy")
        self._cache.set_lengths(np.full(B, S, np.int32))
        logits = self._linear(last_h, "embed_tokens.weight")
        return logits, L.argmax(logits)

    # ---- captured decode loop ------------------------------------------------------------------
    def start_decode(self, first_ids: np.ndarray, first_pos: np.ndarray, max_new_tokens: int,
                     trace: list | None = None):
        """Sets the static step inputs (ids [B], positions [3,B]) and captures the step.  The
        attention split plan is sized for the lengths the loop will reach.  `trace`, if given, holds
        after every run of the step (eager, or a replay of the captured one) the residual stream entering
        each layer and the one leaving the last, as decode_forward documents; inside a captured step these
        are the graph's own buffers, refreshed by each replay."""
        B = self._batch
        self._ids.copy_from_numpy(np.ascontiguousarray(first_ids, dtype=np.int64).reshape(B))
        self._pos.copy_from_numpy(np.ascontiguousarray(first_pos, dtype=np.int64).reshape(3, B))
        bound = min(self._cache.max_len, len(self._cache) + max_new_tokens + 1)
        if self._paged:
            # pages for every token the loop (and the two runs of a capture) can write: allocated now, so
            # that the captured step never touches the page table
            self._cache.reserve(bound - len(self._cache))
        # the captured attention launches attend to at most `bound` keys and append only below it:
        # generate() refuses to run past it (it would silently drop tokens from the cache otherwise)
        self._decode_bound = bound
        # the tokens of every step are gathered on the device, at the row a device-side counter names
        self._log = Tensor(DataType.INT64, [max(max_new_tokens, 1), B], self._device)
        self._counter = Tensor(DataType.INT64, [1], self._device)

        def step():
            if trace is not None:
                del trace[:]
            logits, nxt = self.decode_forward(self._ids, self._pos, bound, trace=trace)
            # the device-side state of the next step, and the token log: one launch
            L.decode_advance(nxt, self._ids, self._pos, self._cache.seq_lens, self._log, self._counter)
            return logits, nxt

        self._step_fn = step
        return step

    def capture(self):
        """Captures one decode step (after a warm-up run) and rewinds the state both runs advanced."""
        B = self._batch
        ids0 = self._ids.numpy().copy()
        pos0 = self._pos.numpy().copy()
        lens0 = self._cache.seq_lens.numpy().copy()
        g = HIPGraph()
        g.capture(self._step_fn)  # runs the step twice (warm-up + recorded run): cache rows get the same values
        self._ids.copy_from_numpy(ids0)
        self._pos.copy_from_numpy(pos0)
        self._cache.seq_lens.copy_from_numpy(lens0)
        self._counter.copy_from_numpy(np.zeros(1, np.int64))
        self._graph = g
        self._graph_out = g.outputs
        return g

    def generate(self, max_new_tokens: int, use_graph: bool = True):
        """Greedy decode loop.  Returns int64 [steps, B] of generated ids.  The tokens of every step
        are gathered on the device (by the step itself) and read back once at the end."""
        if max_new_tokens > self._log.shape[0]:
            raise ValueError("generate(): more steps than start_decode() was told to expect")
        have = len(self._cache)
        if have + max_new_tokens > self._cache.max_len:
            raise RuntimeError(f"generate(): the KV cache is full ({have} of {self._cache.max_len} positions used, "
                               f"{max_new_tokens} more asked for)")
        if have + max_new_tokens > self._decode_bound:
            raise RuntimeError(f"generate(): the step was set up by start_decode() for sequences of up to "
                               f"{self._decode_bound} keys; {have} cached + {max_new_tokens} new exceed that. "
                               f"Call start_decode() (and capture()) again for the new length")
        self._counter.copy_from_numpy(np.zeros(1, np.int64))
        L.synchronize()
        for _ in range(max_new_tokens):
            if use_graph:
                # on the graph's own stream, one replay behind the other: ordering every replay against
                # the default stream as well (launch()) puts two event waits between consecutive steps,
                # measured 8 % of the step
                self._graph.launch_async()
            else:
                self._step_fn()
        if use_graph:
            self._graph.sync()
        L.synchronize()
        if self._fused_tail:
            # the persistent launch needs all its workgroups resident at once; a barrier wait that ran out means
            # something else held compute units, and the tokens of those steps are not to be trusted
            failed = L.decode_layer_tail_failed_waits(reset=True)
            if failed:
                raise RuntimeError(f"generate(): {failed} barrier waits of the fused layer launch ran out; "
                                   "run the model with fused_tail=False when other work shares the device")
        self._cache.note_advanced(max_new_tokens)   # the steps advanced the lengths on the device
        return self._log.numpy()[:max_new_tokens].copy()
