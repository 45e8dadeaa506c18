"""Decode-throughput measurement of the Qwen3-VL-2B-shaped text tower (random init, synthetic ids):
batch 16, a prefilled context of 4096 tokens per sequence, then greedy decode steps replayed from
one captured hipGraph.  tokens/s = batch * steps / wall time of the replays (prefill excluded).

    python -m axono_amd.examples.qwen3vl_text_bench [--steps 128] [--batch 16] [--context 4096]

Per step the device must read every weight once (3.44 GB of fp16) and the whole KV cache of every
layer (28 * 65 536 B per cached token and sequence), which bounds the step at HBM speed.
"""
from __future__ import annotations

import argparse
import json
import sys
import time

import numpy as np

from .. import libaxono as L
from .qwen3vl_text import Qwen3VLTextDecoder, TextConfig, random_weights

HBM_PEAK_GBS = 8000.0


def step_bytes(cfg: TextConfig, batch: int, context: int) -> int:
    """Algorithmic HBM bytes of one decode step at a given cached length."""
    H, D, nq, nkv, I, V = (cfg.hidden_size, cfg.head_dim, cfg.num_attention_heads, cfg.num_key_value_heads,
                           cfg.intermediate_size, cfg.vocab_size)
    per_layer = ((nq + 2 * nkv) * D * H + H * nq * D + 2 * I * H + H * I) * 2
    weights = cfg.num_hidden_layers * per_layer + V * H * 2
    kv = cfg.num_hidden_layers * batch * context * 2 * nkv * D * 2
    return weights + kv


def per_kernel_table(model: Qwen3VLTextDecoder, context: int, reps: int = 10, once_copies: int = 8) -> list:
    """Where a decode step goes, kernel by kernel: every kind of launch of the step is captured as a graph
    of that launch for all layers (each layer's own weights and caches, so nothing is served from the
    memory-side cache) and replayed `reps` times between host clock reads.  Rows: calls per step, us per call
    inside such a back-to-back graph, algorithmic bytes per call and the fraction of HBM peak that is.
    With the fused layer launch the single launches it replaces still run once per step (the last layer; the first
    layer's q/k/v projection): they are timed over all layers as before and counted once.
    The three launches that a step holds once are captured `once_copies` times over, so that the fixed cost of
    replaying a graph (some 20 us, which a one-node graph would charge to its only node) is spread as it is
    in the step; the weight of lm_head is 622 MB, more than the memory-side cache holds, so its copies still
    read HBM.  Run it after the timed loop: the attention launches overwrite the cache row at the current length."""
    from ..core.hip_graph import HIPGraph
    from ..core.tensor import Tensor
    from ..core.types import DataType

    cfg, B = model._cfg, model._batch
    nl, H, D = cfg.num_hidden_layers, cfg.hidden_size, cfg.head_dim
    nq, nkv, I, V = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.intermediate_size, cfg.vocab_size
    rng = np.random.default_rng(0)

    def dev(shape, dtype):
        a = rng.standard_normal(shape).astype(np.float32)
        return Tensor.from_numpy_ref(np.ascontiguousarray(a.astype(np.float16) if dtype == DataType.FLOAT16 else a)).to(model._device)

    xn = dev((B, H), DataType.FLOAT16)
    h = dev((B, H), DataType.FLOAT32)
    qkv = dev((B, (nq + 2 * nkv) * D), DataType.FLOAT32)
    attn = dev((B, nq * D), DataType.FLOAT16)
    act = dev((B, I), DataType.FLOAT16)
    o32 = dev((B, H), DataType.FLOAT32)
    logits = dev((B, V), DataType.FLOAT32)
    lens = model.cache.seq_lens
    W = model._w

    def layers(fn):
        return lambda: [fn(f"layers.{i}.", i) for i in range(nl)]

    def lin_bytes(K, N, out_b):
        return 2 * K * N + 2 * B * K + out_b * B * N

    fused = model._fused_tail
    per = (lambda n: 0 if fused else n)   # with the fused launch no layer runs these as single launches
    n_qkv = (nq + 2 * nkv) * D
    kinds = [
        ("qkv Linear 2048->4096", nl, 1 if fused else nl, lin_bytes(H, n_qkv, 4),
         layers(lambda p, i: model._linear(xn, p + "self_attn.qkv_proj.weight"))),
        ("attention (qk-norm + M-RoPE + KV append + split-K decode + merge)", nl, nl,
         2 * nkv * D * 2 * B * (context + 1) + B * n_qkv * 4 + B * nq * D * 2,
         layers(lambda p, i: model._attention_step(qkv, p, i, model._pos, model._decode_bound))),
        ("o_proj Linear 2048->2048", nl, per(nl), lin_bytes(nq * D, H, 4),
         layers(lambda p, i: model._linear(attn, p + "self_attn.o_proj.weight"))),
        ("add + RMSNorm (fp32 residual, fp16 out)", 2 * nl, 0 if fused else 2 * nl, B * H * (4 + 4 + 4 + 2) + 4 * H,
         lambda: [L.add_rms_norm(o32, h, W(f"layers.{i // 2}.post_attention_layernorm.weight"), cfg.rms_norm_eps,
                                 DataType.FLOAT16) for i in range(2 * nl)]),
        ("gate+up Linear 2048->12288 + SiLU-mul", nl, per(nl), lin_bytes(H, 2 * I, 1),
         layers(lambda p, i: L.linear_packed(xn, model._packed[p + "mlp.gate_up_proj.weight"], 2 * I,
                                             out_dtype=DataType.FLOAT16, glu=True))),
        ("down Linear 6144->2048", nl, per(nl), lin_bytes(I, H, 4), layers(lambda p, i: model._linear(act, p + "mlp.down_proj.weight"))),
        ("lm_head Linear 2048->151936", once_copies, 1, lin_bytes(H, V, 4),
         lambda: [model._linear(xn, "embed_tokens.weight") for _ in range(once_copies)]),
        ("argmax over 151936", once_copies, 1, B * V * 4, lambda: [L.argmax(logits) for _ in range(once_copies)]),
        ("embedding + first RMSNorm", once_copies, 1, B * H * (2 + 4 + 2),
         lambda: [L.embedding_rms_norm(model._ids, W("embed_tokens.weight"), W("layers.0.input_layernorm.weight"),
                                       cfg.rms_norm_eps) for _ in range(once_copies)]),
    ]
    if fused:
        def tails():
            hh = h
            for i in range(nl - 1):
                p, n = f"layers.{i}.", f"layers.{i + 1}."
                hh, _ = L.decode_layer_tail(attn, hh, model._packed[p + "self_attn.o_proj.weight"],
                                            W(p + "post_attention_layernorm.weight"), model._packed[p + "mlp.gate_up_proj.weight"],
                                            model._packed[p + "mlp.down_proj.weight"], W(n + "input_layernorm.weight"),
                                            model._packed[n + "self_attn.qkv_proj.weight"], n_qkv, cfg.rms_norm_eps, model._tail_ws)
        kinds.insert(2, ("layer tail: o_proj + norm + gate/up + SiLU-mul + down + norm + next qkv, one persistent launch",
                         nl - 1, nl - 1, 2 * (nq * D * H + 2 * I * H + H * I + n_qkv * H) + B * (nq * D * 2 + 2 * H * 4 + n_qkv * 4),
                         tails))

        def last_tails():
            hh = h
            for i in range(nl):
                p = f"layers.{i}."
                hh, _ = L.decode_layer_tail_last(attn, hh, model._packed[p + "self_attn.o_proj.weight"],
                                                 W(p + "post_attention_layernorm.weight"),
                                                 model._packed[p + "mlp.gate_up_proj.weight"],
                                                 model._packed[p + "mlp.down_proj.weight"], W("norm.weight"), cfg.rms_norm_eps,
                                                 model._tail_ws)
        kinds.insert(3, ("last layer's tail: the same launch closed by the final norm", nl, 1,
                         2 * (nq * D * H + 2 * I * H + H * I) + B * (nq * D * 2 + 2 * H * 4 + H * 2), last_tails))
        # the single operators below are not part of the fused step: listed for comparison
    rows = []
    for name, graph_calls, calls, nbytes, fn in kinds:
        g = HIPGraph()
        g.capture(fn)
        g.replay()
        L.synchronize()
        # the graph replays on its own stream: host clock around the launch ... sync of `reps` replays
        t0 = time.perf_counter()
        for _ in range(reps):
            g.launch_async()
        g.sync()
        us = (time.perf_counter() - t0) * 1e6 / (reps * graph_calls)
        g.reset()
        rows.append({"kernel": name, "calls_per_step": calls, "us_per_call": round(us, 2),
                     "us_per_step": round(us * calls, 1), "bytes_per_call": int(nbytes),
                     "frac_hbm_peak": round(nbytes / (us * 1e-6) / (HBM_PEAK_GBS * 1e9), 4)})
    return rows


def run(decode_steps: int = 128, batch: int = 16, context: int = 4096, seed: int = 0, log=print,
        cpu_step_hook=None, cfg: TextConfig | None = None, kernel_table: bool = True, paged: bool = False,
        fused_tail: bool | None = None, plan_reuse: bool = True,
        fused_last: bool = True) -> dict:
    """cpu_step_hook(cfg, weights, model, first_ids, pos, batch, max_len, log) -> dict, if given, runs
    after the prefill with the model positioned at the first decode step (the benchmark passes a
    hook that times and compares a CPU restatement of one step); its dict is merged into the result."""
    cfg = cfg or TextConfig()
    t0 = time.perf_counter()
    weights = random_weights(cfg, seed)
    log(f"[decode] random weights: {sum(w.size for w in weights.values()) / 1e9:.2f} G params in {time.perf_counter() - t0:.1f} s")
    max_len = context + decode_steps + 1
    max_len = (max_len + 127) // 128 * 128
    model = Qwen3VLTextDecoder(cfg, weights, batch, max_len, "hip:0", paged=paged, fused_tail=fused_tail,
                               plan_reuse=plan_reuse, fused_last=fused_last)
    rng = np.random.default_rng(seed + 1)
    ids = rng.integers(0, cfg.vocab_size, (batch, context)).astype(np.int64)

    t0 = time.perf_counter()
    logits0, nxt0 = model.prefill(ids)
    L.synchronize()
    prefill_s = time.perf_counter() - t0
    first = nxt0.to_numpy().copy()
    log(f"[decode] prefill {batch} x {context} tokens: {prefill_s:.2f} s ({batch * context / prefill_s:.0f} tok/s)")

    pos = np.full((3, batch), context, np.int64)
    model.start_decode(first, pos, decode_steps)

    result = {}
    if cpu_step_hook is not None:
        result.update(cpu_step_hook(cfg, weights, model, first, pos, batch, max_len, log))

    g = model.capture()
    log(f"[decode] captured step: {g.num_nodes} graph nodes")
    # warm replays, then rewind the device-side state so the timed loop starts at `context`
    state = (model._ids.numpy().copy(), model._pos.numpy().copy(), model.cache.seq_lens.numpy().copy())
    for _ in range(3):
        g.replay()
    model._ids.copy_from_numpy(state[0])
    model._pos.copy_from_numpy(state[1])
    model.cache.set_lengths(state[2])
    L.synchronize()
    t0 = time.perf_counter()
    toks = model.generate(decode_steps, use_graph=True)  # ends with a device synchronisation
    wall = time.perf_counter() - t0
    tok_s = batch * decode_steps / wall
    ms_step = wall / decode_steps * 1e3
    avg_bytes = (step_bytes(cfg, batch, context) + step_bytes(cfg, batch, context + decode_steps - 1)) / 2
    ceiling = batch / (avg_bytes / (HBM_PEAK_GBS * 1e9))
    lens = model.cache.seq_lens.to_numpy()
    assert np.all(lens == context + decode_steps), lens
    assert toks.shape == (decode_steps, batch) and toks.min() >= 0 and toks.max() < cfg.vocab_size
    log(f"[decode] {decode_steps} replays: {ms_step:.3f} ms/step, {tok_s:.0f} tok/s "
        f"({100 * tok_s / ceiling:.1f}% of the {ceiling:.0f} tok/s HBM ceiling)")
    table = per_kernel_table(model, context + decode_steps) if kernel_table else []
    in_kernels = sum(r["us_per_step"] for r in table)
    for r in table:
        log(f"[decode]   {r['kernel']:<68s} {r['calls_per_step']:3d} x {r['us_per_call']:7.2f} us = {r['us_per_step']:7.1f} us"
            f"  ({100 * r['frac_hbm_peak']:.1f}% of HBM peak)")
    log(f"[decode]   sum of the per-kind graphs {in_kernels:.0f} us of the {ms_step * 1e3:.0f} us step")
    result.update({
        "per_kernel": {"how": "each kind of launch captured for all layers (own weights / caches) and replayed back to "
                              "back; host clock around 10 replays; bytes are algorithmic; a kind with 0 calls per step is "
                              "not part of this step (the single operators the fused layer launch replaces), timed for comparison",
                       "cols": ["kernel", "calls_per_step", "us_per_call", "us_per_step", "bytes_per_call", "frac_hbm_peak"],
                       "rows": [[r["kernel"], r["calls_per_step"], r["us_per_call"], r["us_per_step"], r["bytes_per_call"],
                                 r["frac_hbm_peak"]] for r in table],
                       "sum_us_per_step": round(in_kernels, 1)},
        "metric": "decode tok/s 2B-shape B=16", "value": round(tok_s, 1), "unit": "tok/s",
        "ms_per_step": round(ms_step, 4), "steps": decode_steps, "batch": batch, "context": context,
        "graph_nodes": g.num_nodes, "bytes_per_step": int(avg_bytes),
        "achieved_GBps": round(avg_bytes / (ms_step * 1e-3) / 1e9, 1),
        "hbm_ceiling_tok_s": round(ceiling, 1), "frac_of_ceiling": round(tok_s / ceiling, 4),
        "prefill_s": round(prefill_s, 2), "dtype": "f16 weights + f16 KV cache, f32 residual stream",
        "model": "Qwen3-VL-2B text tower shape, random init (28 layers, hidden 2048, 16/8 heads, d 128, "
                 "inter 6144, vocab 151936, M-RoPE [24,20,20], theta 1e6)",
    })
    return result


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--batch", type=int, default=16)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--gqa-two-kernels", type=int, default=0, metavar="SPLITS",
                    help="attention with a fixed split count and a second merge kernel (the default deals "
                         "workgroups by length and merges in the last workgroup)")
    ap.add_argument("--paged", action="store_true", help="keep the KV cache in pages of 128 keys (nn.PagedKVCache)")
    ap.add_argument("--no-fused-tail", action="store_true",
                    help="run the part of a layer behind its attention as six launches instead of one persistent launch")
    ap.add_argument("--no-plan-reuse", action="store_true",
                    help="every attention launch of a step deals the key ranges itself (default: the first layer's "
                         "launch deals, the others take its table)")
    ap.add_argument("--no-fused-last", action="store_true",
                    help="the last layer as single operators (default: the persistent launch closed by the final norm)")
    ap.add_argument("--no-kernel-table", action="store_true",
                    help="skip the per-kernel table (its extra launches would mix into a profiler's kernel statistics)")
    args = ap.parse_args(argv)
    if args.gqa_two_kernels:
        from .. import _lib
        _lib.load().axhip_gqa_decode_tune(-1, args.gqa_two_kernels)
    res = run(args.steps, args.batch, args.context, log=lambda *a: print(*a, file=sys.stderr, flush=True),
              kernel_table=not args.no_kernel_table, paged=args.paged,
              fused_tail=False if args.no_fused_tail else None, plan_reuse=not args.no_plan_reuse,
              fused_last=not args.no_fused_last)
    print(json.dumps(res), flush=True)


if __name__ == "__main__":
    main()
