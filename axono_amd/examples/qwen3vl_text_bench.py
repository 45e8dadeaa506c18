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


def run(decode_steps: int = 128, batch: int = 16, context: int = 4096, seed: int = 0, log=print,
        cpu_step_hook=None, cfg: TextConfig | None = None, fused_tail: bool = False) -> dict:
    """cpu_step_hook(cfg, weights, model, first_ids, pos, batch, max_len, log) -> dict, if given, runs
    after the prefill with the model positioned at the first decode step (the benchmark passes a
    hook that times and compares a CPU restatement of one step); its dict is merged into the result."""
    cfg = cfg or TextConfig()
    t0 = time.perf_counter()
    weights = random_weights(cfg, seed)
    log(f"[decode] random weights: {sum(w.size for w in weights.values()) / 1e9:.2f} G params in {time.perf_counter() - t0:.1f} s")
    max_len = context + decode_steps + 1
    max_len = (max_len + 127) // 128 * 128
    model = Qwen3VLTextDecoder(cfg, weights, batch, max_len, "hip:0")
    model.fused_tail = fused_tail
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
    model.cache.seq_lens.copy_from_numpy(state[2])
    model.cache._host_len = context
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
    result.update({
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
    ap.add_argument("--fused-tail", action="store_true",
                    help="each layer's post-attention part as one persistent launch (measured slower; off by default)")
    args = ap.parse_args(argv)
    if args.gqa_two_kernels:
        from .. import _lib
        _lib.load().axhip_gqa_decode_tune(-1, args.gqa_two_kernels)
    res = run(args.steps, args.batch, args.context, log=lambda *a: print(*a, file=sys.stderr, flush=True),
              fused_tail=args.fused_tail)
    print(json.dumps(res), flush=True)


if __name__ == "__main__":
    main()
