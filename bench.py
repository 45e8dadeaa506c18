#!/usr/bin/env python3
"""Benchmark of the decode hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  The metric is the headline one of this build: "GQA decode HBM GB/s (% of peak) B=32 L=8k
fp16; decode tok/s 2B-shape B=16".  `value` is the first half: achieved algorithmic GB/s of the
split-K GQA decode attention at B=32, Hq=16, Hkv=8, D=128, L=8192, fp16 KV cache resident in HBM.
A "step" is one pass of that operator over one batch (one launch: at this shape every sequence is one key
range of one workgroup, so nothing is merged).  The second half
(tokens/s of the Qwen3-VL-2B-shaped text decode step, B=16, 128 hipGraph replays) is reported in
`decode_step` on the same line.

Algorithmic bytes per step: 4096 * sum_b L_b (K and V: 2 * Hkv * D * 2 bytes per token) + 8192 * B
(q and out) = 1 074 003 968 B.  Split-K workspace traffic is not credited.  Several KV buffers are
rotated so that no step can find its cache lines in the 256 MB Infinity Cache.

The CPU baseline runs Axono's own CPU operator (oracle/_ref, compiled from the reference's sources)
or, where that is absent, the C restatement, on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
# HBM bytes per launch of the headline split kernel, from the rocprofv3 --pmc runs recorded in
# profiles/gqa_decode_split_B32_L8192_f16.md: reported when the counters cannot be read live (measure_traffic)
MEASURED_TRAFFIC_BYTES = 1074196367

F16 = 4


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def gqa_bytes(B, L_sum, Hq=16, Hkv=8, D=128, esz=2):
    return 2 * Hkv * D * esz * L_sum + 2 * Hq * D * esz * B


class GqaBench:
    """Headline workload: fp16 cache [B,Hkv,L,D], one query token per sequence."""

    def __init__(self, B=32, L=8192, Hq=16, Hkv=8, D=128, n_rot=4, seed=0, lens=None):
        from axono_amd import _lib
        from axono_amd.device import DeviceBuffer, check

        self.lib = _lib.load()
        self.check = check
        self.B, self.L, self.Hq, self.Hkv, self.D = B, L, Hq, Hkv, D
        rng = np.random.default_rng(seed)
        cache_elems = B * Hkv * L * D
        # one 64 MiB block of N(0,1) fp16 values tiled over every buffer at shifting offsets: the
        # values do not affect the timing and the parity check below uses its own small case
        block = rng.standard_normal(32 * 1024 * 1024).astype(np.float32).astype(np.float16)
        self.kv = []
        for r in range(n_rot):
            kb, vb = DeviceBuffer(cache_elems * 2), DeviceBuffer(cache_elems * 2)
            for buf, shift in ((kb, 2 * r), (vb, 2 * r + 1)):
                off = 0
                rolled = np.roll(block, 4099 * (shift + 1))
                while off < cache_elems * 2:
                    n = min(rolled.nbytes, cache_elems * 2 - off)
                    buf.upload(rolled[: n // 2], off)
                    off += n
            self.kv.append((kb, vb))
        q = rng.standard_normal((B, Hq, D)).astype(np.float32).astype(np.float16)
        self.q = DeviceBuffer.from_numpy(q)
        self.out = DeviceBuffer(q.nbytes)
        self.lens_host = None if lens is None else np.asarray(lens, np.int32)
        self.lens = DeviceBuffer.from_numpy(self.lens_host) if lens is not None else None
        self.ws_bytes = self.lib.axhip_gqa_decode_workspace_bytes(B, Hq, Hkv, D, L)
        self.ws = DeviceBuffer(max(self.ws_bytes, 256))
        self.step_i = 0
        L_sum = int(self.lens_host.sum()) if lens is not None else B * L
        self.bytes_per_step = gqa_bytes(B, L_sum, Hq, Hkv, D)

    def step(self):
        kb, vb = self.kv[self.step_i % len(self.kv)]
        self.step_i += 1
        B, Hq, Hkv, D, L = self.B, self.Hq, self.Hkv, self.D, self.L
        self.check(self.lib.axhip_gqa_decode(self.q.ptr, kb.ptr, vb.ptr, self.lens.ptr if self.lens else None,
                                             self.out.ptr, self.ws.ptr, self.ws_bytes, F16, B, Hq, Hkv, D, L,
                                             Hkv * L * D, L * D, D, None), "gqa_decode")

    def plan(self):
        s, c = C.c_int(0), C.c_int(0)
        self.lib.axhip_gqa_decode_plan(self.B, self.Hq, self.Hkv, self.L, C.byref(s), C.byref(c))
        return {"n_splits": s.value, "chunk": c.value}


def time_steps(lib, step, steps, warmup):
    """Returns (wall ms per step, HIP-event ms per step) over exactly `steps` steps."""
    from axono_amd.device import check

    for _ in range(warmup):
        step()
    check(lib.axhip_synchronize(), "sync")
    e0, e1 = C.c_void_p(), C.c_void_p()
    check(lib.axhip_event_create(C.byref(e0)), "event")
    check(lib.axhip_event_create(C.byref(e1)), "event")
    t0 = time.perf_counter()
    check(lib.axhip_event_record(e0, None), "event_record")  # same stream as the kernels (default)
    for _ in range(steps):
        step()
    check(lib.axhip_event_record(e1, None), "event_record")
    check(lib.axhip_synchronize(), "sync")
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ms = C.c_float(0)
    check(lib.axhip_event_elapsed_ms(e0, e1, C.byref(ms)), "event_elapsed")
    lib.axhip_event_destroy(e0)
    lib.axhip_event_destroy(e1)
    return wall_ms, ms.value / steps


def cpu_baseline_gqa(budget_s=12.0):
    """Axono's CPU attention on B_s sequences of the headline shape (fp32 math on fp16-rounded
    data), threads = host cores.  Returns the cpu_baseline object."""
    import oracle

    cores = oracle.port.num_threads()
    kind = "reference" if oracle.ref is not None else "port"
    ops = oracle.ref if oracle.ref is not None else oracle.port
    rng = np.random.default_rng(1)
    L, Hq, Hkv, D = 8192, 16, 8, 128
    q = rng.standard_normal((1, Hq, D)).astype(np.float16).astype(np.float32)
    k = rng.standard_normal((L, Hkv, D)).astype(np.float16).astype(np.float32)
    v = rng.standard_normal((L, Hkv, D)).astype(np.float16).astype(np.float32)
    ops.sdpa(q, k, v, False)  # warm
    n, t_total, best = 0, 0.0, float("inf")
    while t_total < budget_s and n < 4096:
        t0 = time.perf_counter()
        ops.sdpa(q, k, v, False)
        dt = time.perf_counter() - t0
        best = min(best, dt)
        t_total += dt
        n += 1
    gbs = gqa_bytes(1, L) / best / 1e9
    return {"value": round(gbs, 3), "unit": "GB/s", "cores": cores, "cpu_model": host_cpu_model(), "kind": kind,
            "sample": f"one sequence of the headline shape (B=1 of 32, L=8192, Hq16/Hkv8/D128), "
                      f"min of {n} runs, fp32 arithmetic on fp16-rounded data; bytes counted as fp16"}


def cpu_decode_step_hook(cfg, weights, model, first, pos, batch, max_len, log):
    """One decode step of the CPU restatement from the post-prefill cache, timed, and compared with
    the device's eager step from the same state."""
    from oracle.decode_step import OracleDecoder
    import oracle

    cpu = OracleDecoder(cfg, weights, batch, max_len)
    ctx = int(model.cache.seq_lens.to_numpy()[0])
    for i in range(cfg.num_hidden_layers):
        kc, vc = model.cache.get(i)
        cpu.k[i][:] = kc.numpy()
        cpu.v[i][:] = vc.numpy()
    cpu.lens[:] = ctx
    # device: one eager step with the residual stream of every layer kept, then rewind
    state = (model._ids.numpy().copy(), model._pos.numpy().copy(), model.cache.seq_lens.numpy().copy())
    trace = []
    g_logits, g_next = model.decode_forward(model._ids, model._pos, trace=trace)
    g_logits, g_next = g_logits.to_numpy().copy(), g_next.to_numpy().copy()
    h_gpu = [t.to_numpy().copy() for t in trace]
    del trace
    for name in list(weights):  # widen the weights outside the timed region
        if weights[name].dtype == np.float16:
            cpu.W(name)
    # (1) free-running CPU step, timed: the baseline, and end-to-end logits
    snap = [(cpu.k[i][:, :, ctx].copy(), cpu.v[i][:, :, ctx].copy()) for i in range(cfg.num_hidden_layers)]
    t0 = time.perf_counter()
    c_logits, c_next = cpu.decode_step(first, pos)
    cpu_s = time.perf_counter() - t0
    err = float(np.abs(g_logits - c_logits).max())
    # greedy tokens: how many sequences choose the same token, and for those that do not, how far below
    # the restatement's maximum the device's choice lies in the restatement's own logits (a near-tie)
    chosen = c_logits[np.arange(batch), g_next]
    same_tok = int(np.sum(g_next == c_next))
    tie_gap = float((c_logits.max(-1) - chosen).max())
    agree = bool(same_tok == batch)
    # (2) layer-wise, every layer evaluated from the device's own input to that layer
    cpu.lens[:] = ctx
    for i, (kk, vv) in enumerate(snap):
        cpu.k[i][:, :, ctx], cpu.v[i][:, :, ctx] = kk, vv
    outs, tf_logits = cpu.decode_layers_teacher_forced(h_gpu, pos)
    layer_err = max(float(np.abs(outs[i] - h_gpu[i + 1]).max()) for i in range(cfg.num_hidden_layers))
    h_abs = max(float(np.abs(h).max()) for h in h_gpu)
    tf_logit_err = float(np.abs(tf_logits - g_logits).max())
    # (3) the same step in float64 with the same fp16 storage points (NumPy): the yardstick for the drift of
    # two correct fp32 pipelines.  Free-running from the same cache, and layer-wise from the device's inputs.
    from oracle.f64_ops import F64Ops

    def restore_row():
        cpu.lens[:] = ctx
        for i, (kk, vv) in enumerate(snap):
            cpu.k[i][:, :, ctx], cpu.v[i][:, :, ctx] = kk, vv

    restore_row()
    t0 = time.perf_counter()
    cpu64 = OracleDecoder(cfg, weights, batch, 1, ops=F64Ops())
    cpu64.k, cpu64.v, cpu64.lens, cpu64._w32 = cpu.k, cpu.v, cpu.lens, cpu._w32   # same cache arrays, same widened weights
    l64, _ = cpu64.decode_step(first, pos)
    restore_row()
    outs64, tf64 = cpu64.decode_layers_teacher_forced(h_gpu, pos)
    f64_s = time.perf_counter() - t0
    d_gpu = float(np.abs(g_logits - l64).max())
    d_cpu = float(np.abs(c_logits - l64).max())
    layer_gpu = max(float(np.abs(h_gpu[i + 1] - outs64[i]).max()) for i in range(cfg.num_hidden_layers))
    layer_cpu = max(float(np.abs(outs[i] - outs64[i]).max()) for i in range(cfg.num_hidden_layers))
    tf_gpu, tf_cpu = float(np.abs(g_logits - tf64).max()), float(np.abs(tf_logits - tf64).max())
    log(f"[decode] float64 yardstick ({f64_s:.0f} s): free-running logits |device - f64| {d_gpu:.2e}, |fp32 restatement - f64| "
        f"{d_cpu:.2e}; per layer on identical inputs |device - f64| {layer_gpu:.2e}, |restatement - f64| {layer_cpu:.2e}")
    log(f"[decode] CPU restatement: one step in {cpu_s:.1f} s ({batch / cpu_s:.2f} tok/s, {oracle.port.num_threads()} threads)")
    log(f"[decode] parity, each layer on identical inputs: max abs err of the residual stream {layer_err:.2e} "
        f"(|h| max {h_abs:.1f}), logits from the same final state {tf_logit_err:.2e}; "
        f"free-running end to end: logits {err:.2e} (|logits| max {np.abs(c_logits).max():.2f}), greedy tokens agree: {agree}")
    cpu.drop_cache()
    base = {"value": round(batch / cpu_s, 3), "unit": "tok/s", "cores": oracle.port.num_threads(),
            "cpu_model": host_cpu_model(), "kind": "port",
            "sample": f"1 decode step (batch {batch}, context {ctx}) of the C restatement from the post-prefill cache"}
    par = {"per_layer_max_abs_err_identical_inputs": layer_err, "residual_abs_max": h_abs,
           "logits_max_abs_err_identical_final_state": tf_logit_err,
           "logits_max_abs_err_free_running": err, "logits_abs_max": float(np.abs(c_logits).max()),
           "greedy_tokens_agree": agree, "greedy_tokens_equal": f"{same_tok}/{batch}",
           "restatement_logit_gap_of_device_choice": tie_gap,
           "float64_yardstick": {
               "logits_free_running": {"device_vs_f64": d_gpu, "restatement_vs_f64": d_cpu},
               "per_layer_identical_inputs": {"device_vs_f64": layer_gpu, "restatement_vs_f64": layer_cpu},
               "logits_identical_final_state": {"device_vs_f64": tf_gpu, "restatement_vs_f64": tf_cpu},
               "device_within_1p5x_of_restatement": bool(d_gpu <= max(1.5 * d_cpu, 1e-3)),
               "per_layer_within_2e-3": bool(layer_gpu <= 2e-3)},
           "note": "fp16 storage points let two correct fp32 pipelines drift apart over 28 layers; f64 = the same op "
                   "sequence in float64 with the same storage points"}
    return {"cpu_baseline": base, "parity": _sig4(par)}



def _cpu_min_us(fn, budget_s=0.6, max_runs=50):
    """min wall time of fn() in microseconds over a bounded number of runs."""
    fn()
    best, spent, n = float("inf"), 0.0, 0
    while spent < budget_s and n < max_runs:
        t0 = time.perf_counter()
        fn()
        dt = time.perf_counter() - t0
        best, spent, n = min(best, dt), spent + dt, n + 1
    return round(best * 1e6, 1)


def config_tables(lib, with_cpu=True):
    """The benchmark configurations 2, 3 and 4 (fused elementwise operators at B = 32, the decode-attention sweep, the
    fp16 Linear), every point timed with HIP events on the device (through the
    C ABI, buffers rotated so that nothing is served from the 256 MB memory-side cache) and, where it costs
    under about a second, the CPU restatement of the same operator on the same shape beside it."""
    from axono_amd.benchmarks import microbench as mb

    out = {"peaks": {"hbm_GBps": HBM_PEAK_GBS, "mfma_f16_dense_TFLOPs": mb.MFMA_F16_PEAK},
           "how": "HIP events around back-to-back launches, us per launch, buffers rotated; config 4: bytes = 2KN+2MK+4MN, "
                  "flops = 2MKN, weights packed; frac = of the bound's peak; cpu_us = the CPU restatement on the same shape"}
    port = None
    if with_cpu:
        import oracle
        port = oracle.port
        out["cpu_threads"] = port.num_threads()
    rng = np.random.default_rng(2)

    def h16(*shape, scale=1.0):
        return (scale * rng.standard_normal(shape)).astype(np.float32).astype(np.float16).astype(np.float32)

    # ---- config 2: the fused elementwise operators at B = 32 -----------------------------------------
    c2 = []
    for r in mb.collect(mb.bench_rowops, lib, 200, (32,)):
        c2.append({"op": r["op"], "us": r["us"], "bytes": r["bytes"], "GBps": r["GBps"],
                   "frac_hbm": round(r["GBps"] / HBM_PEAK_GBS, 5)})
    if port is not None:
        x, res, w = h16(32, 2048), h16(32, 2048), 1 + 0.02 * h16(2048)
        g, u = h16(32, 6144), h16(32, 6144)
        q, k = h16(32, 16, 128), h16(32, 8, 128)
        pos = rng.integers(0, 8192, 32).astype(np.int64)
        kc = np.zeros((32, 8, 8192, 128), np.float16)
        vc = np.zeros_like(kc)
        kn, vn = k.astype(np.float16), h16(32, 8, 128).astype(np.float16)
        cpu = {"add_rms_norm": lambda: port.add_rms_norm(x, res, w, 1e-6), "silu_mul": lambda: port.silu_mul(g, u),
               "rope": lambda: (port.rope(q, pos, 1e6), port.rope(k, pos, 1e6)),
               "kv_append": lambda: port.kv_append(kn, vn, kc, vc, pos)}
        for rec in c2:
            for name, fn in cpu.items():
                if rec["op"].startswith(name):
                    rec["cpu_us"] = _cpu_min_us(fn)
        del kc, vc
    out["config2_elementwise_B32"] = c2

    # ---- config 3: the decode-attention sweep --------------------------------------------------------
    c3 = []
    cpu_seq_us = {}
    if port is not None:
        for L in (1024, 8192, 32768):
            q1, k1, v1 = h16(1, 16, 128), h16(L, 8, 128), h16(L, 8, 128)
            cpu_seq_us[L] = _cpu_min_us(lambda: port.sdpa(q1, k1, v1, False), budget_s=0.8)
    points = [(B, L, None) for B in (1, 8, 32, 64) for L in (1024, 8192, 32768)]
    points.append((32, 32768, np.random.default_rng(0).integers(512, 32769, 32)))
    for B, L, lens in points:
        nbytes = gqa_bytes(B, int(lens.sum()) if lens is not None else B * L)
        steps = int(max(10, min(200, 0.15 / (nbytes / 6e12))))
        r = mb.collect(mb.bench_gqa, lib, B, L, steps, lens)[0]
        rec = {"B": B, "L": L, "ragged_512_32768": lens is not None, "us": r["us"], "bytes": r["bytes"],
               "GBps": r["GBps"], "frac_hbm": round(r["GBps"] / HBM_PEAK_GBS, 4),
               "ranges_per_seq": r["splits"], "keys_per_range": r["chunk"]}
        if lens is None and L in cpu_seq_us:
            rec["cpu_us_one_sequence"] = cpu_seq_us[L]
        c3.append(rec)
    out["config3_gqa_decode_sweep"] = c3
    # the headline shape through a paged cache whose pages were handed out in a random order (and the dense cache
    # of the same buffers beside it)
    out["config3_paged_cache_random_pages"] = [
        {"form": r["op"], "B": r["B"], "L": r["L"], "pages": r["pages"], "us": r["us"], "bytes": r["bytes"], "GBps": r["GBps"],
         "frac_hbm": round(r["GBps"] / HBM_PEAK_GBS, 4)} for r in mb.collect(mb.bench_gqa_paged, lib, 32, 8192, 100)]

    # ---- config 4: the fp16 Linear ---------------------------------------------------------------------
    c4 = []
    shapes = [(2048, 2048), (2048, 4096), (2048, 12288), (6144, 2048), (2048, 151936)]
    for r in mb.collect(mb.bench_linear, lib, 40, shapes, (1, 16, 32, 512), True, 0):
        M, K, N = r["M"], r["K"], r["N"]
        rec = {"M": M, "K": K, "N": N, "us": r["us"]}
        if M <= 32:
            rec.update({"bound": "hbm", "GBps": r["GBps"], "TFLOPs": None, "frac": round(r["GBps"] / HBM_PEAK_GBS, 4)})
        else:
            rec.update({"bound": "mfma", "GBps": None, "TFLOPs": r["TFLOPs"], "frac": round(r["TFLOPs"] / mb.MFMA_F16_PEAK, 4)})
        if port is not None and 2.0 * M * K * N <= 2.1e9:
            xw, ww = h16(M, K), h16(N, K, scale=0.02)
            rec["cpu_us"] = _cpu_min_us(lambda: port.linear(xw, ww), budget_s=0.5, max_runs=5)
        c4.append(rec)
    out["config4_linear_f16_packed"] = c4
    return {k: (_compact(v) if isinstance(v, list) else v) for k, v in out.items()}


def _sig4(x):
    """Floats of a nested dict rounded to four significant digits (distances are quoted, not compared)."""
    if isinstance(x, dict):
        return {k: _sig4(v) for k, v in x.items()}
    if isinstance(x, float):
        return float(f"{x:.4g}")
    return x


def _compact(rows):
    """A list of flat records as {"cols": [...], "rows": [[...], ...]} (the JSON line stays short); nested
    values and missing keys are kept (None where a record lacks a column)."""
    cols = []
    for r in rows:
        for k in r:
            if k not in cols:
                cols.append(k)
    return {"cols": cols, "rows": [[r.get(c) for c in cols] for r in rows]}


def measure_traffic(log, timeout_s=60):
    """HBM bytes per launch of the headline kernel, read from the hardware counters in child processes: four short
    `rocprofv3 --pmc` runs (FETCH_SIZE, then WRITE_SIZE, for the attention microbenchmark and for a plain copy
    kernel of 1 GiB each way, which gives each counter's scale factor).  Returns (bytes, details) or None when
    the profiler is not usable here (the recorded constant is reported then)."""
    import csv
    import glob
    import shutil
    import subprocess
    import tempfile

    exe = shutil.which("rocprofv3") or "/opt/rocm/bin/rocprofv3"
    if not os.path.exists(exe):
        return None
    env = dict(os.environ, PYTHONPATH=ROOT + os.pathsep + os.environ.get("PYTHONPATH", ""), TMPDIR="/tmp")
    base = tempfile.mkdtemp(prefix="axhip_pmc_", dir="/tmp")
    readings = {}

    def run_group(cmd):
        """Runs cmd in a process group of its own and ends the whole group on every exit path (the profiler
        starts helpers that can outlive it); returns its exit code, or None after the time limit."""
        import signal
        proc = subprocess.Popen(cmd, cwd="/tmp", env=env, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL,
                                start_new_session=True)
        try:
            return proc.wait(timeout=timeout_s)
        except subprocess.TimeoutExpired:
            return None
        finally:
            try:
                os.killpg(proc.pid, signal.SIGKILL)
            except (ProcessLookupError, PermissionError):
                pass
            try:
                proc.wait(timeout=10)
            except subprocess.TimeoutExpired:
                pass

    try:
        for counter in ("FETCH_SIZE", "WRITE_SIZE"):
            for what, kernel in (("gqa", "gqa_decode_split_kernel"), ("copy", "copy_bytes_kernel")):
                out = os.path.join(base, f"{counter}_{what}")
                cmd = [exe, "--pmc", counter, "-d", out, "-o", "p", "--output-format", "csv", "--", sys.executable, "-m",
                       "axono_amd.benchmarks.microbench", what, "--steps", "3"]
                rc = run_group(cmd)
                if rc is None:
                    log("traffic counters: a profiler run exceeded its time limit; the recorded constant is reported")
                    return None
                files = glob.glob(os.path.join(out, "**", "*counter_collection.csv"), recursive=True)
                if rc != 0 or not files:
                    log(f"traffic counters: profiler run ended with code {rc} and {len(files)} result files; "
                        "the recorded constant is reported")
                    return None
                with open(files[0]) as fh:
                    vals = [float(row["Counter_Value"]) for row in csv.DictReader(fh)
                            if kernel in row["Kernel_Name"] and row["Counter_Name"] == counter]
                if not vals:
                    return None
                readings[(counter, what)] = sum(vals) / len(vals)   # KiB per dispatch
        gib_kib = float(1 << 20)  # the copy kernel moves 1 GiB each way
        f_fetch, f_write = gib_kib / readings[("FETCH_SIZE", "copy")], gib_kib / readings[("WRITE_SIZE", "copy")]
        kib = readings[("FETCH_SIZE", "gqa")] * f_fetch + readings[("WRITE_SIZE", "gqa")] * f_write
        return int(round(kib * 1024)), {"FETCH_SIZE_KiB": round(readings[("FETCH_SIZE", "gqa")], 2),
                                        "WRITE_SIZE_KiB": round(readings[("WRITE_SIZE", "gqa")], 2),
                                        "fetch_factor": round(f_fetch, 5), "write_factor": round(f_write, 5)}
    except (subprocess.TimeoutExpired, OSError, KeyError, ValueError, ZeroDivisionError) as e:
        log(f"traffic counters not read ({type(e).__name__}): the recorded constant is reported")
        return None
    finally:
        shutil.rmtree(base, ignore_errors=True)


def host_cpu_model():
    """The CPU's model name as the kernel reports it (the CPU baselines are quoted with it)."""
    try:
        with open("/proc/cpuinfo") as fh:
            for line in fh:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    import platform
    return platform.processor() or platform.machine() or "unknown CPU"


def device_label(reported):
    """`name (arch)` from the runtime; some driver versions leave the name empty, then the marketing name that
    rocminfo prints for the first GPU agent stands in."""
    if reported.split("(")[0].strip():
        return reported
    import shutil
    import subprocess
    exe = shutil.which("rocminfo") or "/opt/rocm/bin/rocminfo"
    try:
        txt = subprocess.run([exe], capture_output=True, text=True, timeout=20).stdout
        names = [l.split(":", 1)[1].strip() for l in txt.splitlines() if l.strip().startswith("Marketing Name")]
        gpus = [n for n in names if n and "EPYC" not in n and "Xeon" not in n and "Ryzen" not in n and "CPU" not in n]
        if gpus:
            return f"{gpus[0]} {reported.strip()}"
    except (OSError, subprocess.SubprocessError):
        pass
    return f"(the driver reports no device name) {reported.strip()}"


def smoke_parity(lib):
    """Small invocation checked against the oracle; raises on mismatch."""
    import oracle
    from axono_amd.device import DeviceBuffer, check

    rng = np.random.default_rng(3)
    B, Hq, Hkv, D, L = 2, 16, 8, 128, 600
    q = rng.standard_normal((B, Hq, D)).astype(np.float32).astype(np.float16)
    k = rng.standard_normal((B, Hkv, L, D)).astype(np.float32).astype(np.float16)
    v = rng.standard_normal((B, Hkv, L, D)).astype(np.float32).astype(np.float16)
    lens = np.array([600, 123], np.int32)
    dq, dk, dv, dl = (DeviceBuffer.from_numpy(a) for a in (q, k, v, lens))
    do = DeviceBuffer(q.nbytes)
    wsb = lib.axhip_gqa_decode_workspace_bytes(B, Hq, Hkv, D, L)
    ws = DeviceBuffer(max(wsb, 256))
    check(lib.axhip_gqa_decode(dq.ptr, dk.ptr, dv.ptr, dl.ptr, do.ptr, ws.ptr, wsb, F16, B, Hq, Hkv, D, L,
                               Hkv * L * D, L * D, D, None), "gqa_decode")
    check(lib.axhip_synchronize(), "sync")
    got = do.download(np.float16, q.shape).astype(np.float32)
    want = oracle.port.gqa_decode_cache_native(q, k, v, lens)
    err = float(np.abs(got - want).max())
    if not err <= 2e-3:
        raise RuntimeError(f"GQA decode parity check failed: max abs err {err}")
    return err


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-decode-step", action="store_true")
    ap.add_argument("--no-configs", action="store_true", help="skip the per-point tables of configurations 2-4")
    ap.add_argument("--no-traffic-counters", action="store_true",
                    help="do not read FETCH_SIZE / WRITE_SIZE through rocprofv3 child processes (report the recorded constant)")
    ap.add_argument("--decode-steps", type=int, default=128)
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU; --gpus N with N > 1 is not supported "
              "(the decode path shards by batch or kv-head with no exchange between devices)", file=sys.stderr)
        sys.exit(2)

    from axono_amd import _lib

    lib = _lib.load()
    if _lib.device_count() < 1:
        print("bench.py: no HIP device visible", file=sys.stderr)
        sys.exit(3)
    name = C.create_string_buffer(256)
    gfx, tot, cus = C.c_int(0), C.c_size_t(0), C.c_int(0)
    lib.axhip_device_info(0, name, 256, C.byref(gfx), C.byref(tot), C.byref(cus))
    log(f"device: {device_label(name.value.decode())} CUs={cus.value} mem={tot.value / 2**30:.0f} GiB")
    log(f"host: {host_cpu_model()}, {os.cpu_count()} logical CPUs visible")

    err = smoke_parity(lib)
    log(f"parity (small case vs oracle): max abs err {err:.2e}")

    wl = GqaBench()
    log(f"GQA decode plan: {wl.plan()}  bytes/step={wl.bytes_per_step}")
    wall_ms, ev_ms = time_steps(lib, wl.step, args.steps, args.warmup)
    gbs = wl.bytes_per_step / (ev_ms * 1e-3) / 1e9
    gbs_wall = wl.bytes_per_step / (wall_ms * 1e-3) / 1e9
    log(f"GQA decode: {ev_ms * 1e3:.1f} us/step (events), {wall_ms * 1e3:.1f} us/step (wall): "
        f"{gbs:.0f} GB/s = {100 * gbs / HBM_PEAK_GBS:.1f}% of {HBM_PEAK_GBS:.0f}")

    result = {
        "metric": "GQA decode HBM GB/s (% of peak) B=32 L=8k fp16; decode tok/s 2B-shape B=16",
        "value": round(gbs_wall, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "split-K GQA flash-decoding, fp16 KV cache [B,Hkv,L,D], fp32 accumulate",
                   "B": 32, "Hq": 16, "Hkv": 8, "D": 128, "L": 8192, "plan": wl.plan(),
                   "kv_buffers_rotated": len(wl.kv)},
        "pct_of_hbm_peak": round(100 * gbs_wall / HBM_PEAK_GBS, 2),
        # achieved = algorithmic bytes per step / HIP-event time per step (one launch of the split kernel);
        # traffic = HBM bytes per launch of that kernel from rocprofv3 counters (FETCH_SIZE x 2.0000 +
        # WRITE_SIZE x 1.0000, factors from a 1 GiB copy kernel), see profiles/
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": MEASURED_TRAFFIC_BYTES,
                     "kernel": "gqa_decode_split_kernel<__half,128,2,8> (one range per sequence at this shape: no merge)",
                     "avg_launch_us": round(ev_ms * 1e3, 2), "algorithmic_bytes": wl.bytes_per_step},
    }
    del wl
    if not args.no_traffic_counters:
        # read here, before the decode model takes its memory: the child processes allocate 2 x 1 GiB themselves
        t = measure_traffic(log)
        if t is not None:
            result["roofline"]["traffic"] = t[0]
            result["roofline"]["traffic_source"] = {"how": "rocprofv3 --pmc in child processes of this run, scaled by a "
                                                           "1 GiB copy kernel", **t[1]}
            log(f"HBM traffic per launch by counters: {t[0]} B = {t[0] / result['roofline']['algorithmic_bytes']:.5f} x algorithmic")
        else:
            result["roofline"]["traffic_source"] = "recorded constant (profiles/gqa_decode_split_B32_L8192_f16.md)"

    if not args.no_decode_step:
        try:
            from axono_amd.examples import qwen3vl_text_bench
        except ImportError:
            qwen3vl_text_bench = None
        if qwen3vl_text_bench is not None:
            hook = None if args.no_cpu_baseline else cpu_decode_step_hook
            result["decode_step"] = qwen3vl_text_bench.run(decode_steps=args.decode_steps, log=log, cpu_step_hook=hook)

    if not args.no_configs:
        result["configs"] = config_tables(lib, with_cpu=not args.no_cpu_baseline)
        log(f"configs 2-4: {sum(len(v['rows']) for v in result['configs'].values() if isinstance(v, dict) and 'rows' in v)} points timed")

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline_gqa()
        log(f"cpu baseline: {result['cpu_baseline']}")

    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
