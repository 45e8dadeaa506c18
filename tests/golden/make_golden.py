"""Writes tests/golden/decode_path_golden.npz: seeded inputs and the outputs of the REFERENCE's own
CPU operators for them, taken from `oracle/_ref` (the reference's C++ compiled from its sources by
oracle/Makefile).  Run in the build container, where the reference sources exist:

    python tests/golden/make_golden.py

The fixture is data only (inputs and expected outputs); it lets the restatement and the HIP path be
checked against the reference's results on machines that have no reference sources.
Inputs use the legacy `RandomState` streams (bit-stable across NumPy versions), the same generator
family the reference's tests use.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402


def main():
    ref = oracle.ref
    if ref is None:
        raise SystemExit("oracle/_ref is not built: run `make -C oracle ref` where /root/reference exists")
    g = {}
    rs = np.random.RandomState(3)
    # reference-shaped decode attention, Hq16/Hkv8/D128 (tests/core/test_gqa.py:33-42 shapes)
    for L in (1, 7, 40):
        q = rs.randn(1, 16, 128).astype(np.float32)
        k = rs.randn(L, 8, 128).astype(np.float32)
        v = rs.randn(L, 8, 128).astype(np.float32)
        g[f"gqa_L{L}_q"], g[f"gqa_L{L}_k"], g[f"gqa_L{L}_v"] = q, k, v
        g[f"gqa_L{L}_out"] = ref.sdpa(q, k, v, False)
    # the same on fp16-rounded data (how fp16 parity is defined: fp32 math on fp16-rounded inputs)
    q = rs.randn(1, 16, 128).astype(np.float16)
    k = rs.randn(60, 8, 128).astype(np.float16)
    v = rs.randn(60, 8, 128).astype(np.float16)
    g["gqa16_q"], g["gqa16_k"], g["gqa16_v"] = q, k, v
    g["gqa16_out"] = ref.sdpa(q.astype(np.float32), k.astype(np.float32), v.astype(np.float32), False)
    # causal prefill attention, small
    q = rs.randn(6, 4, 16).astype(np.float32)
    k = rs.randn(6, 2, 16).astype(np.float32)
    v = rs.randn(6, 2, 16).astype(np.float32)
    g["sdpa_q"], g["sdpa_k"], g["sdpa_v"] = q, k, v
    g["sdpa_causal_out"] = ref.sdpa(q, k, v, True)
    g["sdpa_full_out"] = ref.sdpa(q, k, v, False)

    rs = np.random.RandomState(1)
    x = rs.randn(2, 2048).astype(np.float32)
    r = rs.randn(2, 2048).astype(np.float32)
    w = (1 + 0.02 * rs.randn(2048)).astype(np.float32)
    g["arn_x"], g["arn_res"], g["arn_w"] = x, r, w
    g["arn_y"], g["arn_out"] = ref.add_rms_norm(x, r, w, 1e-6)
    g["rms_out"] = ref.rms_norm(x, w, 1e-6)

    rs = np.random.RandomState(0)
    gate = np.concatenate([rs.randn(37 * 53), [-10, -1, 0, 1, 10, -30, 30, 88]]).astype(np.float32)
    up = np.concatenate([rs.randn(37 * 53), np.ones(8)]).astype(np.float32)
    g["silu_gate"], g["silu_up"] = gate, up
    g["silu_out"] = ref.silu_mul(gate, up)

    rs = np.random.RandomState(5)
    x = rs.randn(8, 4, 128).astype(np.float32)
    pos = np.array([0, 1, 2, 63, 1000, 4095, 8191, 5555], np.int64)
    g["rope_x"], g["rope_pos"] = x, pos
    g["rope_out_theta1e6"] = ref.rope(x, pos, 1e6)
    g["rope_out_theta1e4"] = ref.rope(x, pos, 1e4)
    inv = oracle.port.rope_inv_freq(1e6, 128)
    pos3 = rs.randint(0, 8192, size=(3, 8)).astype(np.int64)
    g["mrope_inv_freq"], g["mrope_pos3"] = inv, pos3
    g["rope_thd_out"] = ref.rope_thd(x, pos3, inv, [24, 20, 20])
    g["mrope_cos"], g["mrope_sin"] = ref.mrope_cos_sin(pos3, inv, 20, 20)
    g["rope_cos_sin_out"] = ref.rope_with_cos_sin(x, g["mrope_cos"], g["mrope_sin"])

    rs = np.random.RandomState(6)
    x = rs.randn(16, 256).astype(np.float16)
    w = (0.02 * rs.randn(96, 256)).astype(np.float16)
    b = (0.1 * rs.randn(96)).astype(np.float16)
    g["lin_x"], g["lin_w"], g["lin_b"] = x, w, b
    g["lin_out"] = ref.linear(x.astype(np.float32), w.astype(np.float32))
    g["lin_out_bias"] = ref.linear(x.astype(np.float32), w.astype(np.float32), b.astype(np.float32))

    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "decode_path_golden.npz")
    np.savez_compressed(out, **g)
    print(f"wrote {out}: {len(g)} arrays, {os.path.getsize(out)} bytes")


if __name__ == "__main__":
    main()
