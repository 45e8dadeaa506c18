"""The restatement against the committed outputs of the reference's own CPU operators
(tests/golden/decode_path_golden.npz, written by tests/golden/make_golden.py from oracle/_ref).
Bit for bit: both are compiled without FMA contraction and accumulate in the same order."""
import os

import numpy as np
import pytest

from oracle import port

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "decode_path_golden.npz"))


@pytest.mark.parametrize("L", [1, 7, 40])
def test_gqa_fp32(L):
    np.testing.assert_array_equal(port.gqa_decode(G[f"gqa_L{L}_q"], G[f"gqa_L{L}_k"], G[f"gqa_L{L}_v"]), G[f"gqa_L{L}_out"])


def test_gqa_fp16_rounded_inputs():
    out = port.gqa_decode(G["gqa16_q"].astype(np.float32), G["gqa16_k"].astype(np.float32), G["gqa16_v"].astype(np.float32))
    np.testing.assert_array_equal(out, G["gqa16_out"])


def test_sdpa_causal_and_full():
    np.testing.assert_array_equal(port.sdpa(G["sdpa_q"], G["sdpa_k"], G["sdpa_v"], True), G["sdpa_causal_out"])
    np.testing.assert_array_equal(port.sdpa(G["sdpa_q"], G["sdpa_k"], G["sdpa_v"], False), G["sdpa_full_out"])


def test_fused_and_norm():
    y, out = port.add_rms_norm(G["arn_x"], G["arn_res"], G["arn_w"], 1e-6)
    np.testing.assert_array_equal(y, G["arn_y"])
    np.testing.assert_array_equal(out, G["arn_out"])
    np.testing.assert_array_equal(port.rms_norm(G["arn_x"], G["arn_w"], 1e-6), G["rms_out"])
    np.testing.assert_array_equal(port.silu_mul(G["silu_gate"], G["silu_up"]), G["silu_out"])


def test_rotary():
    x, pos = G["rope_x"], G["rope_pos"]
    np.testing.assert_array_equal(port.rope(x, pos, 1e6), G["rope_out_theta1e6"])
    np.testing.assert_array_equal(port.rope(x, pos, 1e4), G["rope_out_theta1e4"])
    inv, pos3 = G["mrope_inv_freq"], G["mrope_pos3"]
    np.testing.assert_array_equal(port.rope_thd(x, pos3, inv, [24, 20, 20]), G["rope_thd_out"])
    c, s = port.mrope_cos_sin(pos3, inv, 20, 20)
    np.testing.assert_array_equal(c, G["mrope_cos"])
    np.testing.assert_array_equal(s, G["mrope_sin"])
    np.testing.assert_array_equal(port.rope_with_cos_sin(x, c, s), G["rope_cos_sin_out"])


def test_linear_fp16_rounded_operands():
    x, w, b = (G[k].astype(np.float32) for k in ("lin_x", "lin_w", "lin_b"))
    np.testing.assert_array_equal(port.linear(x, w), G["lin_out"])
    np.testing.assert_array_equal(port.linear(x, w, b), G["lin_out_bias"])
