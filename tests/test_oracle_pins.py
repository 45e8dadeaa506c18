"""Pins the CPU oracle before anything is compared with it.

Each oracle function is checked against (1) the known-answer NumPy forms and seeds the reference's
own tests use, (2) what the mathematics fixes (special cases, invariants, fp64 brute force) and
(3) the compiled reference (`oracle/_ref`) bit for bit, where that library is present.
"""
import math

import numpy as np
import pytest

import oracle
from oracle import port

REF = oracle.ref
needs_ref = pytest.mark.skipif(REF is None, reason="oracle/_ref not built (reference sources absent)")


# ---- NumPy known-answer forms (as in the reference's tests) -----------------------------------
def np_gqa(q, k, v):
    """tests/core/test_gqa.py:11-25 of the reference."""
    _, hq, d = q.shape
    skv, hkv = k.shape[:2]
    group = hq // hkv
    out = np.zeros((1, hq, d), np.float32)
    for h in range(hq):
        s = (q[0, h] @ k[:, h // group].T) * (1.0 / math.sqrt(d))
        w = np.exp(s - s.max())
        w /= w.sum()
        out[0, h] = w @ v[:, h // group]
    return out


def np_attention(q, k, v, causal):
    """tests/core/test_sequence_ops.py:31-46 of the reference."""
    sq, hq, d = q.shape
    skv, hkv = k.shape[:2]
    group = hq // hkv
    out = np.zeros((sq, hq, d), np.float32)
    for t in range(sq):
        for h in range(hq):
            end = min(t + 1, skv) if causal else skv
            s = q[t, h] @ k[:end, h // group].T / math.sqrt(d)
            p = np.exp(s - s.max())
            p /= p.sum()
            out[t, h] = p @ v[:end, h // group]
    return out


def np_mrope_cos_sin(pos3, theta, d_head, h_sec, w_sec):
    """tests/core/test_sequence_ops.py:252-259 of the reference."""
    inv = 1.0 / (theta ** (np.arange(0, d_head, 2, dtype=np.float32) / d_head))
    freqs = pos3[:, :, None].astype(np.float32) * inv[None, None, :]
    out = freqs[0].copy()
    out[:, np.arange(1, h_sec * 3, 3)] = freqs[1][:, np.arange(1, h_sec * 3, 3)]
    out[:, np.arange(2, w_sec * 3, 3)] = freqs[2][:, np.arange(2, w_sec * 3, 3)]
    ang = np.concatenate([out, out], axis=-1)
    return np.cos(ang), np.sin(ang)


# ---- attention --------------------------------------------------------------------------------
@pytest.mark.parametrize("skv", [1, 7, 256, 512, 1024])
def test_gqa_known_answers_seed3(skv):
    rng = np.random.RandomState(3)
    for L in (1, 7, 256, 512, 1024):  # the reference draws all five in sequence from one stream
        q = rng.randn(1, 16, 128).astype(np.float32)
        k = rng.randn(L, 8, 128).astype(np.float32)
        v = rng.randn(L, 8, 128).astype(np.float32)
        if L == skv:
            np.testing.assert_allclose(port.gqa_decode(q, k, v), np_gqa(q, k, v), rtol=1e-4, atol=1e-4)


def test_gqa_known_answer_seed4_L300():
    rng = np.random.RandomState(4)
    q = rng.randn(1, 16, 128).astype(np.float32)
    k = rng.randn(300, 8, 128).astype(np.float32)
    v = rng.randn(300, 8, 128).astype(np.float32)
    np.testing.assert_allclose(port.gqa_decode(q, k, v), np_gqa(q, k, v), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("causal", [False, True])
def test_sdpa_small_gqa_4_2(causal):
    rng = np.random.RandomState(11)
    q = rng.randn(4, 4, 8).astype(np.float32)
    k = rng.randn(6, 2, 8).astype(np.float32)
    v = rng.randn(6, 2, 8).astype(np.float32)
    np.testing.assert_allclose(port.sdpa(q, k, v, causal), np_attention(q, k, v, causal), rtol=1e-4, atol=1e-5)


def test_sdpa_fp64_brute_force():
    rng = np.random.default_rng(5)
    q = rng.standard_normal((1, 4, 16)).astype(np.float32)
    k = rng.standard_normal((9, 2, 16)).astype(np.float32)
    v = rng.standard_normal((9, 2, 16)).astype(np.float32)
    got = port.sdpa(q, k, v, False)
    for h in range(4):
        s = np.array([np.dot(q[0, h].astype(np.float64), k[j, h // 2].astype(np.float64)) / 4.0 for j in range(9)])
        p = np.exp(s - s.max())
        p /= p.sum()
        want = sum(p[j] * v[j, h // 2].astype(np.float64) for j in range(9))
        np.testing.assert_allclose(got[0, h], want, rtol=2e-6, atol=2e-6)


def test_sdpa_special_cases():
    rng = np.random.default_rng(6)
    q = rng.standard_normal((1, 4, 32)).astype(np.float32)
    v1 = rng.standard_normal((1, 2, 32)).astype(np.float32)
    # a single key: softmax weight 1, the output is that value row of the head's kv group
    out = port.sdpa(q, rng.standard_normal((1, 2, 32)).astype(np.float32), v1, False)
    np.testing.assert_array_equal(out[0, 0], v1[0, 0])
    np.testing.assert_array_equal(out[0, 3], v1[0, 1])
    # identical keys: uniform weights, the output is the mean of V
    k = np.tile(rng.standard_normal((1, 2, 32)).astype(np.float32), (50, 1, 1))
    v = rng.standard_normal((50, 2, 32)).astype(np.float32)
    out = port.sdpa(q, k, v, False)
    np.testing.assert_allclose(out[0, 1], v[:, 0].mean(0), rtol=1e-5, atol=1e-6)
    # a transposed or mis-grouped head mapping would break this: head h reads kv head h//group only
    v2 = v.copy()
    v2[:, 1] += 100.0
    out2 = port.sdpa(q, k, v2, False)
    np.testing.assert_array_equal(out2[0, :2], out[0, :2])
    assert np.all(out2[0, 2:] > out[0, 2:] + 99.0)


def test_gqa_decode_cache_layouts_agree():
    """The batched [B,Hkv,Lmax,D] form is the reference op per sequence on its first L_b rows."""
    rng = np.random.default_rng(8)
    B, hq, hkv, d, lmax = 3, 4, 2, 16, 20
    q = rng.standard_normal((B, hq, d)).astype(np.float32)
    kc = rng.standard_normal((B, hkv, lmax, d)).astype(np.float32)
    vc = rng.standard_normal((B, hkv, lmax, d)).astype(np.float32)
    lens = np.array([20, 1, 13], np.int32)
    a = port.gqa_decode_cache(q, kc, vc, lens)
    b = port.gqa_decode_cache_native(q, kc, vc, lens)
    np.testing.assert_array_equal(a, b)
    for i in range(B):
        kk = np.transpose(kc[i, :, : lens[i]], (1, 0, 2))
        vv = np.transpose(vc[i, :, : lens[i]], (1, 0, 2))
        np.testing.assert_allclose(a[i:i + 1], np_gqa(q[i:i + 1], kk, vv), rtol=1e-4, atol=1e-5)


# ---- fused ------------------------------------------------------------------------------------
def test_silu_mul_known_answers():
    rng = np.random.RandomState(0)
    g = rng.randn(37, 53).astype(np.float32)
    u = rng.randn(37, 53).astype(np.float32)
    np.testing.assert_allclose(port.silu_mul(g, u), g / (1.0 + np.exp(-g)) * u, rtol=1e-5, atol=1e-6)
    e = np.array([-10.0, -1.0, 0.0, 1.0, 10.0], np.float32)
    np.testing.assert_allclose(port.silu_mul(e, np.ones(5, np.float32)), e / (1.0 + np.exp(-e)), rtol=1e-5, atol=1e-6)
    assert port.silu_mul(np.zeros(1, np.float32), np.full(1, 7.0, np.float32))[0] == 0.0
    # silu(x) -> x for large x; up is a plain factor
    np.testing.assert_allclose(port.silu_mul(np.full(1, 30.0, np.float32), np.full(1, -2.0, np.float32)), [-60.0], rtol=1e-6)


def test_add_rms_norm_known_answers():
    rng = np.random.RandomState(1)
    x = rng.randn(4, 128).astype(np.float32)
    r = rng.randn(4, 128).astype(np.float32)
    w = rng.randn(128).astype(np.float32)
    y, out = port.add_rms_norm(x, r, w, 1e-6)
    s = x + r
    np.testing.assert_allclose(y, s, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(out, s / np.sqrt((s ** 2).mean(-1, keepdims=True) + 1e-6) * w, rtol=1e-4, atol=1e-5)


def test_add_rms_norm_chaining_and_invariants():
    rng = np.random.RandomState(2)
    h = rng.randn(2, 64).astype(np.float32)
    a1 = rng.randn(2, 64).astype(np.float32)
    a2 = rng.randn(2, 64).astype(np.float32)
    w = np.ones(64, np.float32)
    h1, _ = port.add_rms_norm(a1, h, w, 1e-6)
    h2, out2 = port.add_rms_norm(a2, h1, w, 1e-6)
    np.testing.assert_allclose(h2, a2 + a1 + h, rtol=1e-5, atol=1e-6)
    # unit weights, eps -> 0: each output row has unit mean square; scaling the inputs changes nothing
    np.testing.assert_allclose((out2.astype(np.float64) ** 2).mean(-1), 1.0, rtol=1e-4)
    _, out4 = port.add_rms_norm(4 * a2, 4 * h1, w, 0.0)
    _, out1 = port.add_rms_norm(a2, h1, w, 0.0)
    np.testing.assert_allclose(out4, out1, rtol=1e-5, atol=1e-6)
    # equals rms_norm of the sum (src/ops/cpu/llm.cpp:65-73)
    np.testing.assert_allclose(port.rms_norm(h2, w, 1e-6), out2, rtol=1e-6, atol=1e-7)
    # eps is inside the square root, added to the mean square
    z = np.zeros((1, 8), np.float32)
    _, oz = port.add_rms_norm(z + 1e-3, z, np.ones(8, np.float32), 1.0)
    np.testing.assert_allclose(oz, 1e-3 / math.sqrt(1e-6 + 1.0), rtol=1e-5)


def test_rms_norm_closed_form_and_no_weight():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((5, 128)).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(128)).astype(np.float32)
    want = x / np.sqrt((x.astype(np.float64) ** 2).mean(-1, keepdims=True) + 1e-6)
    np.testing.assert_allclose(port.rms_norm(x, w, 1e-6), want * w, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(port.rms_norm(x, None, 1e-6), want, rtol=1e-5, atol=1e-6)


# ---- rotary -----------------------------------------------------------------------------------
def test_rope_known_answer():
    """tests/core/test_sequence_ops.py:62-79 of the reference (theta 1e4, positions 0..3)."""
    rng = np.random.RandomState(2027)
    seq, heads, dim = 4, 2, 8
    x = rng.randn(seq, heads, dim).astype(np.float32)
    pos = np.arange(seq, dtype=np.int64)
    half = dim // 2
    inv = 10000.0 ** (-2.0 * np.arange(0, half, dtype=np.float32) / dim)
    want = np.empty_like(x)
    for t in range(seq):
        c, s = np.cos(pos[t] * inv), np.sin(pos[t] * inv)
        for h in range(heads):
            x0, x1 = x[t, h, :half], x[t, h, half:]
            want[t, h, :half] = x0 * c - x1 * s
            want[t, h, half:] = x1 * c + x0 * s
    np.testing.assert_allclose(port.rope(x, pos, 10000.0), want, rtol=1e-4, atol=1e-5)


def test_rope_invariants_theta_1e6():
    rng = np.random.default_rng(9)
    x = rng.standard_normal((6, 3, 128)).astype(np.float32)
    pos = np.array([0, 1, 77, 4095, 8191, 5000], np.int64)
    out = port.rope(x, pos, 1e6)
    np.testing.assert_array_equal(out[0], x[0])  # position 0 is the identity
    # each (i, i+half) pair is rotated: its norm is preserved
    n_in = x[..., :64] ** 2 + x[..., 64:] ** 2
    n_out = out[..., :64] ** 2 + out[..., 64:] ** 2
    np.testing.assert_allclose(n_out, n_in, rtol=1e-5, atol=1e-6)
    # channel 0 has frequency 1: angle = position exactly; the sign convention is (a c - b s, b c + a s)
    a, b = x[2, 0, 0].astype(np.float64), x[2, 0, 64].astype(np.float64)
    np.testing.assert_allclose(out[2, 0, 0], a * math.cos(77.0) - b * math.sin(77.0), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(out[2, 0, 64], b * math.cos(77.0) + a * math.sin(77.0), rtol=1e-5, atol=1e-6)
    # rotations compose at small angles (rounding of the fp32 angle stays small there)
    p1, p2 = np.full(6, 3, np.int64), np.full(6, 5, np.int64)
    np.testing.assert_allclose(port.rope(port.rope(x, p1, 1e6), p2, 1e6), port.rope(x, p1 + p2, 1e6), rtol=1e-4, atol=1e-5)


def test_rope_inv_freq_matches_fp32_closed_form():
    f = port.rope_inv_freq(1e6, 128)
    want = np.float32(1e6) ** (-2.0 * np.arange(64, dtype=np.float32) / np.float32(128))
    np.testing.assert_allclose(f, want, rtol=3e-7)
    assert f[0] == 1.0


def test_mrope_cos_sin_known_answer():
    rng = np.random.default_rng(7)
    seq, d_head, theta = 33, 128, 5e6
    pos3 = rng.integers(0, 50, size=(3, seq)).astype(np.int64)
    inv = (1.0 / (theta ** (np.arange(0, d_head, 2, dtype=np.float32) / d_head))).astype(np.float32)
    c, s = port.mrope_cos_sin(pos3, inv, 20, 20)
    rc, rs = np_mrope_cos_sin(pos3, theta, d_head, 20, 20)
    np.testing.assert_allclose(c, rc, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(s, rs, rtol=1e-5, atol=1e-6)


def test_rope_thd_reductions():
    rng = np.random.default_rng(10)
    rows, heads, dim = 7, 3, 128
    x = rng.standard_normal((rows, heads, dim)).astype(np.float32)
    inv = port.rope_inv_freq(1e6, dim)
    p = rng.integers(0, 8192, rows).astype(np.int64)
    same = np.stack([p, p, p])
    # T = H = W (the decode case): rope_thd is rope with the same frequency table
    np.testing.assert_array_equal(port.rope_thd(x, same, inv, [24, 20, 20]), port.rope(x, p, 1e6))
    # distinct T/H/W: rope_thd is rope_with_cos_sin over the mrope_cos_sin table
    pos3 = rng.integers(0, 4096, (3, rows)).astype(np.int64)
    c, s = port.mrope_cos_sin(pos3, inv, 20, 20)
    np.testing.assert_array_equal(port.rope_thd(x, pos3, inv, [24, 20, 20]), port.rope_with_cos_sin(x, c, s))
    # channel selection: channel 1 follows H, channel 2 follows W, channel 0 and channel 61 (>= 3*20) follow T
    only_t = np.stack([pos3[0], pos3[0], pos3[0]])
    base = port.rope_thd(x, only_t, inv, [24, 20, 20])
    full = port.rope_thd(x, pos3, inv, [24, 20, 20])
    np.testing.assert_array_equal(full[..., 0], base[..., 0])
    np.testing.assert_array_equal(full[..., 60:64], base[..., 60:64])
    assert not np.array_equal(full[..., 1], base[..., 1])
    assert not np.array_equal(full[..., 2], base[..., 2])


def test_rope_with_cos_sin_uses_second_half_of_table():
    x = np.ones((1, 1, 4), np.float32)
    c = np.array([[1, 1, 0, 0]], np.float32)
    s = np.array([[0, 0, 1, 1]], np.float32)
    # first half: a*c[i] - b*s[i] = 1 ; second half: b*c[i+half] + a*s[i+half] = 1
    np.testing.assert_array_equal(port.rope_with_cos_sin(x, c, s), np.array([[[1, 1, 1, 1]]], np.float32))
    s2 = np.array([[1, 1, 0, 0]], np.float32)
    np.testing.assert_array_equal(port.rope_with_cos_sin(x, c, s2), np.array([[[0, 0, 0, 0]]], np.float32))


# ---- linear / byte ops ------------------------------------------------------------------------
def test_linear_against_fp64():
    rng = np.random.default_rng(12)
    x = rng.standard_normal((5, 96)).astype(np.float32)
    w = (0.05 * rng.standard_normal((7, 96))).astype(np.float32)
    b = rng.standard_normal(7).astype(np.float32)
    want = x.astype(np.float64) @ w.astype(np.float64).T
    np.testing.assert_allclose(port.linear(x, w), want, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(port.linear(x, w, b), want + b, rtol=1e-5, atol=1e-6)
    assert port.linear(x, w).shape == (5, 7)  # weight is (out_features, in_features)


def test_concat_and_kv_append_are_byte_copies():
    rng = np.random.default_rng(13)
    a = rng.standard_normal((5, 8, 16)).astype(np.float16)
    b = rng.standard_normal((1, 8, 16)).astype(np.float16)
    np.testing.assert_array_equal(port.concat_axis0(a, b).view(np.uint16), np.concatenate([a, b], 0).view(np.uint16))
    # scatter-append at pos == current length reproduces concat-append
    B, hkv, lmax, d = 3, 2, 9, 16
    kc = rng.standard_normal((B, hkv, lmax, d)).astype(np.float16)
    vc = rng.standard_normal((B, hkv, lmax, d)).astype(np.float16)
    k0, v0 = kc.copy(), vc.copy()
    kn = rng.standard_normal((B, hkv, d)).astype(np.float16)
    vn = rng.standard_normal((B, hkv, d)).astype(np.float16)
    pos = np.array([4, 0, 8], np.int64)
    port.kv_append(kn, vn, kc, vc, pos)
    for i in range(B):
        old = np.transpose(k0[i, :, : pos[i]], (1, 0, 2))
        cat = np.concatenate([old, kn[i][None]], 0)  # (L+1, hkv, d), the reference's append
        np.testing.assert_array_equal(np.transpose(kc[i, :, : pos[i] + 1], (1, 0, 2)).view(np.uint16), cat.view(np.uint16))
        np.testing.assert_array_equal(kc[i, :, pos[i] + 1:].view(np.uint16), k0[i, :, pos[i] + 1:].view(np.uint16))
        np.testing.assert_array_equal(vc[i, :, pos[i]].view(np.uint16), vn[i].view(np.uint16))


def test_argmax_embedding_add():
    rng = np.random.default_rng(14)
    x = rng.standard_normal((4, 1000)).astype(np.float32)
    x[2, 10] = x[2, 500] = 9.0  # ties: the first maximum wins
    np.testing.assert_array_equal(port.argmax(x), np.argmax(x, -1))
    assert port.argmax(x)[2] == 10
    table = rng.standard_normal((10, 4)).astype(np.float32)
    ids = np.array([[1, 3], [5, 2]], np.int64)
    np.testing.assert_array_equal(port.embedding(ids, table), table[ids])
    np.testing.assert_array_equal(port.add(x, x), x + x)


# ---- the restatement against the compiled reference, bit for bit ------------------------------
@needs_ref
@pytest.mark.parametrize("seed", range(12))
def test_port_equals_reference_bitwise_over_random_shapes(seed):
    """Odd sizes, group sizes 1..4, causal and not, more keys than queries and fewer: the restatement and
    the reference's own C++ agree in every bit."""
    rng = np.random.default_rng(7000 + seed)
    hkv = int(rng.integers(1, 4))
    group = int(rng.integers(1, 5))
    d = int(rng.choice([2, 6, 8, 20, 64, 128]))
    sq, skv = int(rng.integers(1, 12)), int(rng.integers(1, 40))
    q = rng.standard_normal((sq, hkv * group, d)).astype(np.float32)
    k = rng.standard_normal((skv, hkv, d)).astype(np.float32)
    v = rng.standard_normal((skv, hkv, d)).astype(np.float32)
    for causal in (False, True):
        np.testing.assert_array_equal(port.sdpa(q, k, v, causal), REF.sdpa(q, k, v, causal))
    rows, hidden = int(rng.integers(1, 9)), int(rng.integers(1, 300))
    x = (3 * rng.standard_normal((rows, hidden))).astype(np.float32)
    r = rng.standard_normal((rows, hidden)).astype(np.float32)
    w = rng.standard_normal(hidden).astype(np.float32)
    eps = float(rng.choice([1e-6, 1e-5, 1e-3]))
    for a, b in zip(port.add_rms_norm(x, r, w, eps), REF.add_rms_norm(x, r, w, eps)):
        np.testing.assert_array_equal(a, b)
    np.testing.assert_array_equal(port.rms_norm(x, w, eps), REF.rms_norm(x, w, eps))
    np.testing.assert_array_equal(port.silu_mul(10 * x, r), REF.silu_mul(10 * x, r))
    heads, dh = int(rng.integers(1, 5)), 2 * int(rng.integers(1, 40))
    xr = rng.standard_normal((rows, heads, dh)).astype(np.float32)
    pos = rng.integers(0, 100000, rows).astype(np.int64)
    theta = float(rng.choice([1e4, 1e6, 5e6]))
    np.testing.assert_array_equal(port.rope(xr, pos, theta), REF.rope(xr, pos, theta))
    inv = port.rope_inv_freq(theta, dh)
    pos3 = rng.integers(0, 100000, (3, rows)).astype(np.int64)
    half = dh // 2
    h_sec, w_sec = int(rng.integers(0, half // 3 + 1)), int(rng.integers(0, half // 3 + 1))
    sec = [half - h_sec - w_sec, h_sec, w_sec]
    np.testing.assert_array_equal(port.rope_thd(xr, pos3, inv, sec), REF.rope_thd(xr, pos3, inv, sec))
    c, s_ = REF.mrope_cos_sin(pos3, inv, h_sec, w_sec)
    for a, b in zip(port.mrope_cos_sin(pos3, inv, h_sec, w_sec), (c, s_)):
        np.testing.assert_array_equal(a, b)
    np.testing.assert_array_equal(port.rope_with_cos_sin(xr, c, s_), REF.rope_with_cos_sin(xr, c, s_))
    m, kk, n = int(rng.integers(1, 20)), int(rng.integers(1, 70)), int(rng.integers(1, 30))
    xl = rng.standard_normal((m, kk)).astype(np.float32)
    wl = rng.standard_normal((n, kk)).astype(np.float32)
    bl = rng.standard_normal(n).astype(np.float32)
    np.testing.assert_array_equal(port.linear(xl, wl, bl), REF.linear(xl, wl, bl))
    np.testing.assert_array_equal(port.linear(xl, wl), REF.linear(xl, wl))


@needs_ref
def test_port_equals_reference_bitwise():
    rng = np.random.default_rng(2024)
    q = rng.standard_normal((1, 16, 128)).astype(np.float32)
    k = rng.standard_normal((1024, 8, 128)).astype(np.float32)
    v = rng.standard_normal((1024, 8, 128)).astype(np.float32)
    np.testing.assert_array_equal(port.sdpa(q, k, v, False), REF.sdpa(q, k, v, False))
    qq = rng.standard_normal((5, 4, 8)).astype(np.float32)
    kk = rng.standard_normal((7, 2, 8)).astype(np.float32)
    vv = rng.standard_normal((7, 2, 8)).astype(np.float32)
    for causal in (False, True):
        np.testing.assert_array_equal(port.sdpa(qq, kk, vv, causal), REF.sdpa(qq, kk, vv, causal))

    x = rng.standard_normal((32, 2048)).astype(np.float32)
    r = rng.standard_normal((32, 2048)).astype(np.float32)
    w = (1 + 0.02 * rng.standard_normal(2048)).astype(np.float32)
    for a, b in zip(port.add_rms_norm(x, r, w, 1e-6), REF.add_rms_norm(x, r, w, 1e-6)):
        np.testing.assert_array_equal(a, b)
    np.testing.assert_array_equal(port.rms_norm(x, w, 1e-6), REF.rms_norm(x, w, 1e-6))
    np.testing.assert_array_equal(port.rms_norm(x, None, 1e-5), REF.rms_norm(x, None, 1e-5))
    g = rng.standard_normal((32, 6144)).astype(np.float32)
    u = rng.standard_normal((32, 6144)).astype(np.float32)
    np.testing.assert_array_equal(port.silu_mul(g, u), REF.silu_mul(g, u))

    xr = rng.standard_normal((32, 16, 128)).astype(np.float32)
    pos = rng.integers(0, 8192, 32).astype(np.int64)
    np.testing.assert_array_equal(port.rope(xr, pos, 1e6), REF.rope(xr, pos, 1e6))
    inv = port.rope_inv_freq(1e6, 128)
    pos3 = rng.integers(0, 8192, (3, 32)).astype(np.int64)
    np.testing.assert_array_equal(port.rope_thd(xr, pos3, inv, [24, 20, 20]), REF.rope_thd(xr, pos3, inv, [24, 20, 20]))
    for a, b in zip(port.mrope_cos_sin(pos3, inv, 20, 20), REF.mrope_cos_sin(pos3, inv, 20, 20)):
        np.testing.assert_array_equal(a, b)
    c, s = REF.mrope_cos_sin(pos3, inv, 20, 20)
    np.testing.assert_array_equal(port.rope_with_cos_sin(xr, c, s), REF.rope_with_cos_sin(xr, c, s))

    xl = rng.standard_normal((16, 256)).astype(np.float32)
    wl = (0.02 * rng.standard_normal((96, 256))).astype(np.float32)
    bl = rng.standard_normal(96).astype(np.float32)
    np.testing.assert_array_equal(port.linear(xl, wl), REF.linear(xl, wl))
    np.testing.assert_array_equal(port.linear(xl, wl, bl), REF.linear(xl, wl, bl))

    a = rng.standard_normal((9, 8, 128)).astype(np.float16)
    b = rng.standard_normal((1, 8, 128)).astype(np.float16)
    np.testing.assert_array_equal(port.concat_axis0(a, b).view(np.uint16), REF.concat_axis0(a, b).view(np.uint16))
    lg = rng.standard_normal((3, 5000)).astype(np.float32)
    np.testing.assert_array_equal(port.argmax(lg), REF.argmax(lg))
    tb = rng.standard_normal((50, 8)).astype(np.float32)
    ids = rng.integers(0, 50, (2, 3)).astype(np.int64)
    np.testing.assert_array_equal(port.embedding(ids, tb), REF.embedding(ids, tb))


@needs_ref
def test_reference_half_helpers_depart_from_ieee():
    """Documents why fp16 data never goes through the reference's CPU conversion helpers:
    Float2Half truncates normals (include/axono/core/half.h:44-49) and Half2Float halves every
    subnormal (:61-69).  The device path, and this build, use IEEE round-to-nearest-even."""
    rng = np.random.default_rng(0)
    x = rng.standard_normal(20000).astype(np.float32)
    ref_bits = oracle.ref_float2half(x)
    ieee_bits = x.astype(np.float16).view(np.uint16)
    assert np.count_nonzero(ref_bits != ieee_bits) > 1000
    assert np.max(np.abs(ref_bits.astype(np.int32) - ieee_bits.astype(np.int32))) <= 1
    np.testing.assert_array_equal(oracle.ref_float2half(np.array([1.0, -0.5, 65504.0, 0.0], np.float32)),
                                  np.array([1.0, -0.5, 65504.0, 0.0], np.float16).view(np.uint16))
    sub = np.arange(1, 0x400, dtype=np.uint16)
    np.testing.assert_array_equal(oracle.ref_half2float(sub) * 2, sub.view(np.float16).astype(np.float32))
    normal = np.arange(0x400, 0x7C00, dtype=np.uint16)
    np.testing.assert_array_equal(oracle.ref_half2float(normal), normal.view(np.float16).astype(np.float32))
