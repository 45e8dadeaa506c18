"""Fused / row-wise / rotary / cache-append kernels on the GPU against the CPU oracle.

Tolerances: fp32 max abs error <= 1e-5.  fp16 (fp32 oracle on fp16-rounded inputs): the kernel rounds once at
the store, so the bound is half an fp16 ulp of the value plus the operator's own fp32 disagreement term
(assert_fp16_close; always inside the stated 2e-3 for |value| < 4, and above it only where half an ulp alone is);
attention keeps 2e-3 absolute.  Byte movers are bit exact.
"""
import os

import numpy as np
import pytest

from oracle import port

import gpu_util as gu

pytestmark = pytest.mark.gpu

TOL32, TOL16 = 1e-5, 2e-3
G = np.load(os.path.join(os.path.dirname(__file__), "golden", "decode_path_golden.npz"))


def h16(a):
    return np.asarray(a, np.float32).astype(np.float16)


def assert_fp16_close(got, want, rel=0.0, abs_=0.0):
    """The device rounds its fp32 result once to fp16, so against the oracle's fp32 value it may be off by half an
    fp16 ulp plus however far the two fp32 values can be apart before that rounding: `rel` * |want| + `abs_`, stated
    per operator by the caller (nothing for a sum of two fp16 values, which is exact in fp32)."""
    got = got.astype(np.float32)
    err = np.abs(got - want)
    ulp = np.spacing(np.abs(want).astype(np.float16)).astype(np.float32)
    bound = 0.5 * ulp + rel * np.abs(want) + abs_
    assert np.all(err <= bound), (float(err.max()), float((err - bound).max()), float(np.abs(want).max()))


def norm_terms(hidden):
    """fp32 disagreement of an RMSNorm output: the sum of squares in another order (<= 4 sqrt(H) 2^-24 relative, the
    bound the Linear tests use for a reordered sum) and three more roundings (rsqrt, two products)."""
    return dict(rel=(4 * np.sqrt(hidden) + 4) * 2.0 ** -24, abs_=1e-7)


# silu(g) * u in fp32: the exponential's argument is rounded once more on the device (exp2 of a product), the
# exponential and the reciprocal are each good to an ulp: a few 2^-24 relative
SILU = dict(rel=4e-6, abs_=1e-7)
# rotation by an angle formed in fp32 exactly as the oracle forms it; accurate sine / cosine on both sides
# (<= 2 ulp each) and two products + one sum: the fp32 bar of the same operator
ROPE = dict(abs_=TOL32)


def assert_fp16_attention(got, want):
    """Attention in fp16 keeps the stated bar of 2e-3 absolute: on the matrix-core route the probabilities are
    themselves rounded to fp16 before the second product, which is not a reduction-order effect."""
    err = np.abs(got.astype(np.float32) - want)
    assert np.all(err <= TOL16), float(err.max())


# ---- config 1 (fp32 op check) and golden fixtures ---------------------------------------------
def test_add_rms_norm_fp32_config1():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((1, 2048)).astype(np.float32)
    r = rng.standard_normal((1, 2048)).astype(np.float32)
    w = (1 + 0.02 * rng.standard_normal(2048)).astype(np.float32)
    y, out = gu.add_rms_norm(x, r, w, 1e-6)
    wy, wout = port.add_rms_norm(x, r, w, 1e-6)
    np.testing.assert_array_equal(y, wy)  # a single fp32 add
    np.testing.assert_allclose(out, wout, rtol=0, atol=TOL32)


def test_golden_fused_and_rotary_fp32():
    y, out = gu.add_rms_norm(G["arn_x"], G["arn_res"], G["arn_w"], 1e-6)
    np.testing.assert_array_equal(y, G["arn_y"])
    np.testing.assert_allclose(out, G["arn_out"], rtol=0, atol=TOL32)
    np.testing.assert_allclose(gu.rms_norm(G["arn_x"], G["arn_w"], 1e-6), G["rms_out"], rtol=0, atol=TOL32)
    s = gu.silu_mul(G["silu_gate"], G["silu_up"])
    np.testing.assert_allclose(s, G["silu_out"], rtol=2e-6, atol=TOL32)
    x, pos = G["rope_x"], G["rope_pos"]
    np.testing.assert_allclose(gu.rope(x, pos, 1e6), G["rope_out_theta1e6"], rtol=0, atol=TOL32)
    np.testing.assert_allclose(gu.rope(x, pos, 1e4), G["rope_out_theta1e4"], rtol=0, atol=TOL32)
    inv, pos3 = G["mrope_inv_freq"], G["mrope_pos3"]
    np.testing.assert_allclose(gu.rope_thd(x, pos3, inv, [24, 20, 20]), G["rope_thd_out"], rtol=0, atol=TOL32)
    c, s_ = gu.mrope_cos_sin(pos3, inv, 20, 20)
    np.testing.assert_allclose(c, G["mrope_cos"], rtol=0, atol=TOL32)
    np.testing.assert_allclose(s_, G["mrope_sin"], rtol=0, atol=TOL32)
    np.testing.assert_allclose(gu.rope_with_cos_sin(x, G["mrope_cos"], G["mrope_sin"]), G["rope_cos_sin_out"], rtol=0, atol=TOL32)


def test_reference_test_shapes_fp32():
    """Shapes of the reference's own fused tests: 37x53 silu_mul (odd size), 4x128 and 2x64 norms."""
    rs = np.random.RandomState(0)
    g = rs.randn(37, 53).astype(np.float32)
    u = rs.randn(37, 53).astype(np.float32)
    np.testing.assert_allclose(gu.silu_mul(g, u), port.silu_mul(g, u), rtol=2e-6, atol=1e-6)
    rs = np.random.RandomState(1)
    x = rs.randn(4, 128).astype(np.float32)
    r = rs.randn(4, 128).astype(np.float32)
    w = rs.randn(128).astype(np.float32)
    y, out = gu.add_rms_norm(x, r, w, 1e-6)
    wy, wout = port.add_rms_norm(x, r, w, 1e-6)
    np.testing.assert_array_equal(y, wy)
    np.testing.assert_allclose(out, wout, rtol=0, atol=TOL32)
    # rows that are not a multiple of 16 bytes take the element-wise path
    x = rs.randn(5, 53).astype(np.float32)
    w = rs.randn(53).astype(np.float32)
    np.testing.assert_allclose(gu.rms_norm(x, w, 1e-5), port.rms_norm(x, w, 1e-5), rtol=0, atol=TOL32)
    np.testing.assert_allclose(gu.rms_norm(x, None, 1e-5), port.rms_norm(x, None, 1e-5), rtol=0, atol=TOL32)


# ---- config 2 (fp16, B = 32) -------------------------------------------------------------------
def test_add_rms_norm_fp16_config2():
    rng = np.random.default_rng(20)
    x, r = h16(rng.standard_normal((32, 2048))), h16(rng.standard_normal((32, 2048)))
    w32 = (1 + 0.02 * rng.standard_normal(2048)).astype(np.float32)
    wy, wout = port.add_rms_norm(x, r, h16(w32), 1e-6)
    for w in (h16(w32),):
        y, out = gu.add_rms_norm(x, r, w, 1e-6)
        np.testing.assert_array_equal(y.view(np.uint16), wy.astype(np.float16).view(np.uint16))  # one rounding of an exact-in-fp32 sum
        assert_fp16_close(out, wout, **norm_terms(2048))
    # fp32 weights with fp16 activations
    wy, wout = port.add_rms_norm(x, r, w32, 1e-6)
    y, out = gu.add_rms_norm(x, r, w32, 1e-6)
    assert_fp16_close(out, wout, **norm_terms(2048))


def test_silu_mul_fp16_config2():
    rng = np.random.default_rng(21)
    g, u = h16(rng.standard_normal((32, 6144))), h16(rng.standard_normal((32, 6144)))
    assert_fp16_close(gu.silu_mul(g, u), port.silu_mul(g, u), **SILU)


@pytest.mark.parametrize("n", [8 * (1024 * 3 + 700) + 5, 8 * 1024 * 2, 8 * 1023 + 7, 3])
def test_elementwise_whole_and_partial_passes(n):
    """silu_mul and add over sizes that end in a partial pass of the four-groups-per-thread loop and in
    a scalar tail; the large fp16 case takes the streaming form (three arrays beyond the memory-side cache)."""
    rng = np.random.default_rng(n % 1000)
    g, u = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    np.testing.assert_allclose(gu.silu_mul(g, u), port.silu_mul(g, u), rtol=2e-6, atol=1e-6)
    np.testing.assert_array_equal(gu.add(g, u), g + u)
    assert_fp16_close(gu.silu_mul(h16(g), h16(u)), port.silu_mul(h16(g).astype(np.float32), h16(u).astype(np.float32)), **SILU)


def test_elementwise_streaming_form():
    n = 48 * 1024 * 1024 + 8 * 300 + 3  # 3 x 96 MB of fp16: past the cache threshold
    rng = np.random.default_rng(77)
    blk = rng.standard_normal(1 << 20).astype(np.float16)
    g = np.resize(blk, n)
    u = np.resize(blk[::-1], n)
    got = gu.add(g, u)
    np.testing.assert_array_equal(got, (g.astype(np.float32) + u.astype(np.float32)).astype(np.float16))
    got = gu.silu_mul(g[: n // 2], u[: n // 2])  # below the threshold: the plain form on the same data
    got2 = gu.silu_mul(g, u)[: n // 2]
    np.testing.assert_array_equal(got, got2)


def test_rope_fp16_config2():
    rng = np.random.default_rng(22)
    pos = rng.integers(0, 8192, 32).astype(np.int64)
    for heads in (16, 8):
        x = h16(rng.standard_normal((32, heads, 128)))
        assert_fp16_close(gu.rope(x, pos, 1e6), port.rope(x, pos, 1e6), **ROPE)
    # fp32 at the same positions: the fp32 angle products are formed exactly as on the CPU
    x = rng.standard_normal((32, 16, 128)).astype(np.float32)
    np.testing.assert_allclose(gu.rope(x, pos, 1e6), port.rope(x, pos, 1e6), rtol=0, atol=TOL32)


@pytest.mark.parametrize("rows,hq,hk,dim", [(32, 16, 8, 128), (4099, 16, 8, 128), (7, 3, 5, 64), (130, 4, 2, 96),
                                            (9, 2, 1, 512), (5, 2, 2, 8)])
def test_rope_q_and_k_in_one_launch(rows, hq, hk, dim):
    """axhip_rope_qk: the q and k heads of the same rows in one launch, bit-identical to two axhip_rope
    calls and within tolerance of the oracle; fp16 and fp32; row counts that leave the last workgroup
    partly empty; head sizes of 64 / 96 / 512 and one (8) that takes the general kernel."""
    rng = np.random.default_rng(rows + dim)
    pos = rng.integers(0, 8192, rows).astype(np.int64)
    for dtype in (np.float16, np.float32):
        q = rng.standard_normal((rows, hq, dim)).astype(np.float32).astype(dtype)
        k = rng.standard_normal((rows, hk, dim)).astype(np.float32).astype(dtype)
        gq, gk = gu.rope_qk(q, k, pos, 1e6)
        bits = np.uint16 if dtype == np.float16 else np.uint32
        np.testing.assert_array_equal(gq.view(bits), gu.rope(q, pos, 1e6).view(bits))
        np.testing.assert_array_equal(gk.view(bits), gu.rope(k, pos, 1e6).view(bits))
        if dtype == np.float16:
            assert_fp16_close(gq, port.rope(q, pos, 1e6), **ROPE)
            assert_fp16_close(gk, port.rope(k, pos, 1e6), **ROPE)
        else:
            np.testing.assert_allclose(gq, port.rope(q, pos, 1e6), rtol=0, atol=TOL32)
            np.testing.assert_allclose(gk, port.rope(k, pos, 1e6), rtol=0, atol=TOL32)
    l = gu.lib()
    assert l.axhip_rope_qk(None, None, None, 1e6, None, None, 5, 4, 2, 1, 7, None) == 1    # odd dim
    assert l.axhip_rope_qk(None, None, None, 1e6, None, None, 5, 4, 2, 1, 8, None) == 7    # null pointers
    assert l.axhip_rope_qk(None, None, None, 1e6, None, None, 5, 0, 2, 1, 8, None) == 0    # no rows
    assert l.axhip_rope_qk(None, None, None, 1e6, None, None, 2, 4, 2, 1, 8, None) == 3    # INT32 data


def test_mrope_family():
    rng = np.random.default_rng(23)
    rows = 33
    inv = port.rope_inv_freq(1e6, 128)
    pos3 = rng.integers(0, 8192, (3, rows)).astype(np.int64)
    x = rng.standard_normal((rows, 4, 128)).astype(np.float32)
    np.testing.assert_allclose(gu.rope_thd(x, pos3, inv, [24, 20, 20]), port.rope_thd(x, pos3, inv, [24, 20, 20]), rtol=0, atol=TOL32)
    assert_fp16_close(gu.rope_thd(h16(x), pos3, inv, [24, 20, 20]), port.rope_thd(h16(x), pos3, inv, [24, 20, 20]), **ROPE)
    c, s = gu.mrope_cos_sin(pos3, inv, 20, 20)
    wc, ws = port.mrope_cos_sin(pos3, inv, 20, 20)
    np.testing.assert_allclose(c, wc, rtol=0, atol=TOL32)
    np.testing.assert_allclose(s, ws, rtol=0, atol=TOL32)
    np.testing.assert_allclose(gu.rope_with_cos_sin(x, wc, ws), port.rope_with_cos_sin(x, wc, ws), rtol=0, atol=TOL32)
    # decode case T = H = W: rope_thd equals rope
    p = pos3[0]
    np.testing.assert_allclose(gu.rope_thd(x, np.stack([p, p, p]), inv, [24, 20, 20]), port.rope(x, p, 1e6), rtol=0, atol=TOL32)
    # small head (the reference's rope test shape 4x2x8, theta 1e4)
    xs = rng.standard_normal((4, 2, 8)).astype(np.float32)
    np.testing.assert_allclose(gu.rope(xs, np.arange(4), 1e4), port.rope(xs, np.arange(4), 1e4), rtol=0, atol=TOL32)


def test_rope_many_rows_shares_angles_across_heads():
    """Prefill-sized inputs, where one thread rotates several heads of a row with one set of angles
    (2, 4 or 8 heads per thread depending on the row count): all three rope forms, fp16 and fp32,
    a head count that is not a power of two, and bit-equality with the one-head-per-thread result."""
    rng = np.random.default_rng(29)
    inv = port.rope_inv_freq(1e6, 128)
    for rows, heads in ((4096, 16), (16384, 16), (8192, 12), (16384, 8)):
        pos = rng.integers(0, 32768, rows).astype(np.int64)
        x = h16(rng.standard_normal((rows, heads, 128)))
        got = gu.rope(x, pos, 1e6)
        assert_fp16_close(got, port.rope(x, pos, 1e6), **ROPE)
        # the same rows in slices small enough for one head per thread
        part = np.concatenate([gu.rope(x[i:i + 256], pos[i:i + 256], 1e6) for i in range(0, 1024, 256)])
        np.testing.assert_array_equal(got[:1024].view(np.uint16), part.view(np.uint16))
    rows, heads = 8192, 16
    pos3 = rng.integers(0, 8192, (3, rows)).astype(np.int64)
    x = rng.standard_normal((rows, heads, 128)).astype(np.float32)
    np.testing.assert_allclose(gu.rope_thd(x, pos3, inv, [24, 20, 20]), port.rope_thd(x, pos3, inv, [24, 20, 20]), rtol=0, atol=TOL32)
    wc, ws = port.mrope_cos_sin(pos3, inv, 20, 20)
    np.testing.assert_allclose(gu.rope_with_cos_sin(x, wc, ws), port.rope_with_cos_sin(x, wc, ws), rtol=0, atol=TOL32)


def test_kv_append_bit_exact_config2():
    rng = np.random.default_rng(24)
    B, Hkv, Lmax, D = 32, 8, 8192, 128
    kc = rng.integers(0, 65536, (B, Hkv, Lmax, D), dtype=np.uint16).view(np.float16)
    vc = rng.integers(0, 65536, (B, Hkv, Lmax, D), dtype=np.uint16).view(np.float16)
    kn = rng.integers(0, 65536, (B, Hkv, D), dtype=np.uint16).view(np.float16)  # all bit patterns incl. NaNs
    vn = rng.integers(0, 65536, (B, Hkv, D), dtype=np.uint16).view(np.float16)
    pos = rng.integers(0, Lmax, B).astype(np.int64)
    pos[0], pos[1] = 0, Lmax - 1
    gk, gv = gu.kv_append(kn, vn, kc, vc, pos)
    port.kv_append(kn, vn, kc, vc, pos)  # in place on the host copies
    np.testing.assert_array_equal(gk.view(np.uint16), kc.view(np.uint16))  # incl. every untouched byte
    np.testing.assert_array_equal(gv.view(np.uint16), vc.view(np.uint16))


def test_kv_append_int32_pos_fp32_and_out_of_range():
    rng = np.random.default_rng(25)
    B, Hkv, Lmax, D = 3, 2, 16, 64
    kc = rng.standard_normal((B, Hkv, Lmax, D)).astype(np.float32)
    vc = rng.standard_normal((B, Hkv, Lmax, D)).astype(np.float32)
    kn = rng.standard_normal((B, Hkv, D)).astype(np.float32)
    vn = rng.standard_normal((B, Hkv, D)).astype(np.float32)
    pos = np.array([5, 16, -1], np.int32)  # the last two are outside [0,Lmax): skipped
    gk, gv = gu.kv_append(kn, vn, kc, vc, pos)
    wk, wv = kc.copy(), vc.copy()
    wk[0, :, 5], wv[0, :, 5] = kn[0], vn[0]
    np.testing.assert_array_equal(gk, wk)
    np.testing.assert_array_equal(gv, wv)


def test_concat_append_matches_reference_semantics():
    rng = np.random.default_rng(26)
    a = h16(rng.standard_normal((300, 8, 128)))
    b = h16(rng.standard_normal((1, 8, 128)))
    np.testing.assert_array_equal(gu.concat_axis0(a, b).view(np.uint16), port.concat_axis0(a, b).view(np.uint16))
    a8 = rng.integers(0, 255, (7, 3), dtype=np.uint8).view(np.int8)  # unaligned sizes
    b8 = rng.integers(0, 255, (2, 3), dtype=np.uint8).view(np.int8)
    da, db = gu.dev(a8), gu.dev(b8)
    do = gu.DeviceBuffer(27)
    gu._run("axhip_concat", da.ptr, db.ptr, do.ptr, 1, 21, 6, None)
    gu.synchronize()
    np.testing.assert_array_equal(do.download(np.int8, (9, 3)), np.concatenate([a8, b8]))


def test_cast_add_embedding_argmax():
    rng = np.random.default_rng(27)
    x = rng.standard_normal(100003).astype(np.float32) * 10
    np.testing.assert_array_equal(gu.cast(x, np.float16).view(np.uint16), x.astype(np.float16).view(np.uint16))  # IEEE RNE
    np.testing.assert_array_equal(gu.cast(np.array([1.0, -0.5, 65504.0, 0.0, 1e-7, 70000.0], np.float32), np.float16).view(np.uint16),
                                  np.array([1.0, -0.5, 65504.0, 0.0, 1e-7, 70000.0], np.float32).astype(np.float16).view(np.uint16))
    hb = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16)  # every finite non-negative half, subnormals too
    np.testing.assert_array_equal(gu.cast(hb, np.float32), hb.astype(np.float32))
    a, b = rng.standard_normal((16, 2048)).astype(np.float32), rng.standard_normal((16, 2048)).astype(np.float32)
    np.testing.assert_array_equal(gu.add(a, b), a + b)
    np.testing.assert_array_equal(gu.add(h16(a), h16(b)).view(np.uint16), (h16(a).astype(np.float32) + h16(b).astype(np.float32)).astype(np.float16).view(np.uint16))
    table = h16(rng.standard_normal((1000, 2048)))
    ids = rng.integers(0, 1000, (16, 1)).astype(np.int64)
    np.testing.assert_array_equal(gu.embedding(ids, table).view(np.uint16), table[ids].view(np.uint16))
    t32 = rng.standard_normal((10, 4)).astype(np.float32)
    ids2 = np.array([[1, 3], [5, 2]], np.int64)
    np.testing.assert_array_equal(gu.embedding(ids2, t32), port.embedding(ids2, t32))
    lg = rng.standard_normal((16, 151936)).astype(np.float32)
    lg[3, 777] = lg[3, 150000] = 50.0  # tie: first index wins
    np.testing.assert_array_equal(gu.argmax(lg), port.argmax(lg))
    assert gu.argmax(lg)[3] == 777
    np.testing.assert_array_equal(gu.argmax(h16(lg)), port.argmax(h16(lg).astype(np.float32)))
    # many ties (values from a small set): the first index wins inside a 16-byte group, inside a thread, across
    # threads and across the 64 parts of a row; row lengths that are and are not a multiple of 8
    for cols in (151936, 20000, 16387, 100003):
        t = rng.integers(0, 5, (5, cols)).astype(np.float32)
        t[1, -1] = 9.0            # the maximum in the last element
        t[2, cols // 2 + 3] = 9.0
        t[2, cols - 2] = 9.0
        t[3, :] = -np.inf         # nothing compares greater: index 0
        np.testing.assert_array_equal(gu.argmax(t), port.argmax(t))
        np.testing.assert_array_equal(gu.argmax(h16(t)), port.argmax(t))
    # more rows than the 32 whose ticket counters take a cache line each (row 32 takes the word next to row 0's),
    # twice in a row: the counters are back at zero after a launch
    t = rng.standard_normal((70, 16392)).astype(np.float32)
    for _ in range(2):
        np.testing.assert_array_equal(gu.argmax(t), np.argmax(t, -1))


def test_sdpa_prefill_and_small_heads():
    rng = np.random.default_rng(28)
    q = rng.standard_normal((50, 4, 64)).astype(np.float32)
    k = rng.standard_normal((50, 2, 64)).astype(np.float32)
    v = rng.standard_normal((50, 2, 64)).astype(np.float32)
    for causal in (True, False):
        np.testing.assert_allclose(gu.sdpa(q, k, v, causal), port.sdpa(q, k, v, causal), rtol=0, atol=TOL32)
    np.testing.assert_allclose(gu.sdpa(G["sdpa_q"], G["sdpa_k"], G["sdpa_v"], True), G["sdpa_causal_out"], rtol=0, atol=TOL32)
    np.testing.assert_allclose(gu.sdpa(G["sdpa_q"], G["sdpa_k"], G["sdpa_v"], False), G["sdpa_full_out"], rtol=0, atol=TOL32)
    # decode-with-cache equals causal full forward (tests/nn/test_kv_cache.py:120-148 of the reference)
    full = gu.sdpa(q, k, v, True)
    for t in (0, 17, 49):
        step = gu.sdpa(q[t:t + 1], k[:t + 1], v[:t + 1], False)
        np.testing.assert_allclose(step[0], full[t], rtol=0, atol=TOL32)


@pytest.mark.parametrize("Sq,Skv,Hq,Hkv,D", [
    (300, 300, 8, 2, 128),    # four heads per kv head, ragged last tile of queries
    (128, 333, 4, 2, 64),     # more keys than queries
    (260, 100, 6, 2, 128),    # fewer keys than queries: late rows see every key; three heads per kv head
    (32, 1000, 2, 2, 64),     # the fewest query rows this kernel takes
])
def test_sdpa_fp16_on_the_matrix_cores(Sq, Skv, Hq, Hkv, D):
    """fp16 attention with 32 or more query rows runs the tiled MFMA kernel over token-major K/V."""
    rng = np.random.default_rng(Sq + Skv)
    q = h16(rng.standard_normal((Sq, Hq, D)))
    k = h16(rng.standard_normal((Skv, Hkv, D)))
    v = h16(rng.standard_normal((Skv, Hkv, D)))
    f = lambda a: a.astype(np.float32)
    for causal in (True, False):
        assert_fp16_attention(gu.sdpa(q, k, v, causal), port.sdpa(f(q), f(k), f(v), causal))


def test_fp16_output_variants_round_once():
    """Norm / SiLU-mul results stored as fp16 from fp32 inputs equal the fp32 result rounded once."""
    rng = np.random.default_rng(30)
    x = rng.standard_normal((16, 2048)).astype(np.float32)
    r = rng.standard_normal((16, 2048)).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(2048)).astype(np.float32)
    dx, dr, dw = gu.dev(x), gu.dev(r), gu.dev(w)
    dy, do = gu.DeviceBuffer(x.nbytes), gu.DeviceBuffer(x.size * 2)
    gu._run("axhip_add_rms_norm_ex", dx.ptr, dr.ptr, dw.ptr, 1e-6, dy.ptr, do.ptr, gu.F32, gu.F32, gu.F16, 16, 2048, None)
    gu.synchronize()
    y32, o32 = gu.add_rms_norm(x, r, w, 1e-6)
    np.testing.assert_array_equal(dy.download(np.float32, x.shape), y32)
    np.testing.assert_array_equal(do.download(np.float16, x.shape).view(np.uint16), o32.astype(np.float16).view(np.uint16))
    do2 = gu.DeviceBuffer(x.size * 2)
    gu._run("axhip_rms_norm_ex", dx.ptr, dw.ptr, 1e-6, do2.ptr, gu.F32, gu.F32, gu.F16, 16, 2048, None)
    gu.synchronize()
    np.testing.assert_array_equal(do2.download(np.float16, x.shape).view(np.uint16),
                                  gu.rms_norm(x, w, 1e-6).astype(np.float16).view(np.uint16))
    g_u = rng.standard_normal((16, 2 * 6144)).astype(np.float32)
    dg = gu.dev(g_u)
    o_f32, o_f16 = gu.DeviceBuffer(16 * 6144 * 4), gu.DeviceBuffer(16 * 6144 * 2)
    gu._run("axhip_silu_mul_fused", dg.ptr, o_f32.ptr, gu.F32, gu.F32, 16, 6144, None)
    gu._run("axhip_silu_mul_fused", dg.ptr, o_f16.ptr, gu.F32, gu.F16, 16, 6144, None)
    gu.synchronize()
    want = port.silu_mul(np.ascontiguousarray(g_u[:, :6144]), np.ascontiguousarray(g_u[:, 6144:]))
    got32 = o_f32.download(np.float32, (16, 6144))
    np.testing.assert_allclose(got32, want, rtol=2e-6, atol=1e-6)
    np.testing.assert_array_equal(o_f16.download(np.float16, (16, 6144)).view(np.uint16), got32.astype(np.float16).view(np.uint16))
    assert gu.lib().axhip_silu_mul_fused(dg.ptr, o_f32.ptr, gu.F16, gu.F32, 16, 6144, None) == 3  # fp16 in, fp32 out: refused


@pytest.mark.parametrize("B,S,nq,nkv,lmax,lens", [(3, 2, 4, 2, 16, [5, 0, 13]),
                                                   (1, 4096, 4, 2, 4100, [3]),      # two heads per wavefront
                                                   (2, 8192, 5, 1, 8200, [0, 8])])  # q, k and v heads in one wavefront
def test_qkv_norm_rope_append_equals_op_composition(B, S, nq, nkv, lmax, lens):
    """The fused glue against rms_norm -> rope_thd -> round to fp16 -> append of the oracle; with many
    tokens a wavefront takes several heads of a token with one set of rotation angles."""
    rng = np.random.default_rng(31)
    D = 128
    T = B * S
    width = (nq + 2 * nkv) * D
    qkv = rng.standard_normal((T, width)).astype(np.float32)
    qw = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    kw = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    pos = rng.integers(0, 8192, (3, T)).astype(np.int64)
    inv = port.rope_inv_freq(1e6, D)
    lens = np.array(lens, np.int32)
    kc = rng.standard_normal((B, nkv, lmax, D)).astype(np.float16)
    vc = rng.standard_normal((B, nkv, lmax, D)).astype(np.float16)
    dq, dqw, dkw, dp, di, dl, dkc, dvc = (gu.dev(a) for a in (qkv, qw, kw, pos, inv, lens, kc, vc))
    qo = gu.DeviceBuffer(T * nq * D * 2)
    gu._run("axhip_qkv_norm_rope_append", dq.ptr, width, dq.ptr + nq * D * 4, width, dq.ptr + (nq + nkv) * D * 4, width,
            dqw.ptr, dkw.ptr, gu.F32, 1e-6, dp.ptr, di.ptr, 20, 20, dl.ptr, qo.ptr, dkc.ptr, dvc.ptr, gu.F16,
            B, S, nq, nkv, D, lmax, None)
    gu.synchronize()
    q = port.rope_thd(port.rms_norm(qkv[:, : nq * D].reshape(T, nq, D), qw, 1e-6), pos, inv, [24, 20, 20])
    k = port.rope_thd(port.rms_norm(qkv[:, nq * D:(nq + nkv) * D].reshape(T, nkv, D), kw, 1e-6), pos, inv, [24, 20, 20])
    v = qkv[:, (nq + nkv) * D:].reshape(T, nkv, D)
    got_q = qo.download(np.float16, (T, nq, D)).astype(np.float32)
    assert np.abs(got_q - q).max() <= 2e-3
    wk, wv = kc.copy(), vc.copy()
    for t in range(T):
        b, off = t // S, t % S
        wk[b, :, lens[b] + off] = k[t].astype(np.float16)
        wv[b, :, lens[b] + off] = v[t].astype(np.float16)
    gk, gv = dkc.download(np.float16, kc.shape), dvc.download(np.float16, vc.shape)
    np.testing.assert_array_equal(gv.view(np.uint16), wv.view(np.uint16))  # v: one exact rounding
    assert np.abs(gk.astype(np.float32) - wk.astype(np.float32)).max() <= 2e-3
    touched = np.zeros(kc.shape, bool)
    for t in range(T):
        touched[t // S, :, lens[t // S] + t % S] = True
    np.testing.assert_array_equal(gk[~touched].view(np.uint16), kc[~touched].view(np.uint16))  # other rows untouched


def test_index_add():
    a32 = np.array([5, 0, -3], np.int32)
    a64 = np.arange(6, dtype=np.int64).reshape(3, 2) * 1000
    d32, d64 = gu.dev(a32), gu.dev(a64)
    gu._run("axhip_index_add", d32.ptr, gu.I32, 3, 1, None)
    gu._run("axhip_index_add", d64.ptr, gu.I64, 6, 7, None)
    gu.synchronize()
    np.testing.assert_array_equal(d32.download(np.int32, (3,)), a32 + 1)
    np.testing.assert_array_equal(d64.download(np.int64, (3, 2)), a64 + 7)


def test_embedding_rms_norm_equals_the_three_operators():
    """One launch for embedding -> cast to fp32 -> rms_norm (fp16 out): same bits as the three operators."""
    rng = np.random.default_rng(41)
    vocab, dim, n = 1000, 2048, 16
    table = h16(rng.standard_normal((vocab, dim)))
    ids = rng.integers(0, vocab, n).astype(np.int64)
    ids[3] = vocab + 5      # out of range: a zero row, as the gather alone gives
    l = gu.lib()
    for wdt in (np.float32, np.float16):
        w = (1 + 0.1 * rng.standard_normal(dim)).astype(wdt)
        di, dtb, dw = gu.dev(ids), gu.dev(table), gu.dev(w)
        dh, dxn = gu.DeviceBuffer(n * dim * 4), gu.DeviceBuffer(n * dim * 2)
        gu._run("axhip_embedding_rms_norm", di.ptr, gu.I64, dtb.ptr, dw.ptr, gu.dt(w), 1e-6, dh.ptr, dxn.ptr, n, vocab, dim, None)
        gu.synchronize()
        h, xn = dh.download(np.float32, (n, dim)), dxn.download(np.float16, (n, dim))
        rows = table[np.clip(ids, 0, vocab - 1)].astype(np.float32)
        rows[3] = 0
        np.testing.assert_array_equal(h, rows)
        # the separate operators on the device
        e = gu.embedding(ids.reshape(n, 1), table).reshape(n, dim)
        dh2, dxn2 = gu.dev(gu.cast(e, np.float32)), gu.DeviceBuffer(n * dim * 2)
        gu._run("axhip_rms_norm_ex", dh2.ptr, dw.ptr, 1e-6, dxn2.ptr, gu.F32, gu.dt(w), gu.F16, n, dim, None)
        gu.synchronize()
        np.testing.assert_array_equal(xn.view(np.uint16), dxn2.download(np.float16, (n, dim)).view(np.uint16))
        # and the oracle
        want = port.rms_norm(rows, w.astype(np.float32), 1e-6)
        assert_fp16_close(xn, want, **norm_terms(dim))
    # int32 ids; argument checks
    di32 = gu.dev(ids.astype(np.int32))
    gu._run("axhip_embedding_rms_norm", di32.ptr, gu.I32, dtb.ptr, dw.ptr, gu.dt(w), 1e-6, dh.ptr, dxn.ptr, n, vocab, dim, None)
    gu.synchronize()
    np.testing.assert_array_equal(dh.download(np.float32, (n, dim)), rows)
    assert l.axhip_embedding_rms_norm(di.ptr, gu.I64, dtb.ptr, dw.ptr, gu.dt(w), 1e-6, dh.ptr, dxn.ptr, n, vocab, 2044, None) == 1
    assert l.axhip_embedding_rms_norm(di.ptr, gu.F32, dtb.ptr, dw.ptr, gu.dt(w), 1e-6, dh.ptr, dxn.ptr, n, vocab, dim, None) == 3
    assert l.axhip_embedding_rms_norm(di.ptr, gu.I64, None, dw.ptr, gu.dt(w), 1e-6, dh.ptr, dxn.ptr, n, vocab, dim, None) == 7


def test_decode_advance():
    """ids <- next ids, positions and lengths + 1, token log at the device-side counter; several steps,
    a log shorter than the number of steps, optional outputs left out."""
    rng = np.random.default_rng(42)
    l = gu.lib()
    for B in (1, 16, 700):
        ids = rng.integers(0, 1000, B).astype(np.int64)
        pos = rng.integers(0, 8192, (3, B)).astype(np.int64)
        lens = rng.integers(0, 4096, B).astype(np.int32)
        log_rows = 3
        d_ids, d_pos, d_lens = gu.dev(ids), gu.dev(pos), gu.dev(lens)
        d_log, d_cnt = gu.dev(np.full((log_rows, B), -1, np.int64)), gu.dev(np.zeros(1, np.int64))
        want_log = np.full((log_rows, B), -1, np.int64)
        for step in range(5):
            nxt = rng.integers(0, 1000, B).astype(np.int64)
            d_nxt = gu.dev(nxt)
            gu._run("axhip_decode_advance", d_nxt.ptr, d_ids.ptr, d_pos.ptr, 3, d_lens.ptr, d_log.ptr, log_rows, d_cnt.ptr, B, None)
            gu.synchronize()
            if step < log_rows:
                want_log[step] = nxt
            np.testing.assert_array_equal(d_ids.download(np.int64, (B,)), nxt)
            np.testing.assert_array_equal(d_pos.download(np.int64, (3, B)), pos + step + 1)
            np.testing.assert_array_equal(d_lens.download(np.int32, (B,)), lens + step + 1)
            np.testing.assert_array_equal(d_log.download(np.int64, (log_rows, B)), want_log)
            assert d_cnt.download(np.int64, (1,))[0] == step + 1
        # only the ids
        gu._run("axhip_decode_advance", d_nxt.ptr, d_ids.ptr, None, 0, None, None, 0, None, B, None)
        gu.synchronize()
        np.testing.assert_array_equal(d_lens.download(np.int32, (B,)), lens + 5)
    assert l.axhip_decode_advance(None, d_ids.ptr, None, 0, None, None, 0, None, 4, None) == 7
    assert l.axhip_decode_advance(d_nxt.ptr, d_ids.ptr, None, 3, None, None, 0, None, 4, None) == 7
    assert l.axhip_decode_advance(d_nxt.ptr, d_ids.ptr, None, 0, None, None, 0, None, -1, None) == 1


@pytest.mark.parametrize("seed", range(12))
def test_row_operators_random_shapes(seed):
    """Rows and widths at random (widths that are not multiples of 8 take the scalar paths), fp32 and
    fp16: add_rms_norm, rms_norm, silu_mul, rope, rope_thd and the cos/sin table form."""
    rng = np.random.default_rng(9700 + seed)
    rows = int(rng.integers(1, 70))
    hidden = int(rng.choice([1, 5, 8, 72, 250, 512, 1000, 2048, 5000]))
    half = bool(rng.integers(0, 2))
    x = rng.standard_normal((rows, hidden)).astype(np.float32)
    r = rng.standard_normal((rows, hidden)).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    if half:
        xh, rh = h16(x), h16(r)
        y, out = gu.add_rms_norm(xh, rh, w, 1e-6)
        wy, wout = port.add_rms_norm(xh.astype(np.float32), rh.astype(np.float32), w, 1e-6)
        assert_fp16_close(y, wy)       # a sum of two fp16 values is exact in fp32: the one rounding only
        # the norm is computed from the fp32 sum, not from the rounded y
        assert_fp16_close(out, wout, **norm_terms(hidden))
        assert_fp16_close(gu.silu_mul(xh, rh), port.silu_mul(xh.astype(np.float32), rh.astype(np.float32)), **SILU)
    else:
        y, out = gu.add_rms_norm(x, r, w, 1e-6)
        wy, wout = port.add_rms_norm(x, r, w, 1e-6)
        np.testing.assert_array_equal(y, wy)
        np.testing.assert_allclose(out, wout, rtol=0, atol=TOL32 * max(1.0, float(np.abs(wout).max())))
        np.testing.assert_allclose(gu.rms_norm(x, w, 1e-5), port.rms_norm(x, w, 1e-5), rtol=0,
                                   atol=TOL32 * max(1.0, float(np.abs(wout).max())))
        np.testing.assert_allclose(gu.silu_mul(x, r), port.silu_mul(x, r), rtol=2e-6, atol=1e-6)
    heads, d = int(rng.integers(1, 20)), 2 * int(rng.choice([1, 4, 16, 32, 40, 64, 128]))
    xr = rng.standard_normal((rows, heads, d)).astype(np.float32)
    pos = rng.integers(0, 8192, rows).astype(np.int64)
    pos3 = rng.integers(0, 8192, (3, rows)).astype(np.int64)
    inv = port.rope_inv_freq(1e6, d)
    h_sec = w_sec = (d // 2) // 3
    sec = [d // 2 - 2 * h_sec, h_sec, w_sec]
    if half:
        xrh = h16(xr)
        f = xrh.astype(np.float32)
        assert_fp16_close(gu.rope(xrh, pos, 1e6), port.rope(f, pos, 1e6), **ROPE)
        assert_fp16_close(gu.rope_thd(xrh, pos3, inv, sec), port.rope_thd(f, pos3, inv, sec), **ROPE)
    else:
        np.testing.assert_allclose(gu.rope(xr, pos, 1e6), port.rope(xr, pos, 1e6), rtol=0, atol=2e-5)
        np.testing.assert_allclose(gu.rope_thd(xr, pos3, inv, sec), port.rope_thd(xr, pos3, inv, sec), rtol=0, atol=2e-5)
        c, s_ = gu.mrope_cos_sin(pos3, inv, h_sec, w_sec)
        wc, ws = port.mrope_cos_sin(pos3, inv, h_sec, w_sec)
        np.testing.assert_allclose(c, wc, rtol=0, atol=2e-5)
        np.testing.assert_allclose(s_, ws, rtol=0, atol=2e-5)
        np.testing.assert_allclose(gu.rope_with_cos_sin(xr, wc, ws), port.rope_with_cos_sin(xr, wc, ws), rtol=0, atol=TOL32)


@pytest.mark.parametrize("seed", range(12))
def test_general_attention_random_shapes(seed):
    """Query / key counts, head counts and head sizes at random, causal and not, fp32 and fp16: the
    matrix-core route (fp16, head size 64 / 128, 32 or more query rows), the split-K route and the
    plain kernel for other head sizes."""
    rng = np.random.default_rng(9900 + seed)
    sq = int(rng.choice([1, 3, 31, 32, 33, 64, 130, 257]))
    skv = int(rng.choice([1, 5, 64, 100, 257, 600]))
    hkv = int(rng.integers(1, 4))
    group = int(rng.choice([1, 2, 3, 4]))
    d = int(rng.choice([8, 32, 64, 128, 256]))
    half = bool(rng.integers(0, 2))
    q = rng.standard_normal((sq, hkv * group, d)).astype(np.float32)
    k = rng.standard_normal((skv, hkv, d)).astype(np.float32)
    v = rng.standard_normal((skv, hkv, d)).astype(np.float32)
    for causal in (False, True):
        if half:
            qh, kh, vh = h16(q), h16(k), h16(v)
            want = port.sdpa(qh.astype(np.float32), kh.astype(np.float32), vh.astype(np.float32), causal)
            assert_fp16_attention(gu.sdpa(qh, kh, vh, causal), want)
        else:
            np.testing.assert_allclose(gu.sdpa(q, k, v, causal), port.sdpa(q, k, v, causal), rtol=0, atol=TOL32)


@pytest.mark.parametrize("seed", range(6))
def test_cache_and_index_operators_random_shapes(seed):
    rng = np.random.default_rng(9950 + seed)
    B, hkv, lmax, d = int(rng.integers(1, 9)), int(rng.integers(1, 5)), int(rng.integers(1, 300)), int(rng.choice([8, 64, 128]))
    dtype = np.float16 if rng.integers(0, 2) else np.float32
    kc = rng.standard_normal((B, hkv, lmax, d)).astype(dtype)
    vc = rng.standard_normal((B, hkv, lmax, d)).astype(dtype)
    kn = rng.standard_normal((B, hkv, d)).astype(dtype)
    vn = rng.standard_normal((B, hkv, d)).astype(dtype)
    pos = rng.integers(0, lmax, B).astype(np.int64)
    wk, wv = kc.copy(), vc.copy()
    port.kv_append(kn, vn, wk, wv, pos)
    gk, gv = gu.kv_append(kn, vn, kc, vc, pos)
    np.testing.assert_array_equal(gk.view(np.uint8), wk.view(np.uint8))
    np.testing.assert_array_equal(gv.view(np.uint8), wv.view(np.uint8))
    a = rng.standard_normal((int(rng.integers(1, 50)), hkv, d)).astype(dtype)
    b = rng.standard_normal((int(rng.integers(1, 5)), hkv, d)).astype(dtype)
    np.testing.assert_array_equal(gu.concat_axis0(a, b).view(np.uint8), np.concatenate([a, b], 0).view(np.uint8))
    vocab, dim = int(rng.integers(2, 3000)), int(rng.choice([4, 64, 100]))
    table = rng.standard_normal((vocab, dim)).astype(dtype)
    ids = rng.integers(0, vocab, (int(rng.integers(1, 6)), int(rng.integers(1, 9)))).astype(np.int64)
    np.testing.assert_array_equal(gu.embedding(ids, table).view(np.uint8), table[ids].view(np.uint8))
    cols = int(rng.choice([1, 7, 1000, 16384, 40000]))
    lg = rng.standard_normal((int(rng.integers(1, 20)), cols)).astype(np.float32)
    np.testing.assert_array_equal(gu.argmax(lg), np.argmax(lg, -1))
