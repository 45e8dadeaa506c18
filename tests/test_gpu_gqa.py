"""GQA decode attention on the GPU against the CPU oracle (through the C ABI).

fp32: max abs error <= 1e-5.  fp16: inputs are fp16-rounded, the oracle does fp32 arithmetic on
them, the kernel rounds once at the store: max abs error <= 2e-3.
"""
import os

import numpy as np
import pytest

import oracle
from oracle import port

import gpu_util as gu
from gpu_util import gqa_decode, lib

pytestmark = pytest.mark.gpu

TOL32, TOL16 = 1e-5, 2e-3
G = np.load(os.path.join(os.path.dirname(__file__), "golden", "decode_path_golden.npz"))


def _qkv_ref(rng, L, hq=16, hkv=8, d=128, dtype=np.float32):
    q = rng.standard_normal((1, hq, d)).astype(np.float32).astype(dtype)
    k = rng.standard_normal((L, hkv, d)).astype(np.float32).astype(dtype)
    v = rng.standard_normal((L, hkv, d)).astype(np.float32).astype(dtype)
    return q, k, v


def test_reference_shape_fp32_config1():
    """B=1, Hq16/Hkv8, D=128, L=1024, fp32 (the reference's own call shape)."""
    rng = np.random.default_rng(1)
    q, k, v = _qkv_ref(rng, 1024)
    out = gqa_decode(q, k, v, layout="ref")
    np.testing.assert_allclose(out, port.gqa_decode(q, k, v), rtol=0, atol=TOL32)


@pytest.mark.parametrize("L", [1, 7, 256, 512, 1024])
def test_reference_seeds_fp32(L):
    rs = np.random.RandomState(3)
    for n in (1, 7, 256, 512, 1024):
        q = rs.randn(1, 16, 128).astype(np.float32)
        k = rs.randn(n, 8, 128).astype(np.float32)
        v = rs.randn(n, 8, 128).astype(np.float32)
        if n == L:
            np.testing.assert_allclose(gqa_decode(q, k, v, layout="ref"), port.gqa_decode(q, k, v), rtol=0, atol=TOL32)


def test_golden_fixtures():
    for L in (1, 7, 40):
        out = gqa_decode(G[f"gqa_L{L}_q"], G[f"gqa_L{L}_k"], G[f"gqa_L{L}_v"], layout="ref")
        np.testing.assert_allclose(out, G[f"gqa_L{L}_out"], rtol=0, atol=TOL32)
    out = gqa_decode(G["gqa16_q"], G["gqa16_k"], G["gqa16_v"], layout="ref")
    np.testing.assert_allclose(out.astype(np.float32), G["gqa16_out"], rtol=0, atol=TOL16)


@pytest.mark.parametrize("L", [2048, 4097, 16385])
def test_long_context_splits_fp32(L):
    """Lengths the reference would send to its split-K kernels (L >= 2048), incl. a ragged tail."""
    rng = np.random.default_rng(L)
    q, k, v = _qkv_ref(rng, L)
    np.testing.assert_allclose(gqa_decode(q, k, v, layout="ref"), port.gqa_decode(q, k, v), rtol=0, atol=TOL32)


@pytest.mark.parametrize("B,L", [(1, 1024), (8, 1024), (32, 1024), (4, 8192), (2, 32768)])
def test_cache_layout_fp16(B, L):
    rng = np.random.default_rng(B * 100003 + L)
    q = rng.standard_normal((B, 16, 128)).astype(np.float32).astype(np.float16)
    k = rng.standard_normal((B, 8, L, 128)).astype(np.float32).astype(np.float16)
    v = rng.standard_normal((B, 8, L, 128)).astype(np.float32).astype(np.float16)
    out = gqa_decode(q, k, v).astype(np.float32)
    want = port.gqa_decode_cache_native(q, k, v)
    err = np.abs(out - want).max()
    assert err <= TOL16, (err, np.abs(want).max())


def test_ragged_batch_fp16():
    rng = np.random.default_rng(77)
    B, Lmax = 8, 4096
    lens = rng.integers(1, Lmax + 1, B).astype(np.int32)
    lens[0], lens[1], lens[2] = Lmax, 1, 0  # full, single key, empty (zeros by convention)
    q = rng.standard_normal((B, 16, 128)).astype(np.float32).astype(np.float16)
    k = rng.standard_normal((B, 8, Lmax, 128)).astype(np.float32).astype(np.float16)
    v = rng.standard_normal((B, 8, Lmax, 128)).astype(np.float32).astype(np.float16)
    out = gqa_decode(q, k, v, lens).astype(np.float32)
    want = port.gqa_decode_cache_native(q, k, v, lens)
    assert np.abs(out - want).max() <= TOL16
    assert np.all(out[2] == 0)
    np.testing.assert_array_equal(out[1, 0], v[1, 0, 0].astype(np.float32))  # one key: out = v


@pytest.mark.parametrize("hq,hkv,d", [(8, 8, 64), (8, 2, 128), (16, 2, 64), (4, 1, 256), (6, 2, 128)])
def test_head_shapes(hq, hkv, d):
    """group sizes 1, 4, 8, 4 (D=256) and 3 (not a power of two)."""
    rng = np.random.default_rng(hq * 31 + d)
    B, L = 3, 777
    lens = np.array([777, 300, 1], np.int32)
    for dtype, tol in ((np.float32, TOL32), (np.float16, TOL16)):
        q = rng.standard_normal((B, hq, d)).astype(np.float32).astype(dtype)
        k = rng.standard_normal((B, hkv, L, d)).astype(np.float32).astype(dtype)
        v = rng.standard_normal((B, hkv, L, d)).astype(np.float32).astype(dtype)
        out = gqa_decode(q, k, v, lens).astype(np.float32)
        want = port.gqa_decode_cache_native(q, k, v, lens)
        assert np.abs(out - want).max() <= tol


@pytest.mark.parametrize("hq,hkv,d", [(32, 8, 128), (32, 4, 128), (64, 8, 128), (28, 4, 128), (40, 2, 64), (16, 4, 64)])
def test_large_head_groups_on_the_matrix_cores(hq, hkv, d):
    """Four and more query heads per kv head (fp16): the heads are the columns of an MFMA tile.  Group
    sizes 4, 8, 7 (not a power of two), 20 (two workgroups of 10 heads per kv head); lengths that are
    not multiples of the 32 keys of a wavefront or the 128 of a stage, a single key, an empty sequence;
    the reference's (L, Hkv, D) layout; cut into ranges in one launch and in two; and against the vector
    path on the same inputs."""
    rng = np.random.default_rng(hq * 7 + hkv + d)
    Lmax = 1500
    lens = np.array([1500, 0, 1, 33, 127, 129, 1279, 640], np.int32)
    B = len(lens)
    q = rng.standard_normal((B, hq, d)).astype(np.float32).astype(np.float16)
    k = rng.standard_normal((B, hkv, Lmax, d)).astype(np.float32).astype(np.float16)
    v = rng.standard_normal((B, hkv, Lmax, d)).astype(np.float32).astype(np.float16)
    want = port.gqa_decode_cache_native(q, k, v, lens)
    l = lib()
    outs = {}
    try:
        for name, tune in (("default", (0, 0)), ("3 ranges", (0, 3)), ("3 ranges, merge kernel", (-1, 3)),
                           ("vector path", (0, 1000))):
            l.axhip_gqa_decode_tune(*tune)
            outs[name] = gqa_decode(q, k, v, lens).astype(np.float32)
    finally:
        l.axhip_gqa_decode_tune(0, 0)
    for name, out in outs.items():
        assert np.abs(out - want).max() <= TOL16, name
        assert np.all(out[1] == 0), name
    # the matrix-core path rounds the probabilities to fp16 before the second product; the vector path does not
    assert np.abs(outs["default"] - outs["vector path"]).max() <= TOL16
    # the reference's call: one sequence, k/v (L, Hkv, D)
    L = 700
    q1 = rng.standard_normal((1, hq, d)).astype(np.float32).astype(np.float16)
    k1 = rng.standard_normal((L, hkv, d)).astype(np.float32).astype(np.float16)
    v1 = rng.standard_normal((L, hkv, d)).astype(np.float32).astype(np.float16)
    np.testing.assert_allclose(gqa_decode(q1, k1, v1, layout="ref").astype(np.float32), port.gqa_decode(q1, k1, v1),
                               rtol=0, atol=TOL16)


def test_result_independent_of_split_count():
    rng = np.random.default_rng(5)
    q, k, v = _qkv_ref(rng, 5000)
    outs = []
    for splits in (1, 3, 16):
        with gu.gqa_tuned(0, splits):
            outs.append(gqa_decode(q, k, v, layout="ref"))
    want = port.gqa_decode(q, k, v)
    for o in outs:
        np.testing.assert_allclose(o, want, rtol=0, atol=TOL32)


def test_forced_ranges_with_more_than_2048_head_groups():
    """Ticket counters are laid out so that neighbouring (sequence, head group) pairs sit on different cache lines
    and pair 2048 takes the word next to pair 0: a batch with 2080 pairs, every sequence cut into two and three
    merged ranges, twice in a row (the counters must be back at zero after a launch)."""
    rng = np.random.default_rng(2080)
    B, hq, hkv, d, L = 260, 16, 8, 64, 96
    q = rng.standard_normal((B, hq, d)).astype(np.float16)
    k = rng.standard_normal((B, hkv, L, d)).astype(np.float16)
    v = rng.standard_normal((B, hkv, L, d)).astype(np.float16)
    lens = rng.integers(1, L + 1, B).astype(np.int32)
    want = port.gqa_decode_cache(q, k, v, lens)
    for splits in (2, 3, 2):
        with gu.gqa_tuned(0, splits):
            got = gqa_decode(q, k, v, seq_lens=lens)
        np.testing.assert_allclose(got.astype(np.float32), want, rtol=0, atol=TOL16)


def test_invariants_full_size_headline():
    """B=32, L=8192 fp16 (1 GiB of cache): properties that need no oracle pass over the data.
    Identical keys give the mean of V; the first sequence is also checked against the oracle."""
    B, L = 32, 8192
    rng = np.random.default_rng(9)
    q = rng.standard_normal((B, 16, 128)).astype(np.float32).astype(np.float16)
    v = rng.standard_normal((B, 8, L, 128)).astype(np.float32).astype(np.float16)
    k = np.empty((B, 8, L, 128), np.float16)
    k[:] = rng.standard_normal((B, 8, 1, 128)).astype(np.float16)  # every key of a head identical
    k[0] = rng.standard_normal((8, L, 128)).astype(np.float16)      # sequence 0: ordinary keys
    out = gqa_decode(q, k, v).astype(np.float32)
    mean_v = v.astype(np.float32).mean(axis=2)  # [B,8,128]
    for h in range(16):
        assert np.abs(out[1:, h] - mean_v[1:, h // 2]).max() <= TOL16
    want0 = port.gqa_decode_cache_native(q[:1], k[:1], v[:1])
    assert np.abs(out[:1] - want0).max() <= TOL16


class _PeriodicCache:
    """The largest configuration's cache on the device: K and V [64, 8, 32768, 128] fp16 (8.6 GB), every
    (sequence, kv head) row repeating a block of P = 1024 random keys / values (uploaded once per row and
    doubled by device copies).  Attention over r whole repetitions of a block equals attention over the
    block (every copy of a key gets the same weight), so the oracle on the block checks full-size launches;
    a length r*P + t is checked by the oracle on that sequence's rows written out on the host."""
    B, Hq, Hkv, D, L, P = 64, 16, 8, 128, 32768, 1024

    def __init__(self):
        rng = np.random.default_rng(64)
        B, Hq, Hkv, D, L, P = self.B, self.Hq, self.Hkv, self.D, self.L, self.P
        self.q = rng.standard_normal((B, Hq, D)).astype(np.float32).astype(np.float16)
        self.kp = rng.standard_normal((B, Hkv, P, D)).astype(np.float32).astype(np.float16)
        self.vp = rng.standard_normal((B, Hkv, P, D)).astype(np.float32).astype(np.float16)
        l = lib()
        row_bytes, blk = L * D * 2, P * D * 2
        bufs = []
        for host in (self.kp, self.vp):
            big = gu.DeviceBuffer(B * Hkv * row_bytes)
            for r in range(B * Hkv):
                base = big.ptr + r * row_bytes
                gu.check(l.axhip_memcpy_h2d(base, host.reshape(B * Hkv, -1)[r].ctypes.data, blk), "h2d")
                have = blk
                while have < row_bytes:
                    gu.check(l.axhip_memcpy_d2d(base + have, base, have), "d2d")
                    have *= 2
            bufs.append(big)
        self.dk, self.dv = bufs
        self.dq = gu.dev(self.q)
        self.block_out = port.gqa_decode_cache_native(self.q, self.kp, self.vp, np.full(B, P, np.int32))

    def run(self, B, max_len, lens):
        """The first B sequences of the cache, attended up to lens[b] <= max_len keys (rows keep the big
        cache's strides: the batched layout with Lmax = 32768)."""
        l = lib()
        out = gu.DeviceBuffer(B * self.Hq * self.D * 2)
        wsb = l.axhip_gqa_decode_workspace_bytes(B, self.Hq, self.Hkv, self.D, max_len)
        ws = gu.DeviceBuffer(max(wsb, 256))
        dl = gu.dev(np.asarray(lens, np.int32))
        gu.check(l.axhip_gqa_decode(self.dq.ptr, self.dk.ptr, self.dv.ptr, dl.ptr, out.ptr, ws.ptr, wsb, gu.F16, B,
                                    self.Hq, self.Hkv, self.D, max_len, self.Hkv * self.L * self.D, self.L * self.D,
                                    self.D, None), "gqa_decode")
        gu.synchronize()
        return out.download(np.float16, (B, self.Hq, self.D)).astype(np.float32)

    def oracle_rows(self, b, length):
        """The oracle on sequence b's first `length` keys, written out on the host."""
        reps = -(-length // self.P)
        k = np.ascontiguousarray(np.tile(self.kp[b:b + 1], (1, 1, reps, 1))[:, :, :length])
        v = np.ascontiguousarray(np.tile(self.vp[b:b + 1], (1, 1, reps, 1))[:, :, :length])
        return port.gqa_decode_cache_native(self.q[b:b + 1], k, v, np.array([length], np.int32))[0]

    def release(self):
        self.dk.release()
        self.dv.release()


@pytest.fixture(scope="module")
def periodic_cache():
    c = _PeriodicCache()
    yield c
    c.release()


@pytest.mark.parametrize("B", [1, 8, 32, 64])
@pytest.mark.parametrize("L", [1024, 8192, 32768])
def test_config3_sweep_points_at_full_size(B, L, periodic_cache):
    """Every point of the B x L sweep at its full size, uniform lengths, default split plan."""
    c = periodic_cache
    got = c.run(B, L, np.full(B, L, np.int32))
    assert np.abs(got - c.block_out[:B]).max() <= TOL16, (B, L)


def test_largest_config_ragged_whole_blocks(periodic_cache):
    """B=64, Lmax=32768 with ragged multiples of the block (the end-to-end cut of the key axis), a full,
    a one-block and an empty sequence."""
    c = periodic_cache
    rng = np.random.default_rng(65)
    lens = (c.P * rng.integers(1, c.L // c.P + 1, c.B)).astype(np.int32)
    lens[:3] = [c.L, c.P, 0]
    got = c.run(c.B, c.L, lens)
    live = lens > 0
    assert np.abs(got[live] - c.block_out[live]).max() <= TOL16
    assert np.all(got[~live] == 0)


def test_config3_ragged_batch_arbitrary_lengths(periodic_cache):
    """The ragged batch of the sweep: B=32, lengths uniform in [512, 32768] and not multiples of anything
    (both ends of the interval and an odd length forced in), Lmax = 32768.  Each sequence is checked by
    the oracle on its own rows written out on the host."""
    c = periodic_cache
    rng = np.random.default_rng(3232)
    B = 32
    lens = rng.integers(512, 32769, B).astype(np.int32)
    lens[0], lens[1], lens[2], lens[3] = 512, 32768, 32767, 513
    got = c.run(B, c.L, lens)
    worst = 0.0
    for b in range(B):
        worst = max(worst, float(np.abs(got[b] - c.oracle_rows(b, int(lens[b]))).max()))
    assert worst <= TOL16, worst


def test_more_than_64_sequences_take_the_static_plan_by_default():
    """Batches above 64 sequences are cut by the host-side static plan (every sequence into n_splits
    ranges from the grid).  Default tuning: 80 sequences of Hq16/Hkv8 (one range each), and 80 sequences
    with one head group, which the plan cuts into several ranges merged in the kernel."""
    rng = np.random.default_rng(80)
    l = lib()
    for (B, hq, hkv, Lmax, want_splits) in ((80, 16, 8, 1500, 1), (80, 2, 1, 4096, 4), (200, 2, 1, 700, 2)):
        lens = rng.integers(1, Lmax + 1, B).astype(np.int32)
        lens[:4] = [Lmax, 0, 1, 257]
        import ctypes as C
        ns, ch = C.c_int(0), C.c_int(0)
        l.axhip_gqa_decode_plan(B, hq, hkv, Lmax, C.byref(ns), C.byref(ch))
        assert ns.value == want_splits, (B, hq, ns.value)
        q = rng.standard_normal((B, hq, 128)).astype(np.float32).astype(np.float16)
        k = rng.standard_normal((B, hkv, Lmax, 128)).astype(np.float32).astype(np.float16)
        v = rng.standard_normal((B, hkv, Lmax, 128)).astype(np.float32).astype(np.float16)
        got = gqa_decode(q, k, v, lens).astype(np.float32)
        want = port.gqa_decode_cache_native(q, k, v, lens)
        assert np.abs(got - want).max() <= TOL16, (B, hq)
        assert np.all(got[1] == 0)


def test_error_codes():
    l = lib()
    assert l.axhip_gqa_decode(None, None, None, None, None, None, 0, 5, 1, 16, 8, 128, 16, 0, 0, 0, None) == 7
    assert l.axhip_gqa_decode(None, None, None, None, None, None, 0, 5, 1, 16, 5, 128, 16, 0, 0, 0, None) == 4
    assert l.axhip_gqa_decode(None, None, None, None, None, None, 0, 3, 1, 16, 8, 128, 16, 0, 0, 0, None) == 3
    assert l.axhip_gqa_decode(None, None, None, None, None, None, 0, 5, 1, 16, 8, 96, 16, 0, 0, 0, None) == 1


def test_two_kernel_merge_mode_matches_fused_merge():
    """The default plan (workgroups dealt to the sequences by length, merge by the last workgroup of
    a sequence), a fixed split count with the same in-kernel merge, and a fixed split count with a
    second merge kernel give the same result (all against the oracle), also with empty, one-key and
    single-range sequences in the batch."""
    rng = np.random.default_rng(15)
    B, Lmax = 6, 3000
    lens = np.array([3000, 0, 1, 257, 1500, 2999], np.int32)
    q = rng.standard_normal((B, 16, 128)).astype(np.float32).astype(np.float16)
    k = rng.standard_normal((B, 8, Lmax, 128)).astype(np.float32).astype(np.float16)
    v = rng.standard_normal((B, 8, Lmax, 128)).astype(np.float32).astype(np.float16)
    want = port.gqa_decode_cache_native(q, k, v, lens)
    fused = gqa_decode(q, k, v, lens).astype(np.float32)      # default
    # repeated launches reuse the ticket counters
    for _ in range(3):
        again = gqa_decode(q, k, v, lens).astype(np.float32)
        np.testing.assert_array_equal(again, fused)
    with gu.gqa_tuned(0, 5):                                   # 5 ranges per sequence, in-kernel merge
        fixed = gqa_decode(q, k, v, lens).astype(np.float32)
    with gu.gqa_tuned(-1, 5):                                  # 5 ranges per sequence, split kernel + merge kernel
        two = gqa_decode(q, k, v, lens).astype(np.float32)
    for o in (fused, fixed, two):
        assert np.abs(o - want).max() <= TOL16
        assert np.all(o[1] == 0)
    np.testing.assert_array_equal(fixed, two)                  # same ranges, same merge arithmetic
    # a single split and an empty sequence (the split-0 workgroup writes the zeros)
    with gu.gqa_tuned(0, 1):
        one = gqa_decode(q, k, v, lens).astype(np.float32)
    assert np.abs(one - want).max() <= TOL16 and np.all(one[1] == 0)


def _check_decode_step_form(Hq, Hkv, D, lens, rows, max_len, forced=(0, 5), seed=77):
    rng = np.random.default_rng(seed)
    lens = np.asarray(lens, np.int32)
    B = len(lens)
    width = (Hq + 2 * Hkv) * D
    qkv = rng.standard_normal((B, width)).astype(np.float32)
    qw = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    kw = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    pos = rng.integers(0, 8192, (3, B)).astype(np.int64)
    inv = port.rope_inv_freq(1e6, D)
    hw = 10 if D == 64 else 20
    sec = [D // 2 - 2 * hw, hw, hw]
    kc = (0.5 * rng.standard_normal((B, Hkv, rows, D))).astype(np.float16)
    vc = rng.standard_normal((B, Hkv, rows, D)).astype(np.float16)
    l = gu.lib()
    dq, dqw, dkw, dp, di, dl, dkc, dvc = (gu.dev(a) for a in (qkv, qw, kw, pos, inv, lens, kc, vc))
    out = gu.DeviceBuffer(B * Hq * D * 2)
    for force_splits in forced:
        l.axhip_gqa_decode_tune(0, force_splits)
        dkc.upload(kc.reshape(-1))
        dvc.upload(vc.reshape(-1))
        wsb = l.axhip_gqa_decode_workspace_bytes(B, Hq, Hkv, D, max_len)
        ws = gu.DeviceBuffer(max(wsb, 256))
        gu._run("axhip_gqa_decode_qkv", dq.ptr, width, dq.ptr + Hq * D * 4, width, dq.ptr + (Hq + Hkv) * D * 4, width,
                dqw.ptr, dkw.ptr, gu.F32, 1e-6, dp.ptr, di.ptr, hw, hw, dl.ptr, dkc.ptr, dvc.ptr, out.ptr, ws.ptr, wsb,
                gu.F16, B, Hq, Hkv, D, rows, max_len, None)
        gu.synchronize()
        q = port.rope_thd(port.rms_norm(qkv[:, : Hq * D].reshape(B, Hq, D), qw, 1e-6), pos, inv, sec)
        k = port.rope_thd(port.rms_norm(qkv[:, Hq * D:(Hq + Hkv) * D].reshape(B, Hkv, D), kw, 1e-6), pos, inv, sec)
        v = qkv[:, (Hq + Hkv) * D:].reshape(B, Hkv, D)
        wk, wv = kc.copy(), vc.copy()
        attended = lens.copy()
        for b in range(B):
            if lens[b] < max_len:
                wk[b, :, lens[b]] = k[b].astype(np.float16)
                wv[b, :, lens[b]] = v[b].astype(np.float16)
                attended[b] += 1
        gk, gv = dkc.download(np.float16, kc.shape), dvc.download(np.float16, vc.shape)
        np.testing.assert_array_equal(gv.view(np.uint16), wv.view(np.uint16))
        assert np.abs(gk.astype(np.float32) - wk.astype(np.float32)).max() <= 2e-3
        untouched = np.ones(kc.shape, bool)
        for b in range(B):
            if lens[b] < max_len:
                untouched[b, :, lens[b]] = False
        np.testing.assert_array_equal(gk[untouched].view(np.uint16), kc[untouched].view(np.uint16))
        # attention of the oracle over the cache as the device wrote it, with q rounded to the cache dtype
        want = port.gqa_decode_cache_native(q.astype(np.float16).astype(np.float32), gk.astype(np.float32),
                                              gv.astype(np.float32), attended)
        got = out.download(np.float16, (B, Hq, D)).astype(np.float32)
        assert np.abs(got - want).max() <= 2e-3, (force_splits, np.abs(got - want).max())
        if force_splits == 0:
            # the launches of one step share what the first dealt: a launch that leaves its table, launches that take
            # it (twice: the table must survive being read), and one of another max_len, which the table is not for
            def launch(mode, ml):
                dkc.upload(kc.reshape(-1))
                dvc.upload(vc.reshape(-1))
                out.upload(np.full(B * Hq * D // 2, np.nan, np.float32))
                assert l.axhip_set_plan_reuse(mode) == 0
                try:
                    gu._run("axhip_gqa_decode_qkv", dq.ptr, width, dq.ptr + Hq * D * 4, width, dq.ptr + (Hq + Hkv) * D * 4,
                            width, dqw.ptr, dkw.ptr, gu.F32, 1e-6, dp.ptr, di.ptr, hw, hw, dl.ptr, dkc.ptr, dvc.ptr, out.ptr,
                            ws.ptr, wsb, gu.F16, B, Hq, Hkv, D, rows, ml, None)
                finally:
                    l.axhip_set_plan_reuse(0)
                gu.synchronize()
                return (out.download(np.uint16, (B, Hq, D)), dkc.download(np.uint16, kc.shape),
                        dvc.download(np.uint16, vc.shape))
            plain = launch(0, max_len)
            np.testing.assert_array_equal(plain[0], got.astype(np.float16).view(np.uint16))
            for mode in (1, 2, 2):
                for a_, b_ in zip(launch(mode, max_len), plain):
                    np.testing.assert_array_equal(a_, b_)
            if max_len > 300:
                shorter = launch(0, max_len - 128)
                for a_, b_ in zip(launch(2, max_len - 128), shorter):
                    np.testing.assert_array_equal(a_, b_)
    l.axhip_gqa_decode_tune(0, 0)
    return dq, dp, di, dl, dkc, dvc, out, ws, wsb, width, hw


@pytest.mark.parametrize("Hq,Hkv,D", [(4, 2, 128), (8, 1, 64), (3, 3, 256), (8, 2, 128), (20, 1, 128), (32, 4, 64)])
def test_decode_step_form_equals_append_then_attention(Hq, Hkv, D):
    """axhip_gqa_decode_qkv (q/k norm + M-RoPE + append + attention in the split kernel) against the
    oracle's rms_norm -> rope_thd -> fp16 rounding -> append -> attention over len + 1 keys; sequences
    that put the new row in the first split, in the last split, and alone in a split of its own."""
    rows, max_len = 1300, 1280
    lens = [0, 5, 255, 256, 700, 1279, 1280]   # 1280: cache bound reached, nothing appended
    B = len(lens)
    dq, dp, di, dl, dkc, dvc, out, ws, wsb, width, hw = _check_decode_step_form(Hq, Hkv, D, lens, rows, max_len)
    l = gu.lib()
    # argument checks: seq_lens is required; max_len may not exceed the cache
    args = [dq.ptr, width, dq.ptr, width, dq.ptr, width, None, None, gu.F32, 1e-6, dp.ptr, di.ptr, hw, hw]
    assert l.axhip_gqa_decode_qkv(*args, None, dkc.ptr, dvc.ptr, out.ptr, ws.ptr, wsb, gu.F16, B, Hq, Hkv, D, rows,
                                  max_len, None) == 7
    assert l.axhip_gqa_decode_qkv(*args, dl.ptr, dkc.ptr, dvc.ptr, out.ptr, ws.ptr, wsb, gu.F16, B, Hq, Hkv, D, rows,
                                  rows + 1, None) == 1


def test_decode_step_form_ragged_batch_with_one_workgroup_per_sequence_to_share():
    """As many sequences as the launch has workgroups per head group, of very different lengths:
    the workgroups then share the keys of the whole batch end to end, each working through pieces of
    several sequences, and the new token's row may be a piece of its own."""
    rng = np.random.default_rng(5)
    max_len = 2400
    lens = rng.integers(0, max_len, 32)
    lens[[0, 7, 31]] = 0
    lens[[1, 8]] = [max_len, max_len - 1]
    lens[[2, 3]] = [1, 127]
    _check_decode_step_form(16, 8, 128, lens, max_len + 8, max_len, forced=(0,), seed=6)
    # the same with four heads per kv head (the matrix-core path)
    _check_decode_step_form(16, 4, 128, lens, max_len + 8, max_len, forced=(0,), seed=7)


@pytest.mark.parametrize("Hq,Hkv,D,S,start", [(4, 2, 128, 200, [0, 37]), (2, 2, 128, 64, [0, 0]), (8, 2, 64, 130, [5, 300]),
                                               (16, 8, 128, 257, [0, 1])])
def test_prefill_attention_matches_causal_oracle(Hq, Hkv, D, S, start, q_scale=1.0):
    """axhip_prefill_attention (MFMA, fp16 probabilities) against the CPU operator with the causal
    mask, per sequence: query i at absolute position start + i sees cache rows 0 .. start + i.  Cache
    rows past the last visible key hold NaN bit patterns: they must not leak into the result."""
    rng = np.random.default_rng(11)
    B = len(start)
    rows = max(start) + S + 70
    q = (q_scale * rng.standard_normal((B, S, Hq, D))).astype(np.float16)
    kc = rng.standard_normal((B, Hkv, rows, D)).astype(np.float16)
    vc = rng.standard_normal((B, Hkv, rows, D)).astype(np.float16)
    for b in range(B):
        kc[b, :, start[b] + S:] = np.float16(np.nan)
        vc[b, :, start[b] + S:] = np.float16(np.nan)
    st = np.asarray(start, np.int32)
    dq, dk, dv, ds = (gu.dev(a) for a in (q, kc, vc, st))
    out = gu.DeviceBuffer(q.nbytes)
    gu._run("axhip_prefill_attention", dq.ptr, dk.ptr, dv.ptr, ds.ptr, out.ptr, gu.F16, B, S, Hq, Hkv, D, rows, None)
    gu.synchronize()
    got = out.download(np.float16, q.shape).astype(np.float32)
    assert np.isfinite(got).all()
    worst = 0.0
    for b in range(B):
        L = start[b] + S
        k = np.ascontiguousarray(np.transpose(kc[b, :, :L], (1, 0, 2)), dtype=np.float32)   # [L, Hkv, D]
        v = np.ascontiguousarray(np.transpose(vc[b, :, :L], (1, 0, 2)), dtype=np.float32)
        for i in sorted(i for i in {0, 1, 15, 16, 63, min(64, S - 1), S // 2, S - 2, S - 1} if 0 <= i < S):
            vis = start[b] + i + 1
            want = port.sdpa(q[b, i:i + 1].astype(np.float32), k[:vis], v[:vis], False)[0]
            worst = max(worst, float(np.abs(got[b, i] - want).max()))
    assert worst <= 2e-3, worst
    if max(start) == 0:   # whole sequences through the operator's own causal path
        for b in range(B):
            k = np.ascontiguousarray(np.transpose(kc[b, :, :S], (1, 0, 2)), dtype=np.float32)
            v = np.ascontiguousarray(np.transpose(vc[b, :, :S], (1, 0, 2)), dtype=np.float32)
            want = port.sdpa(q[b].astype(np.float32), k, v, True)
            assert np.abs(got[b] - want).max() <= 2e-3
    l = gu.lib()
    assert l.axhip_prefill_attention(dq.ptr, dk.ptr, dv.ptr, ds.ptr, out.ptr, gu.F32, B, S, Hq, Hkv, D, rows, None) == 3
    assert l.axhip_prefill_attention(dq.ptr, dk.ptr, dv.ptr, ds.ptr, out.ptr, gu.F16, B, S, Hq, Hkv, 256, rows, None) == 1


@pytest.mark.parametrize("Hq,Hkv,S,B", [(4, 2, 1100, 1), (16, 8, 600, 8)])
def test_prefill_attention_both_workgroup_shapes_peaked_scores(Hq, Hkv, S, B):
    """Long rows with peaked softmax (queries three times the usual size: the running maximum jumps by more than
    the factor the kernel tolerates without rescaling, and stays put for long stretches) through both workgroup
    shapes: one round of eight-wavefront workgroups (18 of them), and four-wavefront workgroups (more than one
    eight-wavefront workgroup per CU would be needed)."""
    test_prefill_attention_matches_causal_oracle(Hq, Hkv, 128, S, [0] * B, q_scale=3.0)


@pytest.mark.parametrize("gap,peak_at", [(7.9, 3000), (8.1, 3000), (7.9, 5), (7.9, 4150)])
def test_prefill_attention_peak_next_to_a_long_plateau(gap, peak_at):
    """The running maximum of the prefill kernel follows a block only when it exceeds it by more than 8 (log2).
    Rows built to sit on that rule: 4200 keys, all with the same score except one peak `gap` log2 units above
    them - just inside the threshold (the maximum stays at the plateau, the peak's probability is 2^7.9 = 239 in
    fp16) and just outside (the maximum moves, everything accumulated is rescaled) - arriving after the maximum has
    settled, at the start, or in the last block; plus a second tier of 1000 keys 2^-10 below the plateau, whose
    probabilities would be subnormal in fp16 had the maximum followed the peak.  Every query row that sees the peak
    must match the oracle to the usual fp16 bar."""
    rng = np.random.default_rng(int(gap * 10) + peak_at)
    Hq, Hkv, D, S = 4, 2, 128, 4200
    c = 4.0
    x_peak = float(np.float16(gap * np.sqrt(D) / (c * np.log2(np.e))))
    x_low = float(np.float16(-10.0 * np.sqrt(D) / (c * np.log2(np.e))))
    q = np.zeros((1, S, Hq, D), np.float16)
    q[..., 0] = c
    q[..., 1:] = (0.01 * rng.standard_normal((1, S, Hq, D - 1))).astype(np.float16)
    kc = np.zeros((1, Hkv, S, D), np.float16)
    low = rng.choice(np.setdiff1d(np.arange(S), [peak_at]), 1000, replace=False)
    kc[0, :, low, 0] = x_low
    kc[0, :, peak_at, 0] = x_peak
    vc = rng.standard_normal((1, Hkv, S, D)).astype(np.float16)
    dq, dk, dv = (gu.dev(a) for a in (q, kc, vc))
    out = gu.DeviceBuffer(q.nbytes)
    gu._run("axhip_prefill_attention", dq.ptr, dk.ptr, dv.ptr, None, out.ptr, gu.F16, 1, S, Hq, Hkv, D, S, None)
    gu.synchronize()
    got = out.download(np.float16, q.shape).astype(np.float32)[0]
    k = np.ascontiguousarray(np.transpose(kc[0], (1, 0, 2)), dtype=np.float32)
    v = np.ascontiguousarray(np.transpose(vc[0], (1, 0, 2)), dtype=np.float32)
    rows = sorted({peak_at, min(peak_at + 1, S - 1), min(peak_at + 40, S - 1), (peak_at + S) // 2, S - 1, max(peak_at - 1, 0)})
    for i in rows:
        want = port.sdpa(q[0, i:i + 1].astype(np.float32), k[:i + 1], v[:i + 1], False)[0]
        err = float(np.abs(got[i] - want).max())
        assert err <= TOL16, (gap, peak_at, i, err)
    # the weight of the peak against the plateau is what the construction says (a check of the test itself)
    i = S - 1
    sc = (q[0, i, 0].astype(np.float32) @ k[:, 0].T) / np.sqrt(D) * np.log2(np.e)
    assert abs((sc[peak_at] - np.median(sc)) - gap) < 0.05


@pytest.mark.parametrize("B,Hq,Hkv,S", [(3, 4, 2, 300), (8, 2, 2, 130), (5, 16, 8, 200)])
def test_prefill_attention_workgroup_order_over_the_xcds(B, Hq, Hkv, S):
    """The two orders in which the workgroups of a launch are handed to the XCDs (all position blocks of a pair on
    one XCD, or dealt round-robin), each forced on pair counts that do and do not go round eight XCDs evenly: same
    bits, every output row written, and the oracle on a few rows."""
    rng = np.random.default_rng(B * 100 + S)
    D = 128
    q = rng.standard_normal((B, S, Hq, D)).astype(np.float16)
    kc = rng.standard_normal((B, Hkv, S, D)).astype(np.float16)
    vc = rng.standard_normal((B, Hkv, S, D)).astype(np.float16)
    dq, dk, dv = (gu.dev(a) for a in (q, kc, vc))
    outs = []
    l = gu.lib()
    try:
        for order in (0, 1):
            l.axhip_prefill_attention_tune(order)
            out = gu.DeviceBuffer(q.nbytes)
            gu.check(l.axhip_fill_zero(out.ptr, q.nbytes), "fill")
            gu._run("axhip_prefill_attention", dq.ptr, dk.ptr, dv.ptr, None, out.ptr, gu.F16, B, S, Hq, Hkv, D, S, None)
            gu.synchronize()
            outs.append(out.download(np.uint16, q.shape))
    finally:
        l.axhip_prefill_attention_tune(-1)
    np.testing.assert_array_equal(outs[0], outs[1])
    got = outs[1].view(np.float16).astype(np.float32)
    for b in (0, B - 1):
        k = np.ascontiguousarray(np.transpose(kc[b], (1, 0, 2)), dtype=np.float32)
        v = np.ascontiguousarray(np.transpose(vc[b], (1, 0, 2)), dtype=np.float32)
        want = port.sdpa(q[b].astype(np.float32), k, v, True)
        assert np.abs(got[b] - want).max() <= TOL16


def test_workgroups_are_dealt_by_length():
    """Very uneven batches under the default plan: one long sequence among short ones, all equal,
    and lengths that leave some of the launch's workgroup slots unused."""
    rng = np.random.default_rng(33)
    hq, hkv, d, Lmax = 4, 2, 128, 6000
    for lens in ([6000, 17, 130, 1, 0, 900, 64, 3], [2048] * 5, [1] * 7, [6000] * 2, [0, 0, 5999]):
        lens = np.asarray(lens, np.int32)
        B = len(lens)
        q = rng.standard_normal((B, hq, d)).astype(np.float32).astype(np.float16)
        k = rng.standard_normal((B, hkv, Lmax, d)).astype(np.float32).astype(np.float16)
        v = rng.standard_normal((B, hkv, Lmax, d)).astype(np.float32).astype(np.float16)
        out = gqa_decode(q, k, v, lens).astype(np.float32)
        want = port.gqa_decode_cache_native(q, k, v, lens)
        assert np.abs(out - want).max() <= TOL16, lens
        assert np.all(out[lens == 0] == 0)
    # 32 workgroups per head group for up to 32 sequences: uneven lengths make the workgroups share the
    # keys of the batch end to end (a workgroup then works through pieces of several sequences); empty
    # sequences at the start, in the middle and at the end of the batch, and single keys
    hq, hkv, Lmax = 16, 8, 3000
    for B in (32, 9):
        lens = rng.integers(1, Lmax + 1, B).astype(np.int32)
        lens[[0, 4, B - 1]] = 0
        lens[[1, 5]] = 1
        lens[2] = Lmax
        q = rng.standard_normal((B, hq, d)).astype(np.float32).astype(np.float16)
        k = rng.standard_normal((B, hkv, Lmax, d)).astype(np.float32).astype(np.float16)
        v = rng.standard_normal((B, hkv, Lmax, d)).astype(np.float32).astype(np.float16)
        out = gqa_decode(q, k, v, lens).astype(np.float32)
        want = port.gqa_decode_cache_native(q, k, v, lens)
        assert np.abs(out - want).max() <= TOL16, lens
        assert np.all(out[lens == 0] == 0)


@pytest.mark.parametrize("seed", range(16))
def test_random_configurations_against_the_oracle(seed):
    """Batch, head counts (1 to 8 query heads per kv head: the vector kernel and the matrix-core kernel),
    head size, cache capacity, lengths (zeros included) and dtype drawn at random."""
    rng = np.random.default_rng(9100 + seed)
    B = int(rng.integers(1, 10))
    hkv = int(rng.integers(1, 4))
    group = int(rng.choice([1, 2, 3, 4, 5, 8]))
    d = int(rng.choice([64, 128, 256]))
    lmax = int(rng.choice([1, 17, 130, 700, 2100]))
    dtype = np.float16 if rng.integers(0, 2) else np.float32
    lens = rng.integers(0, lmax + 1, B).astype(np.int32)
    if rng.integers(0, 3) == 0:
        lens[:] = lmax
    q = rng.standard_normal((B, hkv * group, d)).astype(np.float32).astype(dtype)
    k = rng.standard_normal((B, hkv, lmax, d)).astype(np.float32).astype(dtype)
    v = rng.standard_normal((B, hkv, lmax, d)).astype(np.float32).astype(dtype)
    got = gqa_decode(q, k, v, seq_lens=lens).astype(np.float32)
    want = port.gqa_decode_cache(q, k, v, lens)
    tol = TOL16 if dtype == np.float16 else TOL32
    assert np.abs(got - want).max() <= tol, (B, hkv, group, d, lmax, dtype, lens, np.abs(got - want).max())
    assert np.all(got[lens == 0] == 0)


@pytest.mark.parametrize("seed", range(8))
def test_decode_step_form_random_configurations(seed):
    """The decode-step form (q/k norm, M-RoPE and append in the attention launch) over random batches,
    head shapes, capacities and lengths, with the plan left to the library."""
    rng = np.random.default_rng(9300 + seed)
    B = int(rng.integers(1, 9))
    hkv = int(rng.integers(1, 4))
    group = int(rng.choice([1, 2, 4, 8]))
    d = int(rng.choice([64, 128]))
    rows = int(rng.choice([16, 200, 900, 2304]))
    lens = rng.integers(0, rows, B)  # at least one free row everywhere
    _check_decode_step_form(hkv * group, hkv, d, lens, rows, rows, forced=(0,), seed=seed)


@pytest.mark.parametrize("seed", range(8))
def test_prefill_attention_random_configurations(seed):
    rng = np.random.default_rng(9800 + seed)
    hkv = int(rng.integers(1, 4))
    group = int(rng.choice([1, 2, 3, 4, 8]))
    d = int(rng.choice([64, 128]))
    S = int(rng.choice([1, 17, 64, 100, 200, 333]))
    start = [int(s) for s in rng.choice([0, 1, 63, 64, 150], int(rng.integers(1, 4)))]
    test_prefill_attention_matches_causal_oracle(hkv * group, hkv, d, S, start)


# ---- paged KV cache ------------------------------------------------------------------------------
def _paged_from_dense(k, v, lens, perm_seed, extra_pages=3):
    """Scatters a dense cache [B,Hkv,Lmax,D] into pools [n_pages,Hkv,128,D] through a random page table."""
    B, Hkv, Lmax, D = k.shape
    P = 128
    max_pages = -(-Lmax // P)
    need = [-(-int(n) // P) for n in lens]
    n_pages = sum(need) + extra_pages
    rng = np.random.default_rng(perm_seed)
    order = rng.permutation(n_pages)
    table = np.full((B, max_pages), -1, np.int32)
    kp = rng.standard_normal((n_pages, Hkv, P, D)).astype(k.dtype)   # unused rows hold noise, not zeros
    vp = rng.standard_normal((n_pages, Hkv, P, D)).astype(k.dtype)
    nxt = 0
    for b in range(B):
        for p in range(need[b]):
            pid = int(order[nxt]); nxt += 1
            table[b, p] = pid
            rows = min(P, Lmax - p * P)
            kp[pid, :, :rows] = k[b, :, p * P:p * P + rows]
            vp[pid, :, :rows] = v[b, :, p * P:p * P + rows]
    return kp, vp, table, n_pages, max_pages


def _gqa_paged(q, kp, vp, table, lens, max_len):
    l = lib()
    B, Hq, D = q.shape
    n_pages, Hkv = kp.shape[:2]
    dq, dk, dv, dt_, dl = (gu.dev(a) for a in (q, kp, vp, table, np.asarray(lens, np.int32)))
    out = gu.DeviceBuffer(q.nbytes)
    wsb = l.axhip_gqa_decode_workspace_bytes(B, Hq, Hkv, D, max_len)
    ws = gu.DeviceBuffer(max(wsb, 256))
    gu.check(l.axhip_gqa_decode_paged(dq.ptr, dk.ptr, dv.ptr, dt_.ptr, dl.ptr, out.ptr, ws.ptr, wsb, gu.dt(q), B, Hq, Hkv,
                                      D, max_len, table.shape[1], n_pages, None), "gqa_decode_paged")
    gu.synchronize()
    return out.download(q.dtype, q.shape)


@pytest.mark.parametrize("dtype,hq,hkv,d", [(np.float16, 16, 8, 128), (np.float32, 16, 8, 128), (np.float16, 8, 8, 64),
                                             (np.float16, 16, 4, 128), (np.float32, 4, 2, 256)])
def test_paged_cache_has_the_bits_of_the_dense_cache(dtype, hq, hkv, d):
    """Pages handed out in a random order: the result equals the dense kernel's on the same keys bit for
    bit (same plan, same summation order) and the oracle's within tolerance.  Ragged lengths incl. empty,
    one key, a page boundary, one past it; default plan, a forced split count (static plan) and the
    two-kernel merge."""
    rng = np.random.default_rng(hq * 13 + d)
    lens = np.array([3000, 0, 1, 128, 129, 2047, 777], np.int32)
    B, Lmax = len(lens), 3000
    q = rng.standard_normal((B, hq, d)).astype(np.float32).astype(dtype)
    k = rng.standard_normal((B, hkv, Lmax, d)).astype(np.float32).astype(dtype)
    v = rng.standard_normal((B, hkv, Lmax, d)).astype(np.float32).astype(dtype)
    kp, vp, table, n_pages, max_pages = _paged_from_dense(k, v, lens, 5)
    want = port.gqa_decode_cache_native(q, k, v, lens)
    bits = np.uint16 if dtype == np.float16 else np.uint32
    tol = TOL16 if dtype == np.float16 else TOL32
    l = lib()
    try:
        for tune in ((0, 0), (0, 3), (-1, 3), (0, 1)):
            l.axhip_gqa_decode_tune(*tune)
            if hq // hkv >= 4:
                l.axhip_gqa_decode_tune(tune[0], tune[1] + 1000)   # dense on the vector path too: same arithmetic
            dense = gqa_decode(q, k, v, lens)
            paged = _gqa_paged(q, kp, vp, table, lens, Lmax)
            np.testing.assert_array_equal(paged.view(bits), dense.view(bits), err_msg=str(tune))
            assert np.abs(paged.astype(np.float32) - want).max() <= tol, tune
            assert np.all(paged[1] == 0)
    finally:
        l.axhip_gqa_decode_tune(0, 0)


@pytest.mark.parametrize("Hq,Hkv,D", [(4, 2, 128), (16, 4, 128), (8, 1, 64), (32, 2, 128)])
def test_decode_step_form_over_pages_has_the_bits_of_the_dense_cache(Hq, Hkv, D):
    """axhip_gqa_decode_qkv_paged against axhip_gqa_decode_qkv on the same keys (two query heads per kv head: the
    vector kernel; four and more: the matrix-core kernel): same output bits, the new token's row lands in its page
    with the bits the dense cache gets, every other byte of the pools stays as it was."""
    rng = np.random.default_rng(Hq * 1000 + Hkv * 10 + D)
    lens = np.array([0, 1, 127, 128, 129, 700, 1279, 300], np.int32)
    B, rows = len(lens), 1280
    width = (Hq + 2 * Hkv) * D
    qkv = rng.standard_normal((B, width)).astype(np.float32)
    qw = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    kw = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    pos = rng.integers(0, 8192, (3, B)).astype(np.int64)
    inv = port.rope_inv_freq(1e6, D)
    hw = 10 if D == 64 else 20
    kc = (0.5 * rng.standard_normal((B, Hkv, rows, D))).astype(np.float16)
    vc = rng.standard_normal((B, Hkv, rows, D)).astype(np.float16)
    kp, vp, table, n_pages, max_pages = _paged_from_dense(kc, vc, lens + 1, 31)  # a page for the new row too
    l = gu.lib()
    dq, dqw, dkw, dp, di, dl = (gu.dev(a) for a in (qkv, qw, kw, pos, inv, lens))
    dkc, dvc, dkp, dvp, dtb = (gu.dev(a) for a in (kc, vc, kp, vp, table))
    out_d, out_p = gu.DeviceBuffer(B * Hq * D * 2), gu.DeviceBuffer(B * Hq * D * 2)
    wsb = l.axhip_gqa_decode_workspace_bytes(B, Hq, Hkv, D, rows)
    ws = gu.DeviceBuffer(max(wsb, 256))
    common = (dq.ptr, width, dq.ptr + Hq * D * 4, width, dq.ptr + (Hq + Hkv) * D * 4, width, dqw.ptr, dkw.ptr, gu.F32,
              1e-6, dp.ptr, di.ptr, hw, hw, dl.ptr)
    gu._run("axhip_gqa_decode_qkv", *common, dkc.ptr, dvc.ptr, out_d.ptr, ws.ptr, wsb, gu.F16, B, Hq, Hkv, D, rows, rows,
            None)
    gu.synchronize()
    gu._run("axhip_gqa_decode_qkv_paged", *common, dkp.ptr, dvp.ptr, dtb.ptr, out_p.ptr, ws.ptr, wsb, gu.F16, B, Hq, Hkv,
            D, rows, max_pages, n_pages, None)
    gu.synchronize()
    np.testing.assert_array_equal(out_p.download(np.uint16, (B, Hq, D)), out_d.download(np.uint16, (B, Hq, D)))
    gk, gv = dkc.download(np.float16, kc.shape), dvc.download(np.float16, vc.shape)
    gkp, gvp = dkp.download(np.float16, kp.shape), dvp.download(np.float16, vp.shape)
    touched = np.zeros(kp.shape, bool)
    for b in range(B):
        pid, r = int(table[b, lens[b] >> 7]), int(lens[b] & 127)
        np.testing.assert_array_equal(gkp[pid, :, r].view(np.uint16), gk[b, :, lens[b]].view(np.uint16))
        np.testing.assert_array_equal(gvp[pid, :, r].view(np.uint16), gv[b, :, lens[b]].view(np.uint16))
        touched[pid, :, r] = True
    np.testing.assert_array_equal(gkp[~touched].view(np.uint16), kp[~touched].view(np.uint16))
    np.testing.assert_array_equal(gvp[~touched].view(np.uint16), vp[~touched].view(np.uint16))


@pytest.mark.parametrize("Hq,Hkv", [(4, 2), (16, 2)])
def test_decode_step_form_over_pages_skips_a_row_whose_page_is_not_in_the_table(Hq, Hkv):
    """A sequence whose pages were given back (table entries -1, length 0) or whose table names a page outside the
    pool, replayed without a new reservation: its new row is not stored anywhere (page 0 and every other byte of the
    pools keep their bits), the other sequences' rows land where their tables say.  Vector and matrix-core kernels."""
    rng = np.random.default_rng(Hq * 100 + Hkv)
    D, rows = 128, 640
    lens = np.array([0, 130, 255, 128, 17], np.int32)
    B = len(lens)
    width = (Hq + 2 * Hkv) * D
    qkv = rng.standard_normal((B, width)).astype(np.float32)
    qw = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    kw = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    pos = rng.integers(0, 8192, (3, B)).astype(np.int64)
    inv = port.rope_inv_freq(1e6, D)
    kc = (0.5 * rng.standard_normal((B, Hkv, rows, D))).astype(np.float16)
    vc = rng.standard_normal((B, Hkv, rows, D)).astype(np.float16)
    kp, vp, table, n_pages, max_pages = _paged_from_dense(kc, vc, lens + 1, 3)
    good = table.copy()
    table[0, :] = -1                       # freed sequence: its row would have gone to page 0 under a clamp
    table[3, 1] = n_pages + 5              # the page of row 128 lies outside the pool
    table[4, 0] = -7
    l = gu.lib()
    dq, dqw, dkw, dp, di, dl = (gu.dev(a) for a in (qkv, qw, kw, pos, inv, lens))
    dkp, dvp, dtb = (gu.dev(a) for a in (kp, vp, table))
    out_p = gu.DeviceBuffer(B * Hq * D * 2)
    wsb = l.axhip_gqa_decode_workspace_bytes(B, Hq, Hkv, D, rows)
    ws = gu.DeviceBuffer(max(wsb, 256))
    gu._run("axhip_gqa_decode_qkv_paged", dq.ptr, width, dq.ptr + Hq * D * 4, width, dq.ptr + (Hq + Hkv) * D * 4, width,
            dqw.ptr, dkw.ptr, gu.F32, 1e-6, dp.ptr, di.ptr, 20, 20, dl.ptr, dkp.ptr, dvp.ptr, dtb.ptr, out_p.ptr, ws.ptr,
            wsb, gu.F16, B, Hq, Hkv, D, rows, max_pages, n_pages, None)
    gu.synchronize()
    gkp, gvp = dkp.download(np.uint16, kp.shape), dvp.download(np.uint16, vp.shape)
    written = np.zeros(kp.shape, bool)
    for b in (1, 2):
        written[int(good[b, lens[b] >> 7]), :, int(lens[b] & 127)] = True
    np.testing.assert_array_equal(gkp[~written], kp.view(np.uint16)[~written])
    np.testing.assert_array_equal(gvp[~written], vp.view(np.uint16)[~written])
    assert np.any(gkp[written] != kp.view(np.uint16)[written])          # sequences 1 and 2 did append
    assert np.all(np.isfinite(out_p.download(np.float16, (B, Hq, D)).astype(np.float32)))


@pytest.mark.parametrize("seed", range(12))
def test_paged_cache_random_configurations(seed):
    """Batch, head counts, head size, capacity, lengths (zeros included), dtype and page order at random: the paged
    kernel against the oracle, and against the dense kernel bit for bit (vector kernel and matrix-core kernel)."""
    rng = np.random.default_rng(77000 + seed)
    B = int(rng.integers(1, 10))
    hkv = int(rng.integers(1, 4))
    group = int(rng.choice([1, 2, 3, 4, 5, 8]))
    d = int(rng.choice([64, 128, 256]))
    lmax = int(rng.choice([1, 17, 130, 700, 2100, 4500]))
    dtype = np.float16 if rng.integers(0, 2) else np.float32
    lens = rng.integers(0, lmax + 1, B).astype(np.int32)
    q = rng.standard_normal((B, hkv * group, d)).astype(np.float32).astype(dtype)
    k = rng.standard_normal((B, hkv, lmax, d)).astype(np.float32).astype(dtype)
    v = rng.standard_normal((B, hkv, lmax, d)).astype(np.float32).astype(dtype)
    kp, vp, table, n_pages, max_pages = _paged_from_dense(k, v, lens, seed)
    got = _gqa_paged(q, kp, vp, table, lens, lmax).astype(np.float32)
    want = port.gqa_decode_cache(q, k, v, lens)
    tol = TOL16 if dtype == np.float16 else TOL32
    assert np.abs(got - want).max() <= tol, (B, hkv, group, d, lmax, dtype, lens)
    assert np.all(got[lens == 0] == 0)
    np.testing.assert_array_equal(got, gqa_decode(q, k, v, seq_lens=lens).astype(np.float32))


def test_paged_cache_headline_shape_random_pages():
    """B=32, L=8192 fp16 through a random page permutation (2048 pages of 32 KB per kv head): equal to the
    dense kernel bit for bit; sequence 0 against the oracle."""
    rng = np.random.default_rng(808)
    B, Hq, Hkv, D, L = 32, 16, 8, 128, 8192
    lens = np.full(B, L, np.int32)
    q = rng.standard_normal((B, Hq, D)).astype(np.float32).astype(np.float16)
    blk = rng.standard_normal((4, Hkv, L, D)).astype(np.float32).astype(np.float16)
    k = np.concatenate([np.roll(blk, s, axis=2) for s in range(0, 8)], 0)       # 32 distinct sequences from 4 blocks
    v = np.concatenate([np.roll(blk, 64 + s, axis=3) for s in range(0, 8)], 0)
    kp, vp, table, n_pages, _ = _paged_from_dense(k, v, lens, 9, extra_pages=7)
    dense = gqa_decode(q, k, v, lens)
    paged = _gqa_paged(q, kp, vp, table, lens, L)
    np.testing.assert_array_equal(paged.view(np.uint16), dense.view(np.uint16))
    want0 = port.gqa_decode_cache_native(q[:1], k[:1], v[:1])
    assert np.abs(paged[:1].astype(np.float32) - want0).max() <= TOL16


def test_paged_append_is_a_byte_copy_through_the_table():
    rng = np.random.default_rng(77)
    B, S, Hkv, D, P = 3, 5, 2, 64, 128
    n_pages, max_pages = 9, 3
    table = np.array([[4, 0, -1], [7, 2, 8], [1, -1, -1]], np.int32)
    start = np.array([126, 250, 0], np.int32)            # crosses a page boundary; crosses two; stays inside
    kn = rng.integers(0, 65536, (B, S, Hkv, D)).astype(np.uint16).view(np.float16)
    vn = rng.integers(0, 65536, (B, S, Hkv, D)).astype(np.uint16).view(np.float16)
    kp0 = rng.integers(0, 65536, (n_pages, Hkv, P, D)).astype(np.uint16)
    vp0 = rng.integers(0, 65536, (n_pages, Hkv, P, D)).astype(np.uint16)
    dk, dv, dkn, dvn, dtb, dst = (gu.dev(a) for a in (kp0, vp0, kn, vn, table, start))
    gu._run("axhip_kv_append_paged", dkn.ptr, dvn.ptr, dk.ptr, dv.ptr, dtb.ptr, dst.ptr, gu.I32, 2, B, S, Hkv, D,
            max_pages, n_pages, None)
    gu.synchronize()
    wk, wv = kp0.copy(), vp0.copy()
    for b in range(B):
        for t in range(S):
            pos = start[b] + t
            pid = table[b, pos // P]
            wk[pid, :, pos % P] = kn[b, t].view(np.uint16)
            wv[pid, :, pos % P] = vn[b, t].view(np.uint16)
    np.testing.assert_array_equal(dk.download(np.uint16, kp0.shape), wk)
    np.testing.assert_array_equal(dv.download(np.uint16, vp0.shape), wv)
    # a position behind the table and a page number outside the pool are skipped, nothing else is touched
    bad_table = np.array([[4, 0, 99], [7, 2, 8], [1, -1, -1]], np.int32)
    dtb2, dst2 = gu.dev(bad_table), gu.dev(np.array([254, 382, 126], np.int32))
    gu._run("axhip_kv_append_paged", dkn.ptr, dvn.ptr, dk.ptr, dv.ptr, dtb2.ptr, dst2.ptr, gu.I32, 2, B, S, Hkv, D,
            max_pages, n_pages, None)
    gu.synchronize()
    got = dk.download(np.uint16, kp0.shape)
    for t in range(2):                                   # sequence 0: positions 254, 255 land in page 0; 256.. hit page 99
        wk[0, :, 126 + t] = kn[0, t].view(np.uint16)
    for t in range(2):                                   # sequence 1: positions 382, 383 in page 8; 384.. are behind the table
        wk[8, :, 126 + t] = kn[1, t].view(np.uint16)
    for t in range(2):                                   # sequence 2: positions 126, 127 in page 1; 128.. have page -1
        wk[1, :, 126 + t] = kn[2, t].view(np.uint16)
    np.testing.assert_array_equal(got, wk)
    l = lib()
    assert l.axhip_gqa_decode_paged(None, None, None, None, None, None, None, 0, 4, 1, 16, 8, 128, 300, 2, 4, None) == 1  # table too short
    assert l.axhip_gqa_decode_paged(None, None, None, None, None, None, None, 0, 4, 1, 16, 8, 128, 256, 2, 4, None) == 7
