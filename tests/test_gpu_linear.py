"""fp16 Linear (x @ W^T + b, fp16 operands, fp32 accumulate on MFMA) against the CPU oracle.

Products of two fp16 values are exact in fp32, so the only difference from the oracle's sequential
fp32 sum is accumulation order; the bound used is 1e-5 + 4 * sqrt(K) * 2^-24 * sum|terms| per
output (fp32 output), and 2e-3 for the fp16-output variant at |out| < 2.
"""
import os

import numpy as np
import pytest

from oracle import port

import gpu_util as gu
import gpu_util as gu_mod

pytestmark = pytest.mark.gpu
G = np.load(os.path.join(os.path.dirname(__file__), "golden", "decode_path_golden.npz"))


def h16(a):
    return np.asarray(a, np.float32).astype(np.float16)


def check_linear(x, w, b=None):
    out = gu.linear_f16(x, w, b)
    x32 = x.astype(np.float16).astype(np.float32)  # fp32 activations are rounded to fp16 first (RNE)
    w32 = w.astype(np.float32)
    want = port.linear(x32, w32, None if b is None else b.astype(np.float32))
    K = x.shape[1]
    mag = np.abs(x32) @ np.abs(w32).T
    bound = 1e-5 + 4 * np.sqrt(K) * 2.0 ** -24 * mag
    err = np.abs(out - want)
    assert np.all(err <= bound), (err.max(), bound.min(), x.shape, w.shape)
    return out


def test_golden_fixture():
    np.testing.assert_allclose(gu.linear_f16(G["lin_x"], G["lin_w"]), G["lin_out"], rtol=0, atol=2e-5)
    np.testing.assert_allclose(gu.linear_f16(G["lin_x"], G["lin_w"], G["lin_b"]), G["lin_out_bias"], rtol=0, atol=2e-5)


@pytest.mark.parametrize("M", [1, 16, 32, 512])
@pytest.mark.parametrize("K,N", [(2048, 2048), (2048, 12288), (6144, 2048)])
def test_config4_shapes(M, K, N):
    rng = np.random.default_rng(M * 7 + K + N)
    x = h16(rng.standard_normal((M, K)))
    w = h16(0.02 * rng.standard_normal((N, K)))
    check_linear(x, w)


@pytest.fixture(scope="module")
def lm_head_weight():
    """The lm_head of the 2B shape: 151936 x 2048 fp16 ~ N(0, 0.02) (622 MB on the device)."""
    rng = np.random.default_rng(99)
    return h16(0.02 * rng.standard_normal((151936, 2048), dtype=np.float32))


def _lm_head_columns(N, step):
    # a regular subsample plus both ends of the matrix (first / last weight-row tiles, N % 256 != 0)
    return np.unique(np.concatenate([np.arange(0, N, step), np.arange(0, 40), np.arange(N - 40, N)]))


@pytest.mark.parametrize("M", [1, 16, 32, 512])
def test_lm_head_every_row_count(M, lm_head_weight):
    """2048 -> 151936 at every row count of the benchmark configuration, row-major and packed weights:
    the oracle on a column subsample (the full CPU product takes minutes), the summation-order bound of
    check_linear, and the two weight layouts bit-identical to each other over the whole output."""
    w = lm_head_weight
    N, K = w.shape
    rng = np.random.default_rng(1000 + M)
    x = h16(rng.standard_normal((M, K)))
    out = gu.linear_f16(x, w)
    assert out.shape == (M, N) and np.isfinite(out).all()
    cols = _lm_head_columns(N, 37 if M <= 32 else 301)
    x32, w32 = x.astype(np.float32), w[cols].astype(np.float32)
    want = port.linear(x32, w32)
    bound = 1e-5 + 4 * np.sqrt(K) * 2.0 ** -24 * (np.abs(x32) @ np.abs(w32).T)
    err = np.abs(out[:, cols] - want)
    assert np.all(err <= bound), (M, float(err.max()))
    packed = gu.linear_f16_packed(x, w)
    err_p = np.abs(packed[:, cols] - want)
    assert np.all(err_p <= bound), (M, float(err_p.max()))
    if M == 16:
        # at this row count the two skinny kernels cut K the same way: the same sums in the same order
        np.testing.assert_array_equal(packed, out)
    else:
        assert np.abs(packed - out).max() <= 2 * float(bound.max())


def _order_bound(x32, w32, K, b32=None):
    mag = np.abs(x32) @ np.abs(w32).T + (0 if b32 is None else np.abs(b32))
    return 1e-5 + 4 * np.sqrt(K) * 2.0 ** -24 * mag


@pytest.mark.parametrize("M", [1, 16, 32])
@pytest.mark.parametrize("K,N", [(2048, 2048), (2048, 12288), (6144, 2048), (2048, 4096)])
def test_packed_weights_config4_shapes(M, K, N):
    """The packed-weight (weight-streaming) kernels at the decode row counts of every narrow benchmark shape -
    among them 2048 -> 12288 without the gate/up layout, which takes three row tiles per workgroup, at M = 32
    with two x row tiles per wavefront - against the oracle, and close to the row-major path."""
    rng = np.random.default_rng(M * 11 + K + N)
    x = h16(rng.standard_normal((M, K)))
    w = h16(0.02 * rng.standard_normal((N, K)))
    out = gu.linear_f16_packed(x, w)
    x32, w32 = x.astype(np.float32), w.astype(np.float32)
    want = port.linear(x32, w32)
    bound = _order_bound(x32, w32, K)
    assert np.all(np.abs(out - want) <= bound), float(np.abs(out - want).max())
    assert np.all(np.abs(out - gu.linear_f16(x, w)) <= 2 * bound)
    # fp32 activations are rounded to fp16 on load: the same bits
    np.testing.assert_array_equal(gu.linear_f16_packed(x32, w), out)


@pytest.mark.parametrize("M,K,N", [(33, 2048, 2048), (64, 6144, 2048), (50, 520, 130), (64, 2048, 2064), (65, 2048, 2048),
                                   (200, 6144, 2048), (100, 1024, 1000), (130, 1536, 4096)])
def test_packed_weights_33_to_64_rows(M, K, N):
    """Narrow matrices keep the weight-streaming kernels up to 64 rows (two blocks of rows); one column
    tile more, or one row more, and the tiled GEMM takes over - for problems this small its form whose
    loads run four K steps ahead (K a multiple of 512).  Same oracle either side of each switch."""
    rng = np.random.default_rng(M + K + N)
    x = h16(rng.standard_normal((M, K)))
    w = h16(0.02 * rng.standard_normal((N, K)))
    out = gu.linear_f16_packed(x, w)
    x32, w32 = x.astype(np.float32), w.astype(np.float32)
    want = port.linear(x32, w32)
    bound = _order_bound(x32, w32, K)
    assert np.all(np.abs(out - want) <= bound)
    # fp32 activations are rounded to fp16 on load: the same values enter the products.  The weight-streaming
    # kernels then sum in the same order (same bits); the tiled GEMM may pick another tile for fp32 x (the form
    # that sums K in two halves takes fp16 x only), i.e. another order within the same bound
    out32 = gu.linear_f16_packed(x32, w)
    if M <= 64 and N <= 2048:
        np.testing.assert_array_equal(out32, out)
    else:
        assert np.all(np.abs(out32 - want) <= bound)


@pytest.mark.parametrize("nt", [1, 2, 3, 4])
@pytest.mark.parametrize("M,K,N,glu", [(16, 2048, 1232, False), (32, 1024, 800, False), (7, 520, 130, False),
                                       (32, 2048, 1216, True), (16, 512, 160, True), (32, 6144, 2048, False)])
def test_packed_skinny_every_row_tile_count(nt, M, K, N, glu):
    """One to four 16-row weight tiles per workgroup, forced, on column counts whose tile number is not a multiple of
    the forced count (the last workgroup has absent tiles), with one and two x row tiles per wavefront and with the
    gate/up layout: against the oracle, and the same bits whatever the tile count (four K slices per workgroup in every case)."""
    rng = np.random.default_rng(nt * 1000 + M + K + N)
    x = h16(rng.standard_normal((M, K)))
    w = h16(0.03 * rng.standard_normal((N, K)))
    b = None if glu else h16(0.05 * rng.standard_normal(N))
    l = gu.lib()
    l.axhip_linear_f16_tune(0, nt, 4, 0)
    try:
        out = gu.linear_f16_packed(x, w, b, glu=glu)
        out16 = gu.linear_f16_packed(x, w, b, out_dtype=np.float16, glu=glu)
    finally:
        l.axhip_linear_f16_tune(0, 0, 0, 0)
    l.axhip_linear_f16_tune(0, 1, 4, 0)
    try:
        base = gu.linear_f16_packed(x, w, b, glu=glu)
    finally:
        l.axhip_linear_f16_tune(0, 0, 0, 0)
    np.testing.assert_array_equal(out, base)
    x32, w32 = x.astype(np.float32), w.astype(np.float32)
    if glu:
        full = port.linear(x32, w32)
        want = port.silu_mul(np.ascontiguousarray(full[:, : N // 2]), np.ascontiguousarray(full[:, N // 2:]))
        # the reordered sums of the two projections (a few 1e-6 at K = 2048) carried through silu(g) * u
        np.testing.assert_allclose(out, want, rtol=2e-5, atol=2e-5)
    else:
        want = port.linear(x32, w32, b.astype(np.float32))
        assert np.all(np.abs(out - want) <= _order_bound(x32, w32, K, b.astype(np.float32)))
    ulp = np.spacing(np.abs(want).astype(np.float16)).astype(np.float32)
    assert np.all(np.abs(out16.astype(np.float32) - want) <= 0.5 * ulp + 2e-5 + 4 * np.sqrt(K) * 2.0 ** -24 * 64)


def test_fp32_activations_bias_odd_shapes():
    """Row-major weights: fp32 activations (what the reference's Linear.forward passes,
    src/ops/cuda/linear.cu:108-111), bias, shapes that are multiples of nothing but K % 8."""
    rng = np.random.default_rng(5)
    for (M, K, N) in [(8, 64, 32), (3, 72, 50), (17, 136, 33), (33, 520, 130), (130, 264, 190)]:
        x = rng.standard_normal((M, K)).astype(np.float32)
        w = h16(0.05 * rng.standard_normal((N, K)))
        b = h16(0.05 * rng.standard_normal(N))
        check_linear(x, w, b)
        check_linear(x, w)


def test_fp16_output_variant():
    rng = np.random.default_rng(6)
    x = h16(rng.standard_normal((16, 2048)))
    w = h16(0.02 * rng.standard_normal((2048, 2048)))
    out16 = gu.linear_f16(x, w, out_dtype=np.float16)
    x32, w32 = x.astype(np.float32), w.astype(np.float32)
    want = port.linear(x32, w32)
    ulp = np.spacing(np.abs(want).astype(np.float16)).astype(np.float32)
    assert np.all(np.abs(out16.astype(np.float32) - want) <= 0.5 * ulp + _order_bound(x32, w32, 2048))


def test_matches_fp32_linear_loosely_like_reference_test():
    """tests/core/test_fp16.py:28-46 of the reference: fp16 Linear against fp32 Linear at 5e-2."""
    rng = np.random.default_rng(1)
    x = rng.normal(size=(8, 64)).astype(np.float32)
    w = (rng.normal(size=(32, 64)) * 0.05).astype(np.float32)
    b = (rng.normal(size=(32,)) * 0.05).astype(np.float32)
    out = gu.linear_f16(x, h16(w), h16(b))
    np.testing.assert_allclose(out, x @ w.T + b, rtol=5e-2, atol=5e-2)
    np.testing.assert_allclose(gu.linear_f16_packed(x, h16(w), h16(b)), x @ w.T + b, rtol=5e-2, atol=5e-2)


def test_error_codes():
    l = gu.lib()
    assert l.axhip_linear_f16(None, 4, None, None, None, 5, 4, 60, 8, None, 0, None) == 1  # K % 8
    assert l.axhip_linear_f16(None, 2, None, None, None, 5, 4, 64, 8, None, 0, None) == 3  # x dtype
    assert l.axhip_linear_f16(None, 4, None, None, None, 5, 4, 64, 8, None, 0, None) == 7  # null pointers
    assert l.axhip_linear_f16_packed(None, 2, None, None, None, 5, 4, 64, 8, 0, None) == 3
    assert l.axhip_linear_f16_packed(None, 4, None, None, None, 5, 4, 64, 8, 0, None) == 7
    assert l.axhip_linear_f16_packed(None, 4, None, None, None, 5, 4, 64, 40, 1, None) == 1  # gate/up needs N % 32 == 0
    assert l.axhip_linear_f16_pack(None, None, 40, 64, 1, None) == 1


def test_packed_weights_odd_shapes_bias_fp32_x_fp16_out():
    rng = np.random.default_rng(8)
    for (M, K, N) in [(3, 72, 50), (17, 136, 33), (32, 520, 130), (5, 8, 7), (16, 40, 16)]:
        x = rng.standard_normal((M, K)).astype(np.float32)
        w = h16(0.05 * rng.standard_normal((N, K)))
        b = h16(0.05 * rng.standard_normal(N))
        want = port.linear(x.astype(np.float16).astype(np.float32), w.astype(np.float32), b.astype(np.float32))
        np.testing.assert_allclose(gu.linear_f16_packed(x, w, b), want, rtol=0, atol=2e-5)
        o16 = gu.linear_f16_packed(x, w, b, out_dtype=np.float16)
        assert np.abs(o16.astype(np.float32) - want).max() <= 2e-3
    l = gu.lib()
    assert l.axhip_linear_f16_packed(None, 4, None, None, None, 5, 33, 60, 8, 0, None) == 1  # K % 8
    assert l.axhip_linear_f16_packed_bytes(17, 40) == 2 * 2 * 1024


@pytest.mark.parametrize("M,K,I", [(16, 2048, 6144), (1, 2048, 6144), (32, 2048, 6144), (32, 256, 96), (5, 72, 32)])
def test_packed_gate_up_with_silu_mul_epilogue(M, K, I):
    """Fused [gate ; up] projection with the SiLU-mul epilogue against Linear then silu_mul of the oracle."""
    rng = np.random.default_rng(M + K + I)
    x = h16(rng.standard_normal((M, K)))
    w = h16(0.02 * rng.standard_normal((2 * I, K)))
    gu = port.linear(x.astype(np.float32), w.astype(np.float32))
    want = port.silu_mul(np.ascontiguousarray(gu[:, :I]), np.ascontiguousarray(gu[:, I:]))
    got32 = gu_mod.linear_f16_packed(x, w, glu=True)
    assert got32.shape == (M, I)
    np.testing.assert_allclose(got32, want, rtol=0, atol=2e-5)
    got16 = gu_mod.linear_f16_packed(x, w, out_dtype=np.float16, glu=True)
    assert np.abs(got16.astype(np.float32) - want).max() <= 2e-3


@pytest.mark.parametrize("M,K,N", [(512, 2048, 2048), (512, 2048, 12288), (512, 6144, 2048), (33, 72, 50), (130, 264, 190),
                                   (257, 136, 600), (4096, 256, 264)])
def test_packed_gemm_large_M(M, K, N):
    """M > 32 over packed weights (MFMA GEMM, 256 x 128 tiles, XCD-aware tile order)."""
    rng = np.random.default_rng(M + K + N)
    x = h16(rng.standard_normal((M, K)))
    w = h16(0.02 * rng.standard_normal((N, K)))
    b = h16(0.05 * rng.standard_normal(N))
    out = gu.linear_f16_packed(x, w, b)
    want = port.linear(x.astype(np.float32), w.astype(np.float32), b.astype(np.float32))
    mag = np.abs(x.astype(np.float32)) @ np.abs(w.astype(np.float32)).T
    assert np.all(np.abs(out - want) <= 1e-5 + 4 * np.sqrt(K) * 2.0 ** -24 * mag + 1e-3 * 2.0 ** -11)
    x32 = rng.standard_normal((M, K)).astype(np.float32)  # fp32 activations are rounded to fp16 on the way in
    out2 = gu.linear_f16_packed(x32, w)
    want2 = port.linear(x32.astype(np.float16).astype(np.float32), w.astype(np.float32))
    assert np.abs(out2 - want2).max() <= 1e-4


def test_packed_gemm_glu_large_M():
    rng = np.random.default_rng(77)
    M, K, I = 300, 256, 160
    x = h16(rng.standard_normal((M, K)))
    w = h16(0.05 * rng.standard_normal((2 * I, K)))
    gu_ = port.linear(x.astype(np.float32), w.astype(np.float32))
    want = port.silu_mul(np.ascontiguousarray(gu_[:, :I]), np.ascontiguousarray(gu_[:, I:]))
    np.testing.assert_allclose(gu.linear_f16_packed(x, w, glu=True), want, rtol=0, atol=2e-5)
    got16 = gu.linear_f16_packed(x, w, out_dtype=np.float16, glu=True)
    assert np.abs(got16.astype(np.float32) - want).max() <= 2e-3


@pytest.mark.parametrize("tiles", [1, 2, 4])
def test_packed_gemm_row_tiles_per_wavefront(tiles):
    """The GEMM's weight-row tile (64, 128 or 256 rows per workgroup; chosen by problem size) forced to each
    height on one ragged shape: same bits from all three (K is summed in the same order), bias, and the
    gate/up layout where a wavefront holds a gate tile and its up tile."""
    rng = np.random.default_rng(5)
    M, K, N = 300, 264, 600
    x = h16(rng.standard_normal((M, K)))
    w = h16(0.05 * rng.standard_normal((N, K)))
    b = h16(0.05 * rng.standard_normal(N))
    l = gu.lib()
    base = gu.linear_f16_packed(x, w, b)
    l.axhip_linear_f16_tune(0, 0, 0, 1000 * tiles + 64)
    try:
        out = gu.linear_f16_packed(x, w, b)
        glu = gu.linear_f16_packed(x, w[:576], glu=True) if tiles >= 2 else None
    finally:
        l.axhip_linear_f16_tune(0, 0, 0, 0)
    np.testing.assert_array_equal(out, base)
    want = port.linear(x.astype(np.float32), w.astype(np.float32), b.astype(np.float32))
    mag = np.abs(x.astype(np.float32)) @ np.abs(w.astype(np.float32)).T
    assert np.all(np.abs(out - want) <= 1e-5 + 4 * np.sqrt(K) * 2.0 ** -24 * mag + 1e-3 * 2.0 ** -11)
    if glu is not None:
        gu_ = port.linear(x.astype(np.float32), w[:576].astype(np.float32))
        wantg = port.silu_mul(np.ascontiguousarray(gu_[:, :288]), np.ascontiguousarray(gu_[:, 288:]))
        np.testing.assert_allclose(glu, wantg, rtol=0, atol=2e-5)


@pytest.mark.parametrize("M,K,N", [(128, 128, 256), (700, 384, 520), (1000, 2048, 768)])
def test_packed_gemm_256x128_tile(M, K, N):
    """The 256 x 128 tile (two workgroups per CU, W fragments held two chunks ahead), forced on small shapes:
    M and N that are not multiples of the tile, bias, fp16 output, the gate/up layout; same bits as the
    64-row tile (K is summed in the same order)."""
    rng = np.random.default_rng(M + K + N)
    x = h16(rng.standard_normal((M, K)))
    w = h16(0.02 * rng.standard_normal((N, K)))
    b = h16(0.05 * rng.standard_normal(N))
    l = gu.lib()
    l.axhip_linear_f16_tune(0, 0, 0, 64)
    try:
        base = gu.linear_f16_packed(x, w, b)
    finally:
        l.axhip_linear_f16_tune(0, 0, 0, 0)
    l.axhip_linear_f16_tune(0, 0, 0, 256)
    try:
        out = gu.linear_f16_packed(x, w, b)
        out16 = gu.linear_f16_packed(x, w, b, out_dtype=np.float16)
        n2 = N // 32 * 32
        glu = gu.linear_f16_packed(x, w[:n2], glu=True)
    finally:
        l.axhip_linear_f16_tune(0, 0, 0, 0)
    np.testing.assert_array_equal(out, base)
    want = port.linear(x.astype(np.float32), w.astype(np.float32), b.astype(np.float32))
    mag = np.abs(x.astype(np.float32)) @ np.abs(w.astype(np.float32)).T
    assert np.all(np.abs(out - want) <= 1e-5 + 4 * np.sqrt(K) * 2.0 ** -24 * mag + 1e-3 * 2.0 ** -11)
    assert np.abs(out16.astype(np.float32) - want).max() <= 2e-3
    gu_ = port.linear(x.astype(np.float32), w[:n2].astype(np.float32))
    wantg = port.silu_mul(np.ascontiguousarray(gu_[:, : n2 // 2]), np.ascontiguousarray(gu_[:, n2 // 2:]))
    np.testing.assert_allclose(glu, wantg, rtol=0, atol=2e-5)


@pytest.mark.parametrize("order", [(0, 0), (1, 16), (4, 4), (8, 8), (2, 32), (16, 1), (3, 5)])
@pytest.mark.parametrize("M,K,N", [(1000, 256, 2100), (2200, 128, 530), (128, 384, 256)])
def test_packed_gemm_tile_order_over_the_xcds(order, M, K, N):
    """The 256 x 128 tile handed to the XCDs in rectangles of A weight-row blocks x B blocks of x rows, every
    rectangle shape forced on grids it does not divide (rectangles that hang over both edges, fewer rectangles than
    XCDs, a single tile): every output element is written exactly once with the bits of the plain order."""
    rng = np.random.default_rng(M + K + N)
    x = h16(rng.standard_normal((M, K)))
    w = h16(0.02 * rng.standard_normal((N, K)))
    b = h16(0.05 * rng.standard_normal(N))
    with gu.linear_tuned(100000, 0, 0, 256):
        plain = gu.linear_f16_packed(x, w, b)
    with gu.linear_tuned(100000 + 256 * order[0] + order[1], 0, 0, 256):
        out = gu.linear_f16_packed(x, w, b)
    np.testing.assert_array_equal(out, plain)
    x32, w32 = x.astype(np.float32), w.astype(np.float32)
    want = port.linear(x32, w32, b.astype(np.float32))
    assert np.all(np.abs(out - want) <= _order_bound(x32, w32, K, b.astype(np.float32)))


def test_packed_gemm_default_order_at_a_prefill_shape():
    """A shape whose default is the rectangle order (x does not fit an XCD's L2): 8192 rows through 2048 -> 4096,
    against the plain order bit for bit and the oracle on a sample of rows."""
    rng = np.random.default_rng(77)
    M, K, N = 8192, 2048, 4096
    x = h16(rng.standard_normal((M, K)))
    w = h16(0.02 * rng.standard_normal((N, K)))
    out = gu.linear_f16_packed(x, w)
    with gu.linear_tuned(100000, 0, 0, 256):
        plain = gu.linear_f16_packed(x, w)
    np.testing.assert_array_equal(out, plain)
    rows = np.unique(np.concatenate([np.arange(0, M, 257), [M - 1]]))
    x32, w32 = x[rows].astype(np.float32), w.astype(np.float32)
    want = port.linear(x32, w32)
    assert np.all(np.abs(out[rows] - want) <= _order_bound(x32, w32, K))


@pytest.mark.parametrize("tiles,M,K,N", [(1, 512, 2048, 2048), (1, 512, 6144, 2048), (2, 512, 2048, 4096), (1, 130, 512, 200),
                                         (2, 333, 1024, 1000), (1, 65, 1536, 64)])
def test_packed_gemm_k_in_two_halves(tiles, M, K, N):
    """The tile for problems that give a CU one tile only (eight wavefronts, K summed in two halves that are
    added at the end), forced on edge shapes and at its own sizes: against the oracle, fp16 output, twice the
    same bits, and the halves really are S(first half) + S(second half) of the sequential kernel."""
    rng = np.random.default_rng(M + K + N)
    x = h16(rng.standard_normal((M, K)))
    w = h16(0.02 * rng.standard_normal((N, K)))
    b = h16(0.05 * rng.standard_normal(N))
    l = gu.lib()
    l.axhip_linear_f16_tune(0, 0, 0, 1000 * tiles + 512)
    try:
        out = gu.linear_f16_packed(x, w, b)
        again = gu.linear_f16_packed(x, w, b)
        out16 = gu.linear_f16_packed(x, w, b, out_dtype=np.float16)
    finally:
        l.axhip_linear_f16_tune(0, 0, 0, 0)
    np.testing.assert_array_equal(out, again)
    want = port.linear(x.astype(np.float32), w.astype(np.float32), b.astype(np.float32))
    mag = np.abs(x.astype(np.float32)) @ np.abs(w.astype(np.float32)).T
    assert np.all(np.abs(out - want) <= 1e-5 + 4 * np.sqrt(K) * 2.0 ** -24 * mag + 1e-3 * 2.0 ** -11)
    assert np.abs(out16.astype(np.float32) - want).max() <= 2e-3 + 2.0 ** -11 * np.abs(want).max()
    # the two halves, each from the sequential kernel (64-row tile), added in fp32 and then the bias
    l.axhip_linear_f16_tune(0, 0, 0, 64)
    try:
        s0 = gu.linear_f16_packed(np.ascontiguousarray(x[:, : K // 2]), np.ascontiguousarray(w[:, : K // 2]))
        s1 = gu.linear_f16_packed(np.ascontiguousarray(x[:, K // 2:]), np.ascontiguousarray(w[:, K // 2:]))
    finally:
        l.axhip_linear_f16_tune(0, 0, 0, 0)
    np.testing.assert_array_equal(out, (s0 + s1) + b.astype(np.float32))


@pytest.mark.parametrize("seed", range(16))
def test_packed_linear_random_shapes(seed):
    """Rows, K (a multiple of 8), columns, bias, activation dtype and output dtype at random: every route
    (weight-streaming kernels, tiled GEMMs of every tile size, their edge handling) against the oracle."""
    rng = np.random.default_rng(9500 + seed)
    M = int(rng.choice([1, 5, 16, 31, 32, 33, 64, 65, 130, 300, 520]))
    K = 8 * int(rng.integers(1, 200))
    if rng.integers(0, 3) == 0:
        K = 128 * int(rng.integers(1, 17))
    N = int(rng.choice([1, 7, 16, 50, 64, 257, 700, 2048, 2300]))
    x = rng.standard_normal((M, K)).astype(np.float32)
    if rng.integers(0, 2):
        x = h16(x)
    w = h16(0.05 * rng.standard_normal((N, K)))
    b = h16(0.05 * rng.standard_normal(N)) if rng.integers(0, 2) else None
    xr = x.astype(np.float16).astype(np.float32)
    want = port.linear(xr, w.astype(np.float32), None if b is None else b.astype(np.float32))
    mag = np.abs(xr) @ np.abs(w.astype(np.float32)).T + (0 if b is None else np.abs(b.astype(np.float32)))
    got = gu.linear_f16_packed(x, w, b)
    assert np.all(np.abs(got - want) <= 1e-5 + 4 * np.sqrt(K) * 2.0 ** -24 * mag), (M, K, N)
    got16 = gu.linear_f16_packed(x, w, b, out_dtype=np.float16).astype(np.float32)
    ulp = np.spacing(np.abs(want).astype(np.float16)).astype(np.float32)
    assert np.all(np.abs(got16 - want) <= 0.5 * ulp + 1e-5 + 4 * np.sqrt(K) * 2.0 ** -24 * mag), (M, K, N)


# ---- fp32 weights: a Linear that has not been cast (src/ops/cuda/linear.cu:178-251) ------------------------------
def linear_f32(x, w, b=None):
    M, K = x.shape
    N = w.shape[0]
    dx, dw = gu.dev(x), gu.dev(w)
    db = gu.dev(b) if b is not None else None
    do = gu.DeviceBuffer(M * N * 4)
    gu._run("axhip_linear_f32", dx.ptr, dw.ptr, db.ptr if db else None, do.ptr, M, K, N, None)
    gu.synchronize()
    return do.download(np.float32, (M, N))


@pytest.mark.parametrize("M,K,N", [(8, 64, 32), (1, 2048, 2048), (16, 2048, 4096), (3, 72, 50), (130, 264, 190),
                                   (65, 37, 129), (512, 1024, 300), (64, 32, 64)])
def test_linear_f32_against_the_oracle(M, K, N):
    """fp32 x, W and bias: fp32 products summed in K order, so against the oracle's sequential fp32 sum only
    the rounding of partial sums differs: 1e-5 + 8 sqrt(K) 2^-24 sum|terms| (products are no longer exact as
    in the fp16 case, hence the factor 8 where the fp16 tests have 4).  K = 37 takes the scalar loads."""
    rng = np.random.default_rng(M * 3 + K + N)
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = (0.05 * rng.standard_normal((N, K))).astype(np.float32)
    b = (0.05 * rng.standard_normal(N)).astype(np.float32)
    want = port.linear(x, w, b)
    bound = 1e-5 + 8 * np.sqrt(K) * 2.0 ** -24 * (np.abs(x) @ np.abs(w).T + np.abs(b))
    got = linear_f32(x, w, b)
    assert np.all(np.abs(got - want) <= bound), float(np.abs(got - want).max())
    got0 = linear_f32(x, w)
    assert np.all(np.abs(got0 - port.linear(x, w)) <= bound)
    l = gu.lib()
    assert l.axhip_linear_f32(None, None, None, None, 4, 0, 8, None) == 1
    assert l.axhip_linear_f32(None, None, None, None, 4, 8, 8, None) == 7
    assert l.axhip_linear_f32(None, None, None, None, 0, 8, 8, None) == 0
