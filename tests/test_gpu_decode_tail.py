"""axhip_decode_layer_tail (o_proj + residual, norm, gate/up + SiLU-mul, down_proj + residual, norm and the next
layer's q/k/v Linear in one persistent launch) against the CPU oracle's single operators with the same fp16
storage points: the activation entering each Linear and `act` are fp16, everything else fp32.  Tolerances: the
residual stream differs by fp32 summation order and, behind a norm, by activations that round to the neighbouring
fp16 value (1e-3 in all; values up to 14); and, tighter, the device may be no
farther from the same composition evaluated in float64 (same storage points) than 1.5 x what the fp32 oracle is."""
import ctypes as C

import numpy as np
import pytest

import gpu_util as gu
from oracle import port
from oracle.f64_ops import F64Ops

pytestmark = pytest.mark.gpu


def h16(a):
    return np.asarray(a, np.float32).astype(np.float16)


def _pack(w, glu=False):
    l = gu.lib()
    n, k = w.shape
    dw = gu.dev(w)
    p = gu.DeviceBuffer(l.axhip_linear_f16_packed_bytes(n, k))
    gu._run("axhip_linear_f16_pack", dw.ptr, p.ptr, n, k, int(glu), None)
    gu.synchronize()
    return p


def _oracle(attn, h_in, wo, w_post, wgu, wd, w_next, wn, eps, ops=port, f=np.float32):
    """The composition with the oracle's operators (ops=port, fp32) or in float64 (ops=F64Ops(), f=np.float64)."""
    c = lambda a: np.asarray(a, f)
    inter = wd.shape[1]
    h_mid = ops.linear(c(attn), c(wo)) + c(h_in)
    xn2 = c(h16(ops.rms_norm(h_mid, w_post, eps)))
    gu_ = ops.linear(xn2, c(wgu))
    act = h16(ops.silu_mul(np.ascontiguousarray(gu_[:, :inter]), np.ascontiguousarray(gu_[:, inter:])))
    h_out = ops.linear(c(act), c(wd)) + h_mid
    xn = c(h16(ops.rms_norm(h_out, w_next, eps)))
    return h_out, ops.linear(xn, c(wn))


@pytest.mark.parametrize("M,H,K1,I,N_next", [(16, 512, 512, 1024, 512), (5, 512, 512, 1024, 1024), (1, 512, 512, 1024, 16),
                                             (16, 2048, 2048, 6144, 4096), (7, 2048, 2048, 6144, 4096)])
def test_layer_tail_matches_operator_composition(M, H, K1, I, N_next):
    rng = np.random.default_rng(100 + M + H)
    eps = 1e-6
    attn = h16(rng.standard_normal((M, K1)))
    h_in = rng.standard_normal((M, H)).astype(np.float32) * 3
    wo, wd, wn = (h16(0.02 * rng.standard_normal(s)) for s in ((H, K1), (H, I), (N_next, H)))
    wgu = h16(0.02 * rng.standard_normal((2 * I, H)))
    w_post = (1 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    w_next = (1 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    l = gu.lib()
    d_wp, d_wn = gu.dev(w_post), gu.dev(w_next)
    p_o, p_gu, p_d, p_n = _pack(wo), _pack(wgu, glu=True), _pack(wd), _pack(wn)
    wsb = l.axhip_decode_layer_tail_workspace_bytes(H, I)
    ws = gu.DeviceBuffer(wsb)
    h_out, y = (gu.DeviceBuffer(n) for n in (M * H * 4, M * N_next * 4))
    failed = C.c_uint(0)
    assert l.axhip_decode_layer_tail_status(1, C.byref(failed)) == 0
    for it in range(3):   # the barrier state must be clean again after every launch; new inputs every time, so that
        # a block served from a cache line of the launch before would be a wrong value
        attn_i = h16(attn * (1.0 + 0.5 * it))
        h_i = (h_in * (1.0 - 0.3 * it)).astype(np.float32)
        want = _oracle(attn_i, h_i, wo, w_post, wgu, wd, w_next, wn, eps)
        exact = _oracle(attn_i, h_i, wo, w_post, wgu, wd, w_next, wn, eps, ops=F64Ops(), f=np.float64)
        d_attn, d_h = gu.dev(attn_i), gu.dev(h_i)
        print(f"tail M={M} H={H} I={I} N_next={N_next} launch {it}", flush=True)
        gu._run("axhip_decode_layer_tail", d_attn.ptr, d_h.ptr, p_o.ptr, d_wp.ptr, p_gu.ptr, p_d.ptr, d_wn.ptr,
                p_n.ptr, h_out.ptr, y.ptr, ws.ptr, wsb, M, H, K1, I, N_next, eps, None)
        gu.synchronize()
        assert l.axhip_decode_layer_tail_status(0, C.byref(failed)) == 0 and failed.value == 0
        got = (h_out.download(np.float32, (M, H)), y.download(np.float32, (M, N_next)))
        for name, g_, w_, e_ in (("h_out", got[0], want[0], exact[0]), ("y", got[1], want[1], exact[1])):
            err = np.abs(g_ - w_)
            d_dev, d_cpu = float(np.abs(g_ - e_).max()), float(np.abs(w_ - e_).max())
            print(f"  {name}: max abs err {float(err.max()):.3e} (max |value| {float(np.abs(w_).max()):.3f}); against float64: "
                  f"device {d_dev:.3e}, fp32 oracle {d_cpu:.3e}", flush=True)
            # a few activations that round to the other fp16 neighbour behind a norm (each moves a sum by about
            # 2^-11 x |activation| x |weight| <= 2e-4): 1e-3 holds with a factor of two to spare at the large widths
            assert float(err.max()) <= 1e-3, (name, float(err.max()))
            # no farther from the float64 evaluation than 1.5 x the fp32 oracle (floor: what one activation that rounds
            # to the other fp16 neighbour moves a sum, 2^-11 x |activation| x |weight| ~ 5e-4 x 4 x 0.08)
            assert d_dev <= max(1.5 * d_cpu, 2e-4), (name, d_dev, d_cpu)
        # poison the outputs so that a launch that did nothing cannot pass
        for b in (h_out, y):
            b.upload(np.full(b.nbytes // 4, np.nan, np.float32))


@pytest.mark.parametrize("M,H,K1,I", [(16, 512, 512, 1024), (3, 512, 512, 1024), (16, 2048, 2048, 6144), (9, 2048, 2048, 6144)])
def test_last_layer_form_ends_with_the_final_norm(M, H, K1, I):
    """axhip_decode_layer_tail_last: h_out has the bits of the launch with a projection behind it (same phases 1-3),
    and xn is the RMSNorm of exactly that h_out, rounded once to fp16 (the norm's sum runs over per-unit partial sums:
    1 ulp of fp16 where the fp32 value sits next to a rounding boundary)."""
    rng = np.random.default_rng(300 + M + H)
    eps = 1e-6
    attn = h16(rng.standard_normal((M, K1)))
    h_in = rng.standard_normal((M, H)).astype(np.float32) * 3
    wo, wd, wn = (h16(0.02 * rng.standard_normal(s)) for s in ((H, K1), (H, I), (64, H)))
    wgu = h16(0.02 * rng.standard_normal((2 * I, H)))
    w_post = (1 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    w_fin = (1 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    l = gu.lib()
    assert l.axhip_decode_layer_tail_supported(M, H, K1, I, 0) == 1
    d_attn, d_h, d_wp, d_wf = (gu.dev(a) for a in (attn, h_in, w_post, w_fin))
    p_o, p_gu, p_d, p_n = _pack(wo), _pack(wgu, glu=True), _pack(wd), _pack(wn)
    wsb = l.axhip_decode_layer_tail_workspace_bytes(H, I)
    ws = gu.DeviceBuffer(wsb)
    h_a, h_b, y, xn = (gu.DeviceBuffer(n) for n in (M * H * 4, M * H * 4, M * 64 * 4, M * H * 2))
    failed = C.c_uint(0)
    assert l.axhip_decode_layer_tail_status(1, C.byref(failed)) == 0
    print(f"tail M={M} H={H}: with a projection behind it", flush=True)
    gu._run("axhip_decode_layer_tail", d_attn.ptr, d_h.ptr, p_o.ptr, d_wp.ptr, p_gu.ptr, p_d.ptr, d_wf.ptr, p_n.ptr,
            h_a.ptr, y.ptr, ws.ptr, wsb, M, H, K1, I, 64, eps, None)
    gu.synchronize()
    for it in range(2):
        xn.upload(np.full(M * H // 2, np.nan, np.float32))
        print(f"tail M={M} H={H}: last-layer form, launch {it}", flush=True)
        gu._run("axhip_decode_layer_tail_last", d_attn.ptr, d_h.ptr, p_o.ptr, d_wp.ptr, p_gu.ptr, p_d.ptr, d_wf.ptr, h_b.ptr,
                xn.ptr, ws.ptr, wsb, M, H, K1, I, eps, None)
        gu.synchronize()
        assert l.axhip_decode_layer_tail_status(0, C.byref(failed)) == 0 and failed.value == 0
        ha, hb = h_a.download(np.float32, (M, H)), h_b.download(np.float32, (M, H))
        np.testing.assert_array_equal(ha.view(np.uint32), hb.view(np.uint32))
        got = xn.download(np.float16, (M, H))
        want = port.rms_norm(hb, w_fin, eps)
        assert np.all(np.isfinite(got))
        ulp = np.spacing(np.abs(want).astype(np.float16)).astype(np.float32)
        assert np.all(np.abs(got.astype(np.float32) - want) <= 0.5 * ulp + 2e-6 * np.abs(want) + 1e-7)
    # against the oracle's whole composition as well (a few fp16 flips behind the first norm: the bound of the test above)
    ref_h, _ = _oracle(attn, h_in, wo, w_post, wgu, wd, w_fin, wn, eps)
    assert float(np.abs(hb - ref_h).max()) <= 1e-3
    assert l.axhip_decode_layer_tail_last(d_attn.ptr, d_h.ptr, p_o.ptr, d_wp.ptr, p_gu.ptr, p_d.ptr, d_wf.ptr, h_b.ptr,
                                          None, ws.ptr, wsb, M, H, K1, I, eps, None) == 7


def test_layer_tail_argument_checks():
    l = gu.lib()
    b = gu.DeviceBuffer(1 << 22)
    big = 1 << 22
    args = [b.ptr] * 9 + [b.ptr + 4096, b.ptr, big]      # h_out differs from h_in
    assert l.axhip_decode_layer_tail(*args, 17, 2048, 2048, 6144, 4096, 1e-6, None) == 1   # more than 16 rows
    assert l.axhip_decode_layer_tail(*args, 16, 1024, 2048, 6144, 4096, 1e-6, None) == 1   # widths it is not built for
    assert l.axhip_decode_layer_tail(*args, 16, 2048, 2048, 6144, 4100, 1e-6, None) == 1   # N_next not whole tiles
    assert l.axhip_decode_layer_tail(*args, 16, 2048, 2048, 6144, 8192, 1e-6, None) == 1   # more tiles than workgroups
    assert l.axhip_decode_layer_tail(*([None] + args[1:]), 16, 2048, 2048, 6144, 4096, 1e-6, None) == 7
    same = [b.ptr] * 11 + [big]
    assert l.axhip_decode_layer_tail(*same, 16, 2048, 2048, 6144, 4096, 1e-6, None) == 1   # h_out is h_in
    assert l.axhip_decode_layer_tail(*args[:11], 1024, 16, 2048, 2048, 6144, 4096, 1e-6, None) == 1   # workspace too small
    assert l.axhip_decode_layer_tail(*args, 0, 2048, 2048, 6144, 4096, 1e-6, None) == 0
    assert l.axhip_decode_layer_tail(*args, 16, 2048, 2048, 6144, 0, 1e-6, None) == 1      # no projection: the _last form
    # the question a caller asks before it chooses between this launch and the single operators
    assert l.axhip_decode_layer_tail_supported(16, 2048, 2048, 6144, 4096) == 1
    assert l.axhip_decode_layer_tail_supported(16, 512, 512, 1024, 48) == 1
    assert l.axhip_decode_layer_tail_supported(17, 2048, 2048, 6144, 4096) == 0
    assert l.axhip_decode_layer_tail_supported(16, 1024, 1024, 3072, 2048) == 0
    assert l.axhip_decode_layer_tail_supported(16, 2048, 2048, 6144, 8192) == 0


def test_a_wait_that_runs_out_is_counted_and_later_launches_give_up_at_once_until_the_reset():
    """The barrier's wait is bounded.  Forced from the host (a spin limit of one look): the launch ends by itself,
    the failure is counted, the next launch - with the normal limit - gives up at its first barrier instead of
    spinning on counters in disorder, and after the reset a launch is correct again."""
    rng = np.random.default_rng(7)
    M, H, K1, I, N_next, eps = 16, 512, 512, 1024, 256, 1e-6
    attn = h16(rng.standard_normal((M, K1)))
    h_in = rng.standard_normal((M, H)).astype(np.float32)
    wo, wd, wn = (h16(0.02 * rng.standard_normal(s)) for s in ((H, K1), (H, I), (N_next, H)))
    wgu = h16(0.02 * rng.standard_normal((2 * I, H)))
    ones = np.ones(H, np.float32)
    want = _oracle(attn, h_in, wo, ones, wgu, wd, ones, wn, eps)
    l = gu.lib()
    d_attn, d_h, d_w = gu.dev(attn), gu.dev(h_in), gu.dev(ones)
    p_o, p_gu, p_d, p_n = _pack(wo), _pack(wgu, glu=True), _pack(wd), _pack(wn)
    wsb = l.axhip_decode_layer_tail_workspace_bytes(H, I)
    ws = gu.DeviceBuffer(wsb)
    h_out, y = (gu.DeviceBuffer(n) for n in (M * H * 4, M * N_next * 4))
    failed = C.c_uint(0)
    assert l.axhip_decode_layer_tail_status(1, C.byref(failed)) == 0

    def launch():
        gu._run("axhip_decode_layer_tail", d_attn.ptr, d_h.ptr, p_o.ptr, d_w.ptr, p_gu.ptr, p_d.ptr, d_w.ptr, p_n.ptr,
                h_out.ptr, y.ptr, ws.ptr, wsb, M, H, K1, I, N_next, eps, None)
        gu.synchronize()
        assert l.axhip_decode_layer_tail_status(0, C.byref(failed)) == 0
        return failed.value

    try:
        l.axhip_decode_layer_tail_tune(256)
        print("tail: launch with a spin limit of one look", flush=True)
        first = launch()
        assert first > 0
        l.axhip_decode_layer_tail_tune(0)
        print("tail: launch on the state that launch left behind", flush=True)
        assert launch() == first            # gave up at once: no new wait ran out, nothing was waited for
    finally:
        l.axhip_decode_layer_tail_tune(0)
        assert l.axhip_decode_layer_tail_status(1, C.byref(failed)) == 0
    print("tail: launch after the reset", flush=True)
    assert launch() == 0
    np.testing.assert_allclose(y.download(np.float32, (M, N_next)), want[1], rtol=0, atol=2e-3)
