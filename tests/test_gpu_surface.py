"""The Python surface on the hip device: the reference's own test cases for the decode path,
re-stated (tests/core/test_fused.py, test_gqa.py, test_sequence_ops.py, test_fp16.py,
test_cuda_graph.py, tests/nn/test_kv_cache.py of the reference), plus compile() and the allocator.
Expected values come from the CPU oracle / NumPy closed forms."""
import math

import numpy as np
import pytest

import axono_amd as axono
from axono_amd import DataType, Tensor, nn
from axono_amd import libaxono as L
from oracle import port

pytestmark = pytest.mark.gpu

DEV = "hip:0"


def t(arr, device=DEV):
    return Tensor.from_numpy(np.ascontiguousarray(arr)).to(device)


def ids_t(arr, device=DEV):
    x = Tensor.zeros(tuple(np.asarray(arr).shape), dtype=DataType.INT64, device=device)
    x.copy_from_numpy(np.asarray(arr, dtype=np.int64))
    return x


@pytest.fixture
def hip_env():
    axono.set_backend("hip")
    yield
    axono.set_backend("cpu")


def test_tensor_device_round_trip_and_zero_init(hip_env):
    assert axono.hip_available()
    z = Tensor(DataType.FLOAT32, [3, 5], "hip:0")
    assert np.all(z.to_numpy() == 0) and z.is_hip and not z.is_cuda
    x = np.random.default_rng(0).standard_normal((4, 7)).astype(np.float32)
    d = Tensor.from_numpy(x)  # default device is hip inside hip_env
    assert d.device == "hip"
    np.testing.assert_array_equal(d.to_numpy(), x)
    assert d.to("hip") is d and d.to("hip:0") is d
    back = d.to("cpu")
    assert back is not d and back.device == "cpu"
    np.testing.assert_array_equal(back.to_numpy(), x)
    h = d.cast_to(DataType.FLOAT16)
    np.testing.assert_array_equal(h.numpy(), x.astype(np.float16))
    np.testing.assert_array_equal(h.cast_to(DataType.FLOAT32).to_numpy(), x.astype(np.float16).astype(np.float32))
    d.copy_from_numpy(2 * x)
    np.testing.assert_array_equal(d.to_numpy(), 2 * x)
    d.fill_zero()
    assert np.all(d.to_numpy() == 0)
    with pytest.raises(IndexError):
        Tensor(DataType.FLOAT32, [1], "hip:7")


def test_transpose_and_plus_on_the_device():
    """Tensor.transpose / T on hip (axhip_transpose) for every element width and dim pair, and `+`."""
    rng = np.random.default_rng(2)
    a = rng.standard_normal((3, 5, 4, 7)).astype(np.float32)
    d = t(a)
    for d0, d1 in ((0, 1), (0, 3), (1, 2), (2, 3), (1, 3), (-1, -2), (3, 0)):
        np.testing.assert_array_equal(d.transpose(d0, d1).to_numpy(), np.swapaxes(a, d0, d1))
    np.testing.assert_array_equal(t(a[0, 0]).T.to_numpy(), a[0, 0].T)
    h = a.astype(np.float16)
    np.testing.assert_array_equal(t(h).transpose(1, 3).numpy(), np.swapaxes(h, 1, 3))
    i64 = rng.integers(-9, 9, (6, 10)).astype(np.int64)
    np.testing.assert_array_equal(ids_t(i64).T.to_numpy(), i64.T)
    big = rng.standard_normal((1024, 2048)).astype(np.float32)
    np.testing.assert_array_equal(t(big).T.to_numpy(), big.T)
    assert d.transpose(2, 2).data_ptr == d.data_ptr        # equal dims: an alias
    b = rng.standard_normal(a.shape).astype(np.float32)
    np.testing.assert_array_equal((d + t(b)).to_numpy(), a + b)
    np.testing.assert_array_equal(d.data_float32(), a)     # a device tensor's accessor is a host copy
    with pytest.raises(NotImplementedError):
        d * d


def test_fused_ops_reference_cases():
    rs = np.random.RandomState(0)
    g, u = rs.randn(37, 53).astype(np.float32), rs.randn(37, 53).astype(np.float32)
    y = axono.fused.silu_mul(t(g), t(u)).to_numpy()
    np.testing.assert_allclose(y, g / (1.0 + np.exp(-g)) * u, rtol=1e-5, atol=1e-6)
    e = np.array([-10.0, -1.0, 0.0, 1.0, 10.0, 0, 0, 0], np.float32)
    np.testing.assert_allclose(axono.silu_mul(t(e), t(np.ones(8, np.float32))).to_numpy(), e / (1.0 + np.exp(-e)), rtol=1e-5, atol=1e-6)
    rs = np.random.RandomState(1)
    x, r, w = rs.randn(4, 128).astype(np.float32), rs.randn(4, 128).astype(np.float32), rs.randn(128).astype(np.float32)
    yt, out = axono.fused.add_rms_norm(t(x), t(r), t(w), 1e-6)
    s = x + r
    np.testing.assert_allclose(yt.to_numpy(), s, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(out.to_numpy(), s / np.sqrt((s ** 2).mean(-1, keepdims=True) + 1e-6) * w, rtol=1e-4, atol=1e-5)
    # y feeds the next layer's residual
    rs = np.random.RandomState(2)
    h, a1, a2 = (rs.randn(2, 64).astype(np.float32) for _ in range(3))
    w1 = np.ones(64, np.float32)
    h1, _ = axono.add_rms_norm(t(a1), t(h), t(w1), 1e-6)
    h2, _ = axono.add_rms_norm(t(a2), h1, t(w1), 1e-6)
    np.testing.assert_allclose(h2.to_numpy(), a2 + a1 + h, rtol=1e-5, atol=1e-6)
    with pytest.raises(RuntimeError) as ei:
        axono.silu_mul(t(g), t(u[:5]))
    assert "silu_mul 失败, 错误代码: 4" in str(ei.value)


def test_gqa_matches_numpy_and_sdpa_op():
    rs = np.random.RandomState(3)
    for skv in (1, 7, 256, 512, 1024, 3000):
        q = rs.randn(1, 16, 128).astype(np.float32)
        k = rs.randn(skv, 8, 128).astype(np.float32)
        v = rs.randn(skv, 8, 128).astype(np.float32)
        out = axono.gqa_decode_attention(t(q), t(k), t(v))
        assert out.shape == [1, 16, 128]
        np.testing.assert_allclose(out.to_numpy(), port.gqa_decode(q, k, v), rtol=1e-4, atol=1e-4)
    rs = np.random.RandomState(4)
    q, k, v = rs.randn(1, 16, 128).astype(np.float32), rs.randn(300, 8, 128).astype(np.float32), rs.randn(300, 8, 128).astype(np.float32)
    a1 = axono.gqa_decode_attention(t(q), t(k), t(v)).to_numpy()
    a2 = axono.scaled_dot_product_attention(t(q), t(k), t(v), False).to_numpy()
    np.testing.assert_allclose(a1, a2, rtol=1e-4, atol=1e-4)
    with pytest.raises(RuntimeError) as ei:
        axono.gqa_decode_attention(t(np.zeros((2, 16, 128), np.float32)), t(k), t(v))
    assert "错误代码: 1" in str(ei.value)  # decode takes exactly one query token


def test_sequence_ops_reference_cases():
    rs = np.random.RandomState(2027)
    x = rs.randn(4, 2, 8).astype(np.float32)
    out = axono.rope(t(x), ids_t(np.arange(4)), 10000.0).to_numpy()
    np.testing.assert_allclose(out, port.rope(x, np.arange(4), 10000.0), rtol=1e-4, atol=1e-5)
    rng = np.random.default_rng(8)
    pos3 = rng.integers(0, 50, size=(3, 17)).astype(np.int64)
    inv = (1.0 / (5e6 ** (np.arange(0, 128, 2, dtype=np.float32) / 128))).astype(np.float32)
    c, s = axono.mrope_cos_sin(ids_t(pos3), t(inv), 20, 20)
    wc, ws = port.mrope_cos_sin(pos3, inv, 20, 20)
    np.testing.assert_allclose(c.to_numpy(), wc, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(s.to_numpy(), ws, rtol=1e-5, atol=1e-6)
    xr = rng.standard_normal((17, 4, 128)).astype(np.float32)
    np.testing.assert_allclose(axono.rope_thd(t(xr), ids_t(pos3), t(inv), [24, 20, 20]).to_numpy(),
                               port.rope_thd(xr, pos3, inv, [24, 20, 20]), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(axono.rope_with_cos_sin(t(xr), c, s).to_numpy(), port.rope_with_cos_sin(xr, wc, ws), rtol=1e-5, atol=1e-5)
    a, b = rng.standard_normal((2, 3, 4)).astype(np.float32), rng.standard_normal((2, 3, 5)).astype(np.float32)
    np.testing.assert_array_equal(axono.concat(t(a), t(b), -1).to_numpy(), np.concatenate([a, b], -1))
    np.testing.assert_array_equal(axono.concat(t(a), t(a), 0).to_numpy(), np.concatenate([a, a], 0))
    np.testing.assert_array_equal(axono.slice_(t(b), -1, 1, 3).to_numpy(), b[..., 1:4])
    np.testing.assert_array_equal(axono.slice_(t(b), 0, 1, 1).to_numpy(), b[1:2])
    table = rng.standard_normal((10, 4)).astype(np.float32)
    ids = np.array([[1, 3], [5, 2]], np.int64)
    np.testing.assert_array_equal(axono.embedding(ids_t(ids), t(table)).to_numpy(), table[ids])
    lg = rng.standard_normal((3, 100)).astype(np.float32)
    am = axono.argmax(t(lg))
    assert am.dtype == DataType.INT64
    np.testing.assert_array_equal(am.to_numpy(), np.argmax(lg, -1))
    np.testing.assert_array_equal(axono.add(t(a), t(a)).to_numpy(), a + a)
    w = rng.standard_normal(5).astype(np.float32)
    np.testing.assert_allclose(axono.rms_norm(t(b), t(w), 1e-6).to_numpy(), port.rms_norm(b, w, 1e-6), rtol=1e-5, atol=1e-5)


def test_linear_fp16_module_path(hip_env):
    """tests/core/test_fp16.py:28-46 of the reference: nn.Linear after cast_linear_fp16()."""
    rng = np.random.default_rng(1)
    x_np = rng.normal(size=(8, 64)).astype(np.float32)
    w_np = (rng.normal(size=(32, 64)) * 0.05).astype(np.float32)
    b_np = (rng.normal(size=(32,)) * 0.05).astype(np.float32)
    lin = nn.Linear(64, 32, device="hip")
    lin.load_state_dict({"weight": w_np, "bias": b_np})
    lin.cast_linear_fp16()
    assert lin.weight.dtype == DataType.FLOAT16 and lin.weight.is_hip
    out = lin(Tensor.from_numpy(x_np))
    assert out.dtype == DataType.FLOAT32 and out.shape == [8, 32]
    np.testing.assert_allclose(out.to_numpy(), x_np @ w_np.T + b_np, rtol=5e-2, atol=5e-2)
    want = port.linear(x_np.astype(np.float16).astype(np.float32), w_np.astype(np.float16).astype(np.float32),
                       b_np.astype(np.float16).astype(np.float32))
    np.testing.assert_allclose(out.to_numpy(), want, rtol=0, atol=2e-5)
    nb = nn.Linear(64, 32, bias=False, device="hip")
    nb.load_state_dict({"weight": w_np})
    nb.cast_linear_fp16()
    np.testing.assert_allclose(nb(Tensor.from_numpy(x_np)).to_numpy(), want - b_np.astype(np.float16).astype(np.float32), rtol=0, atol=2e-5)


def test_linear_fp32_module_path_before_the_cast(hip_env):
    """nn.Linear as created (FLOAT32 weight and bias): forward runs the fp32 operator, like the reference's Linear
    before cast_linear_fp16() (tests/nn/test_layers.py of the reference compares it with x @ W^T + b)."""
    rng = np.random.default_rng(2)
    x_np = rng.normal(size=(5, 3, 64)).astype(np.float32)
    w_np = (rng.normal(size=(32, 64)) * 0.05).astype(np.float32)
    b_np = (rng.normal(size=(32,)) * 0.05).astype(np.float32)
    lin = nn.Linear(64, 32, device="hip")
    lin.load_state_dict({"weight": w_np, "bias": b_np})
    assert lin.weight.dtype == DataType.FLOAT32
    out = lin(Tensor.from_numpy(x_np))
    assert out.dtype == DataType.FLOAT32 and out.shape == [5, 3, 32]
    want = port.linear(x_np.reshape(15, 64), w_np, b_np).reshape(5, 3, 32)
    np.testing.assert_allclose(out.to_numpy(), want, rtol=0, atol=1e-5)
    nb = nn.Linear(64, 32, bias=False, device="hip")
    nb.load_state_dict({"weight": w_np})
    np.testing.assert_allclose(nb(Tensor.from_numpy(x_np)).to_numpy(), want - b_np, rtol=0, atol=1e-5)
    # fp16 activations with fp32 weights are a dtype mismatch, as in the reference (linear.cu:178-181)
    with pytest.raises(RuntimeError):
        lin(Tensor.from_numpy(x_np.astype(np.float16)))


def test_linear_follows_weights_written_after_a_forward(hip_env):
    """A Linear that has run once keeps a packed copy of its weight; load_state_dict / copy_from /
    copy_from_numpy write the weight in place, and the next forward must use the new values (the
    reference's Linear reads the live weight on every call, nn/layers.py:72-80)."""
    rng = np.random.default_rng(11)
    x_np = rng.normal(size=(8, 64)).astype(np.float16)
    lin = nn.Linear(64, 32, bias=False, device="hip")
    lin.cast_linear_fp16()
    x = Tensor.from_numpy(x_np)

    def want(w16):
        return port.linear(x_np.astype(np.float32), w16.astype(np.float32), None)

    w0 = lin.weight.numpy().copy()
    np.testing.assert_allclose(lin(x).to_numpy(), want(w0), rtol=0, atol=2e-5)
    w1 = (rng.normal(size=(32, 64)) * 0.05).astype(np.float16)
    lin.load_state_dict({"weight": w1})
    np.testing.assert_allclose(lin(x).to_numpy(), want(w1), rtol=0, atol=2e-5)
    w2 = (rng.normal(size=(32, 64)) * 0.05).astype(np.float16)
    lin.weight.copy_from_numpy(w2)
    np.testing.assert_allclose(lin(x).to_numpy(), want(w2), rtol=0, atol=2e-5)
    w3 = (rng.normal(size=(32, 64)) * 0.05).astype(np.float16)
    lin.weight.copy_from(Tensor.from_numpy(w3))
    np.testing.assert_allclose(lin(x).to_numpy(), want(w3), rtol=0, atol=2e-5)
    lin.weight.fill_zero()
    assert np.all(lin(x).to_numpy() == 0)


def _np_attention(q, k, v, causal):
    sq, hq, d = q.shape
    skv, hkv = k.shape[:2]
    out = np.zeros((sq, hq, d), np.float32)
    for i in range(sq):
        for h in range(hq):
            end = min(i + 1, skv) if causal else skv
            s = q[i, h] @ k[:end, h // (hq // hkv)].T / math.sqrt(d)
            p = np.exp(s - s.max())
            p /= p.sum()
            out[i, h] = p @ v[:end, h // (hq // hkv)]
    return out


def test_dynamic_kv_cache_with_attention():
    """tests/nn/test_kv_cache.py of the reference: append / len / reset, and decode with the cache
    equals the causal full forward."""
    rng = np.random.default_rng(0)
    cache = nn.DynamicKVCache(2, device=DEV)
    k1 = rng.standard_normal((5, 2, 8)).astype(np.float32)
    k2 = rng.standard_normal((1, 2, 8)).astype(np.float32)
    cache.update(0, t(k1), t(k1))
    assert len(cache) == 5
    cache.update(0, t(k2), t(k2))
    assert len(cache) == 6
    np.testing.assert_allclose(cache.get(0)[0].to_numpy(), np.concatenate([k1, k2], 0), rtol=1e-6)
    cache.reset()
    assert len(cache) == 0
    sq, hq, hkv, d = 6, 4, 2, 64
    q, k, v = (rng.standard_normal(s).astype(np.float32) for s in ((sq, hq, d), (sq, hkv, d), (sq, hkv, d)))
    full = axono.scaled_dot_product_attention(t(q), t(k), t(v), True).to_numpy()
    np.testing.assert_allclose(full, _np_attention(q, k, v, True), rtol=1e-4, atol=1e-5)
    cache = nn.DynamicKVCache(1, device=DEV)
    for i in range(sq):
        cache.update(0, t(k[i:i + 1]), t(v[i:i + 1]))
        kk, vv = cache.get(0)
        step = axono.gqa_decode_attention(t(q[i:i + 1]), kk, vv) if i > 0 else axono.scaled_dot_product_attention(t(q[i:i + 1]), kk, vv, False)
        np.testing.assert_allclose(step.to_numpy()[0], full[i], rtol=1e-4, atol=1e-5)


def test_custom_sliding_window_cache_component():
    """tests/nn/test_kv_cache.py:75-114 of the reference: a user-written KVCache that keeps the last
    two steps with concat + slice_; also get() before update() and independent layers (:60-73)."""

    class SlidingWindowCache(nn.KVCache):
        def __init__(self, window=2):
            self.window, self.k, self.v = window, None, None

        def update(self, layer_idx, k_new, v_new):
            if self.k is None:
                self.k, self.v = k_new, v_new
            else:
                self.k, self.v = axono.concat(self.k, k_new, 0), axono.concat(self.v, v_new, 0)
            extra = int(self.k.shape[0]) - self.window
            if extra > 0:
                self.k = axono.slice_(self.k, 0, extra, self.window)
                self.v = axono.slice_(self.v, 0, extra, self.window)

        def get(self, layer_idx):
            return self.k, self.v

        def reset(self):
            self.k = self.v = None

        def __len__(self):
            return 0 if self.k is None else int(self.k.shape[0])

    def kv(seed, steps=1):
        return np.random.RandomState(seed).randn(steps, 1, 4).astype(np.float32)

    cache = SlidingWindowCache(window=2)
    for i in range(4):
        cache.update(0, t(kv(i)), t(kv(i + 10)))
    assert len(cache) == 2
    np.testing.assert_array_equal(cache.get(0)[0].to_numpy(), np.concatenate([kv(2), kv(3)]))
    np.testing.assert_array_equal(cache.get(0)[1].to_numpy(), np.concatenate([kv(12), kv(13)]))
    cache.reset()
    assert len(cache) == 0

    dyn = nn.DynamicKVCache(2, device=DEV)
    with pytest.raises(RuntimeError):
        dyn.get(0)
    dyn.update(0, t(kv(0, 2)), t(kv(1, 2)))
    dyn.update(1, t(kv(2, 5)), t(kv(3, 5)))
    assert len(dyn) == 2                      # the first non-empty layer's length
    assert dyn.get(0)[0].to_numpy().shape == (2, 1, 4) and dyn.get(1)[0].to_numpy().shape == (5, 1, 4)


def test_static_kv_cache_matches_dynamic():
    rng = np.random.default_rng(5)
    B, hkv, d, lmax = 3, 2, 64, 16
    st = nn.StaticKVCache(1, B, hkv, lmax, d, DataType.FLOAT16, DEV)
    dyn = [nn.DynamicKVCache(1, device=DEV) for _ in range(B)]
    for step in range(5):
        kn = rng.standard_normal((B, hkv, d)).astype(np.float16)
        vn = rng.standard_normal((B, hkv, d)).astype(np.float16)
        st.update(0, t(kn), t(vn))
        st.advance()
        for b in range(B):
            dyn[b].update(0, t(kn[b:b + 1]), t(vn[b:b + 1]))
    assert len(st) == 5
    np.testing.assert_array_equal(st.seq_lens.to_numpy(), [5, 5, 5])
    kc = st.get(0)[0].numpy()
    for b in range(B):
        np.testing.assert_array_equal(np.transpose(kc[b, :, :5], (1, 0, 2)).view(np.uint16), dyn[b].get(0)[0].numpy().view(np.uint16))
    assert np.all(kc[:, :, 5:] == 0)


def test_graph_capture_replay_semantics():
    """tests/core/test_cuda_graph.py of the reference: replay is idempotent, an in-place input update
    is visible after replay, temporaries inside the body are fine, replay before capture raises, an
    empty capture raises, reset allows a new capture."""
    rng = np.random.default_rng(0)
    a = t(rng.standard_normal((8, 256)).astype(np.float32))
    b = t(rng.standard_normal((8, 256)).astype(np.float32))
    w = t(np.ones(256, np.float32))

    def body():
        s = axono.add(a, b)                      # a temporary
        y, o = axono.add_rms_norm(s, a, w, 1e-6)
        return axono.silu_mul(o, y), y

    eager = [x.to_numpy().copy() for x in body()]
    g = axono.HIPGraph()
    with pytest.raises(RuntimeError):
        g.replay()
    g.capture(body)
    assert g.is_captured and g.num_nodes >= 3
    for _ in range(3):  # several replays, each checked against the eager result
        g.replay()
        L.synchronize()
        for got, want in zip(g.outputs, eager):
            np.testing.assert_allclose(got.to_numpy(), want, rtol=1e-6, atol=1e-6)
    a_new = rng.standard_normal((8, 256)).astype(np.float32)
    a.copy_from_numpy(a_new)  # refresh the static input in place
    g.replay()
    eager2 = [x.to_numpy().copy() for x in body()]
    for got, want in zip(g.outputs, eager2):
        np.testing.assert_allclose(got.to_numpy(), want, rtol=1e-6, atol=1e-6)
    assert g.output is g.outputs[0]
    g.reset()
    assert not g.is_captured
    g.capture(lambda: axono.add(a, b))
    g.replay()
    np.testing.assert_allclose(g.output.to_numpy(), a_new + b.to_numpy(), rtol=1e-6)
    g.reset()
    with pytest.raises(RuntimeError):
        axono.HIPGraph().capture(lambda: None)  # nothing captured
    # context-manager form: the block is captured as it runs
    with axono.hip_graph() as g2:
        y = axono.add(a, b)
        g2.output = y
    a.copy_from_numpy(np.zeros((8, 256), np.float32))
    g2.replay()
    np.testing.assert_allclose(g2.output.to_numpy(), b.to_numpy(), rtol=1e-6)
    # a failing body aborts the capture and leaves the library usable
    with pytest.raises(ZeroDivisionError):
        axono.HIPGraph().capture(lambda: 1 / 0)
    assert L._lib_().axhip_is_capturing() == 0
    np.testing.assert_allclose(axono.add(a, b).to_numpy(), b.to_numpy(), rtol=1e-6)


def test_graphs_replayed_side_by_side_on_ticket_lanes():
    """Two graphs, each with an attention launch that merges key ranges in the kernel and a wide argmax
    (both finish through static ticket counters), captured under different ticket lanes and replayed
    side by side on their own streams: every replay gives the eager result."""
    rng = np.random.default_rng(5)
    graphs, wants, inputs = [], [], []  # the graphs read their inputs at fixed addresses: they stay alive
    for lane in (0, 1):
        q = t(rng.standard_normal((1, 16, 128)).astype(np.float32))
        k = t(rng.standard_normal((4096 + 512 * lane, 8, 128)).astype(np.float32))
        v = t(rng.standard_normal((4096 + 512 * lane, 8, 128)).astype(np.float32))
        x = t(rng.standard_normal((8, 40000)).astype(np.float32))

        def body(q=q, k=k, v=v, x=x):
            return axono.gqa_decode_attention(q, k, v), axono.argmax(x)

        inputs.append((q, k, v, x))
        wants.append([o.to_numpy().copy() for o in body()])
        L.set_ticket_lane(lane)
        try:
            graphs.append(axono.HIPGraph().capture(body))
        finally:
            L.set_ticket_lane(0)
    assert L._lib_().axhip_ticket_lane() == 0
    with pytest.raises(RuntimeError):
        L.set_ticket_lane(8)
    for _ in range(4):
        for _ in range(16):
            for g in graphs:
                g.launch_async()
        for g in graphs:
            g.sync()
        for g, want in zip(graphs, wants):
            np.testing.assert_allclose(g.outputs[0].to_numpy(), want[0], rtol=0, atol=1e-6)
            np.testing.assert_array_equal(g.outputs[1].to_numpy(), want[1])
    for g in graphs:
        g.reset()


def test_compile_caches_by_signature_and_refreshes_inputs():
    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.w = t(np.linspace(0.5, 1.5, 128).astype(np.float32))

        def forward(self, x, res):
            y, o = axono.add_rms_norm(x, res, self.w, 1e-6)
            return axono.silu_mul(o, y)

    m = Block()
    cm = axono.compile(m)
    rng = np.random.default_rng(2)
    for trial in range(3):
        x, r = rng.standard_normal((4, 128)).astype(np.float32), rng.standard_normal((4, 128)).astype(np.float32)
        got = cm(t(x), t(r)).to_numpy().copy()
        want = m(t(x), t(r)).to_numpy()
        np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-6)
    assert len(cm._graphs) == 1
    x8 = rng.standard_normal((8, 128)).astype(np.float32)
    np.testing.assert_allclose(cm(t(x8), t(x8)).to_numpy(), m(t(x8), t(x8)).to_numpy(), rtol=1e-6, atol=1e-6)
    assert len(cm._graphs) == 2 and "graphs=2" in repr(cm)
    assert cm.w is m.w  # attribute access passes through to the model


def test_allocator_cache_and_budget():
    L.synchronize()
    L.empty_cache()
    base = L.cached_bytes()
    assert base == 0
    x = Tensor(DataType.FLOAT32, [1 << 20], DEV)  # 4 MiB
    p = x.data_ptr
    assert np.all(x.to_numpy() == 0)
    x.copy_from_numpy(np.ones(1 << 20, np.float32))
    del x
    assert L.cached_bytes() == 4 << 20            # released blocks stay cached
    y = Tensor(DataType.FLOAT32, [1 << 20], DEV)
    assert y.data_ptr == p                         # same-size request reuses the cached block
    assert np.all(y.to_numpy() == 0)               # and a new tensor still reads as zeros
    assert L.cached_bytes() == 0
    del y
    L.set_cache_budget(1 << 20)                    # smaller than the block: evicted on release
    assert L.cached_bytes() == 0
    z = Tensor(DataType.FLOAT32, [1 << 20], DEV)
    del z
    assert L.cached_bytes() <= 1 << 20
    L.set_cache_budget(64 << 30)
    # many release / reuse cycles of a few sizes (the eviction queue is compacted, the cache stays exact)
    L.empty_cache()
    for i in range(5000):
        t1 = Tensor(DataType.INT8, [4096 * (1 + i % 3)], DEV, _zero=False)
        del t1
    assert L.cached_bytes() == 4096 * (1 + 2 + 3)
    L.set_cache_budget(4096 * 3)                   # oldest first: the newest block that still fits stays
    assert 0 < L.cached_bytes() <= 4096 * 3
    L.set_cache_budget(64 << 30)
    L.empty_cache()
    assert L.cached_bytes() == 0


def test_ticket_counters_can_be_reset_for_recovery():
    """axhip_reset_tickets zeroes the static ticket counters (empty_cache leaves them alone); attention that
    merges key ranges in the kernel and the wide argmax give the same results before and after."""
    from axono_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(31)
    q = rng.standard_normal((1, 16, 128)).astype(np.float32)
    k = rng.standard_normal((3000, 8, 128)).astype(np.float32)
    v = rng.standard_normal((3000, 8, 128)).astype(np.float32)
    x = rng.standard_normal((3, 151936)).astype(np.float32)
    before = axono.gqa_decode_attention(t(q), t(k), t(v)).to_numpy()
    am_before = axono.argmax(t(x)).to_numpy()
    assert lib.axhip_reset_tickets() == 0
    L.empty_cache()
    np.testing.assert_array_equal(axono.gqa_decode_attention(t(q), t(k), t(v)).to_numpy(), before)
    np.testing.assert_array_equal(axono.argmax(t(x)).to_numpy(), am_before)
    np.testing.assert_array_equal(am_before, x.argmax(-1))
    np.testing.assert_allclose(before, port.gqa_decode(q, k, v), rtol=0, atol=1e-5)


def test_axm_weights_go_straight_to_the_device(tmp_path):
    """save_axm -> load_axm_to_device: values arrive unchanged; dtype="float16" converts floating
    tensors on the way (one IEEE rounding) and leaves integer tensors alone."""
    from axono_amd.format import load_axm_to_device, save_axm

    rng = np.random.default_rng(3)
    sd = {"w": rng.standard_normal((33, 70)).astype(np.float32), "h": rng.standard_normal((5, 8)).astype(np.float16),
          "ids": np.arange(12, dtype=np.int64)}
    p = str(tmp_path / "w.axm")
    save_axm(sd, p)
    dev = load_axm_to_device(p, "hip")
    assert set(dev) == set(sd)
    for k, v in sd.items():
        assert dev[k].device.startswith("hip") and dev[k].shape == list(v.shape)
        np.testing.assert_array_equal(dev[k].numpy(), v)
    dev16 = load_axm_to_device(p, "hip", dtype="float16", names=["w", "ids"])
    assert set(dev16) == {"w", "ids"}
    np.testing.assert_array_equal(dev16["w"].numpy(), sd["w"].astype(np.float16))
    np.testing.assert_array_equal(dev16["ids"].numpy(), sd["ids"])


def test_paged_kv_cache_component():
    """nn.PagedKVCache: prefill rows per sequence, one-token updates, attention through the page table
    equal to the static cache's bit for bit, page accounting, freeing a sequence, running out of pages."""
    rng = np.random.default_rng(41)
    B, hq, hkv, d, lmax = 3, 4, 2, 64, 512
    order = rng.permutation(10)
    pg = nn.PagedKVCache(2, B, hkv, d, n_pages=10, max_len=lmax, dtype=DataType.FLOAT16, device=DEV, page_order=order)
    st = nn.StaticKVCache(2, B, hkv, lmax, d, DataType.FLOAT16, DEV)
    assert len(pg) == 0 and pg.pages_in_use == 0
    prompt = [130, 5, 256]
    for layer in range(2):
        for b, n in enumerate(prompt):
            kr = rng.standard_normal((n, hkv, d)).astype(np.float16)
            vr = rng.standard_normal((n, hkv, d)).astype(np.float16)
            pg.update_rows(layer, b, t(kr), t(vr))
            # the static cache row by row (its layout is [B, hkv, L, d])
            kc, vc = st.get(layer)
            kh, vh = kc.numpy(), vc.numpy()
            kh[b, :, :n], vh[b, :, :n] = np.transpose(kr, (1, 0, 2)), np.transpose(vr, (1, 0, 2))
            kc.copy_from_numpy(kh)
            vc.copy_from_numpy(vh)
    for b, n in enumerate(prompt):
        pg.advance_rows(b, n)
    st.set_lengths(prompt)
    assert pg.pages_in_use == 2 + 1 + 2 and len(pg) == 256
    np.testing.assert_array_equal(pg.seq_lens.to_numpy(), prompt)
    for step in range(3):
        q = rng.standard_normal((B, hq, d)).astype(np.float16)
        for layer in range(2):
            kn = rng.standard_normal((B, hkv, d)).astype(np.float16)
            vn = rng.standard_normal((B, hkv, d)).astype(np.float16)
            pg.update(layer, t(kn), t(vn))
            st.update(layer, t(kn), t(vn))
            got = pg.attend(layer, t(q), extra_tokens=1).numpy()
            lens1 = Tensor(DataType.INT32, [B], DEV)
            lens1.copy_from_numpy((np.array(prompt) + step + 1).astype(np.int32))
            want = axono.gqa_decode_attention_cache(t(q), *st.get(layer), lens1, max_len=int(max(prompt)) + step + 1).numpy()
            np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16))
        pg.advance()
        st.advance()
    assert pg.pages_in_use == 2 + 1 + 3                  # sequence 2 crossed into its third page at 257 tokens
    pg.free_sequence(0)
    assert pg.pages_in_use == 4 and int(pg.seq_lens.to_numpy()[0]) == 0
    with pytest.raises(MemoryError):
        pg.reserve([512, 0, 0])                          # 4 pages for sequence 0, then 512 more tokens for it: 6 free
        pg.reserve([0, 512 - 8, 512 - 259])
    with pytest.raises(ValueError):
        pg.reserve([0, 0, 300])                          # past max_len
    pg.reset()
    assert pg.pages_in_use == 0 and len(pg) == 0


def test_paged_kv_cache_step_captured_in_a_graph():
    """One decode step over a PagedKVCache (append through the page table, attention over the pages, length
    advance) captured once and replayed: pages for all replays are reserved before the capture, so the body
    has no host <-> device traffic.  Every replay equals the static cache driven eagerly with the same inputs."""
    rng = np.random.default_rng(43)
    B, hq, hkv, d, lmax, steps = 2, 4, 2, 64, 384, 5
    pg = nn.PagedKVCache(1, B, hkv, d, n_pages=6, max_len=lmax, device=DEV, page_order=[5, 1, 4, 0, 3, 2])
    st = nn.StaticKVCache(1, B, hkv, lmax, d, DataType.FLOAT16, DEV)
    prompt = [126, 250]                         # both sequences cross a page boundary during the replays
    for b, n in enumerate(prompt):
        kr = rng.standard_normal((n, hkv, d)).astype(np.float16)
        vr = rng.standard_normal((n, hkv, d)).astype(np.float16)
        pg.update_rows(0, b, t(kr), t(vr))
        pg.advance_rows(b, n)
        kc, vc = st.get(0)
        kh, vh = kc.numpy(), vc.numpy()
        kh[b, :, :n], vh[b, :, :n] = np.transpose(kr, (1, 0, 2)), np.transpose(vr, (1, 0, 2))
        kc.copy_from_numpy(kh)
        vc.copy_from_numpy(vh)
    st.set_lengths(prompt)
    pg.reserve(steps + 2)                       # warm-up run + recorded run + replays never allocate a page
    q_in = Tensor(DataType.FLOAT16, [B, hq, d], DEV)
    k_in = Tensor(DataType.FLOAT16, [B, hkv, d], DEV)
    v_in = Tensor(DataType.FLOAT16, [B, hkv, d], DEV)
    bound = max(prompt) + steps + 2

    def step():
        pg.update(0, k_in, v_in)
        out = pg.attend(0, q_in, extra_tokens=1, max_len=bound)
        pg.advance()
        return out

    lens0 = pg.seq_lens.to_numpy().copy()
    g = axono.HIPGraph().capture(step)          # runs the body twice
    pg.seq_lens.copy_from_numpy(lens0)
    pg.sync_from_device()
    for s_ in range(steps):
        qn = rng.standard_normal((B, hq, d)).astype(np.float16)
        kn = rng.standard_normal((B, hkv, d)).astype(np.float16)
        vn = rng.standard_normal((B, hkv, d)).astype(np.float16)
        q_in.copy_from_numpy(qn)
        k_in.copy_from_numpy(kn)
        v_in.copy_from_numpy(vn)
        g.replay()
        got = g.output.numpy().copy()
        st.update(0, t(kn), t(vn))
        lens1 = Tensor(DataType.INT32, [B], DEV)
        lens1.copy_from_numpy((np.array(prompt) + s_ + 1).astype(np.int32))
        want = axono.gqa_decode_attention_cache(t(qn), *st.get(0), lens1, max_len=bound).numpy()
        st.advance()
        np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16))
    pg.sync_from_device()
    assert len(pg) == max(prompt) + steps
    np.testing.assert_array_equal(pg.seq_lens.to_numpy(), np.array(prompt) + steps)
