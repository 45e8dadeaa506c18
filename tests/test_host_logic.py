"""Host-side logic of the Python surface that needs no GPU: Tensor metadata and host storage
semantics, device-string handling, the nn.Module registry, signature keys of compile()."""
import copy

import numpy as np
import pytest

import axono_amd as axono
from axono_amd import DataType, Status, Tensor, nn
from axono_amd.core.compile import _call_key
from axono_amd.core.tensor import parse_device
from axono_amd.device import AxhipError


def test_enum_values_match_reference():
    assert [int(d) for d in (DataType.INT8, DataType.INT16, DataType.INT32, DataType.INT64, DataType.FLOAT16,
                             DataType.FLOAT32, DataType.FLOAT64, DataType.BOOLEAN)] == list(range(8))
    assert [int(s) for s in (Status.OK, Status.INVALID_ARGUMENT, Status.OUT_OF_MEMORY, Status.UNSUPPORTED_TYPE,
                             Status.SHAPE_MISMATCH, Status.INTERNAL_ERROR, Status.DEVICE_ERROR, Status.INVALID_PTR,
                             Status.DEVICE_MISMATCH)] == list(range(9))


def test_device_strings():
    assert parse_device("cpu") == ("cpu", None)
    assert parse_device("hip") == ("hip", 0)
    assert parse_device("hip:3") == ("hip", 3)
    for bad in ("cuda", "cuda:0", "gpu", "", "hip:x"):
        with pytest.raises(ValueError):
            parse_device(bad)
    with pytest.raises(ValueError):
        axono.set_backend("cuda")
    axono.set_backend("cpu")
    assert axono.get_backend() == "cpu"
    assert axono.cuda_available() is False


def test_new_tensor_is_zero_and_numpy_view_shares_memory():
    t = Tensor(DataType.FLOAT32, [2, 3])
    assert t.shape == [2, 3] and t.ndim == 2 and t.num_elements == 6 and t.num_bytes == 24 and t.device == "cpu"
    view = t.to_numpy()
    assert np.all(view == 0)
    view[:] = 5
    assert np.all(t.to_numpy() == 5)
    assert Tensor(DataType.FLOAT32).num_elements == 0


def test_from_numpy_copies_and_ref_borrows():
    a = np.arange(6, dtype=np.float32).reshape(2, 3)
    t = Tensor.from_numpy(a)
    a[0, 0] = 99
    assert t.to_numpy()[0, 0] == 0
    r = Tensor.from_numpy_ref(a)
    a[0, 1] = 77
    assert r.to_numpy()[0, 1] == 77
    assert Tensor.from_numpy(np.array([[1, 2], [3, 4]])).dtype == DataType.INT64
    assert Tensor.from_numpy(np.ones(3, np.complex64)).dtype == DataType.FLOAT32


def test_float16_bit_patterns():
    x = np.array([[1.0, 2.0], [3.0, 4.0]], np.float16)
    t = Tensor.from_numpy_ref(x)
    assert t.dtype == DataType.FLOAT16
    assert t.to_numpy().dtype == np.int16  # the reference exposes FLOAT16 as int16 bit patterns
    np.testing.assert_array_equal(t.to_numpy().view(np.float16), x)
    np.testing.assert_array_equal(t.numpy(), x)
    back = t.cast_to(DataType.FLOAT32).to_numpy()
    np.testing.assert_array_equal(back, x.astype(np.float32))
    # host conversion is IEEE round-to-nearest-even, as on the device
    v = np.random.default_rng(0).standard_normal(1000).astype(np.float32)
    np.testing.assert_array_equal(Tensor.from_numpy(v).cast_to(DataType.FLOAT16).numpy(), v.astype(np.float16))
    np.testing.assert_allclose(Tensor.from_numpy(np.array([1.0, -0.5, 65504.0, 0.0], np.float32))
                               .cast_to(DataType.FLOAT16).cast_to(DataType.FLOAT32).to_numpy(),
                               [1.0, -0.5, 65504.0, 0.0], rtol=1e-3)


def test_copy_aliases_storage_and_deepcopy_does_not():
    t = Tensor.from_numpy(np.zeros(4, np.float32))
    alias = copy.copy(t)
    alias.to_numpy()[:] = 3
    assert np.all(t.to_numpy() == 3)
    deep = copy.deepcopy(t)
    deep.to_numpy()[:] = 9
    assert np.all(t.to_numpy() == 3)
    same = t.cast_to(DataType.FLOAT32)  # same dtype: an alias
    same.to_numpy()[0] = -1
    assert t.to_numpy()[0] == -1
    assert t.to("cpu") is t


def test_reshape_in_place_and_resize():
    t = Tensor.from_numpy(np.arange(24, dtype=np.float32).reshape(2, 3, 4))
    assert t.reshape([6, 4]) is t and t.shape == [6, 4]
    assert t.reshape([-1, 8]).shape == [3, 8]
    with pytest.raises(ValueError):
        t.reshape([-1, -1])
    with pytest.raises(ValueError):
        t.reshape([-1, 7])
    with pytest.raises(RuntimeError):
        t.reshape([5, 5])
    np.testing.assert_array_equal(t.to_numpy().reshape(-1), np.arange(24))
    t.resize([4, 6])  # same element count: data kept
    np.testing.assert_array_equal(t.to_numpy().reshape(-1), np.arange(24))
    t.resize([2, 2])  # new element count: fresh zeroed storage
    assert np.all(t.to_numpy() == 0) and t.shape == [2, 2]


def test_copy_from_numpy_checks_and_fill():
    t = Tensor.zeros([2, 3])
    t.copy_from_numpy(np.ones((2, 3), np.float32))
    assert np.all(t.to_numpy() == 1)
    with pytest.raises(ValueError):
        t.copy_from_numpy(np.ones((3, 2), np.float32))
    with pytest.raises(ValueError):
        t.copy_from_numpy(np.ones((2, 3), np.float64))
    assert np.all(Tensor.full([3], 7, DataType.INT64).to_numpy() == 7)
    assert np.all(Tensor.ones([3]).fill_zero().to_numpy() == 0)
    with pytest.raises(AxhipError):
        Tensor.zeros([2]).copy_from(Tensor.zeros([3]))


def test_operators_refuse_host_tensors():
    """There is no CPU operator path: a host tensor is an error, never a silent fallback."""
    a = Tensor.from_numpy(np.ones((2, 8), np.float32))
    with pytest.raises(RuntimeError) as e:
        axono.fused.silu_mul(a, a)
    assert "错误代码: 8" in str(e.value)  # DEVICE_MISMATCH
    with pytest.raises(RuntimeError):
        axono.rms_norm(a, None)
    with pytest.raises(RuntimeError):
        axono.gqa_decode_attention(a, a, a)


def test_module_registry_and_state_dict():
    class MLP(nn.Module):
        def __init__(self):
            super().__init__()
            self.fc1 = nn.Linear(8, 4, device="cpu")
            self.blocks = [nn.Linear(4, 4, bias=False, device="cpu") for _ in range(2)]
            self.norm = nn.RMSNorm(4, device="cpu")
            self.scale = Tensor.ones([1])

    m = MLP()
    names = list(m.parameters())
    assert names == ["scale", "fc1.weight", "fc1.bias", "blocks.0.weight", "blocks.0.bias", "blocks.1.weight",
                     "blocks.1.bias", "norm.weight"]
    assert m.parameters()["blocks.0.bias"] is None
    assert len(m.weights()) == 6
    assert m.fc1.weight.shape == [4, 8] and m.fc1.bias.shape == [4]
    w = np.arange(32, dtype=np.float32).reshape(4, 8)
    m.fc1.load_state_dict({"weight": w, "bias": np.ones(4, np.float32)})
    np.testing.assert_array_equal(m.fc1.weight.to_numpy(), w)
    with pytest.raises(KeyError):
        m.fc1.load_state_dict({"weight": w})
    m.fc1.load_state_dict({"weight": w}, strict=False)
    m.cast_linear_fp16()
    assert m.fc1.weight.dtype == DataType.FLOAT16 and m.fc1.bias.dtype == DataType.FLOAT16
    assert m.blocks[1].weight.dtype == DataType.FLOAT16
    assert m.norm.weight.dtype == DataType.FLOAT32  # only Linear layers are converted
    np.testing.assert_array_equal(m.fc1.weight.numpy(), w.astype(np.float16))
    assert repr(m.fc1).startswith("Linear(in_features=8")
    assert m.eval() is m and m._is_training is False


def test_linear_needs_fp16_weights_before_forward():
    fc = nn.Linear(8, 4, device="cpu")
    with pytest.raises(RuntimeError):
        fc(Tensor.zeros([1, 8]))


def test_dynamic_kv_cache_bookkeeping():
    """The reference's component tests (axono/python/tests/nn/test_kv_cache.py:27-73) on host tensors:
    length, append order, byte-exact contents, independent layers, reset, growth past the first capacity."""
    rng = np.random.default_rng(3)
    c = nn.DynamicKVCache(3)
    assert len(c) == 0
    with pytest.raises(RuntimeError):
        c.get(0)
    with pytest.raises(IndexError):
        c.update(3, Tensor.zeros([1, 2, 4]), Tensor.zeros([1, 2, 4]))
    ks, vs = [], []
    for step, rows in enumerate([5, 1, 1, 70, 1, 130]):   # crosses the first capacity (64) twice
        k = rng.standard_normal((rows, 2, 4)).astype(np.float32)
        v = rng.standard_normal((rows, 2, 4)).astype(np.float32)
        ks.append(k)
        vs.append(v)
        c.update(1, Tensor.from_numpy(k), Tensor.from_numpy(v))
        got_k, got_v = c.get(1)
        assert len(c) == sum(a.shape[0] for a in ks) and got_k.shape == [len(c), 2, 4]
        np.testing.assert_array_equal(got_k.to_numpy(), np.concatenate(ks, 0))
        np.testing.assert_array_equal(got_v.to_numpy(), np.concatenate(vs, 0))
    with pytest.raises(RuntimeError):
        c.get(0)                                # layers are independent
    c.update(0, Tensor.from_numpy(ks[0]), Tensor.from_numpy(vs[0]))
    assert len(c) == 5                          # the lowest-numbered layer that holds something
    with pytest.raises(RuntimeError):
        c.update(0, Tensor.zeros([1, 3, 4]), Tensor.zeros([1, 3, 4]))   # row shape differs
    c.reset()
    assert len(c) == 0
    with pytest.raises(RuntimeError):
        c.get(1)


def test_compile_signature_keys():
    a, b = Tensor.zeros([2, 3]), Tensor.zeros([2, 3])
    assert _call_key((a, 1), {"x": b}) == _call_key((b, 1), {"x": a})
    assert _call_key((a,), {}) != _call_key((Tensor.zeros([3, 2]),), {})
    assert _call_key((a, 1), {}) != _call_key((a, 2), {})
    assert _call_key((a,), {}) != _call_key((Tensor.zeros([2, 3], DataType.FLOAT16),), {})
    with pytest.raises(ValueError):
        axono.compile(lambda x: x, mode="max")


def test_missing_library_raises_instead_of_falling_back(monkeypatch, tmp_path):
    """Without libaxhip.so (and with nothing to build it from) loading raises; there is no other path."""
    from axono_amd import _lib

    def cannot_build():
        raise RuntimeError("hipcc not available")

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libaxhip.so"))
    monkeypatch.setattr(_lib._build, "build_library", cannot_build)
    with pytest.raises(RuntimeError):
        _lib.load()
    # a file that is not the library
    (tmp_path / "libaxhip.so").write_bytes(b"not a shared object")
    with pytest.raises(RuntimeError):
        _lib.load()


def test_tensor_transpose_borrowed_and_accessors_on_host():
    """Tensor.transpose / T, from_borrowed[_i64] and the data_<dtype>() accessors of the reference's binding
    (axono/python/src/nanobind_module.cpp:206-377) on host tensors."""
    a = np.arange(2 * 3 * 4, dtype=np.float32).reshape(2, 3, 4)
    t = Tensor.from_numpy(a)
    np.testing.assert_array_equal(t.transpose().to_numpy(), np.swapaxes(a, -2, -1))
    np.testing.assert_array_equal(t.transpose(0, 2).to_numpy(), np.swapaxes(a, 0, 2))
    np.testing.assert_array_equal(t.transpose(-1, 0).to_numpy(), np.swapaxes(a, 0, 2))
    assert t.transpose(1, 1).shape == [2, 3, 4]
    m = Tensor.from_numpy(a[0])
    np.testing.assert_array_equal(m.T.to_numpy(), a[0].T)
    with pytest.raises(ValueError):
        t.transpose(0, 3)
    # borrowed memory is shared, both ways
    b = np.ones((2, 5), np.float32)
    tb = Tensor.from_borrowed(b)
    b[1, 2] = 7
    assert tb.dtype == DataType.FLOAT32 and tb.to_numpy()[1, 2] == 7
    tb.data_float32()[0, 0] = -3
    assert b[0, 0] == -3
    h = np.array([1.0, -0.5, 65504.0], np.float16)
    th = Tensor.from_borrowed(h.view(np.uint16))
    assert th.dtype == DataType.FLOAT16
    np.testing.assert_array_equal(th.data_float16(), h.view(np.int16))
    np.testing.assert_array_equal(th.numpy(), h)
    ti = Tensor.from_borrowed_i64(np.arange(4, dtype=np.int64))
    assert ti.dtype == DataType.INT64 and list(ti.data_int64()) == [0, 1, 2, 3]
    with pytest.raises(RuntimeError):
        Tensor.from_borrowed(np.zeros(3, np.float64))
    with pytest.raises(RuntimeError):
        Tensor.from_borrowed_i64(np.zeros(3, np.int32))
    with pytest.raises(RuntimeError):
        tb.data_float16()
    with pytest.raises(RuntimeError):
        tb.data_int64()                      # 4-byte elements are not read as 8-byte ones
    assert tb.data_int32().dtype == np.int32   # same width: the bits reinterpreted, as the binding does
    # operators outside the decode path say so instead of computing something else
    for bad in (lambda: tb - tb, lambda: tb * tb, lambda: tb / tb, lambda: tb @ tb, lambda: -tb, lambda: abs(tb)):
        with pytest.raises(NotImplementedError):
            bad()
