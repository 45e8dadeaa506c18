"""AXM1 weight container: the reference's own test cases (tests/core/test_axm.py:11-72) on this
build's implementation, plus a byte-level check against the documented layout
(axono/python/axono/format/axm.py:19-33) built by hand, so that files are interchangeable."""
import json
import os
import struct

import numpy as np
import pytest

from axono_amd.format import AxmReader, load_axm, read_axm_index, save_axm


def test_roundtrip_mixed_dtypes(tmp_path):
    p = str(tmp_path / "w.axm")
    sd = {"layer.weight": np.random.RandomState(0).randn(64, 32).astype(np.float32),
          "layer.bias": np.arange(64, dtype=np.float32),
          "embed": np.random.RandomState(1).randn(100, 16).astype(np.float16)}
    save_axm(sd, p)
    out = load_axm(p)
    assert set(out) == set(sd)
    for k in sd:
        assert out[k].dtype == sd[k].dtype
        np.testing.assert_array_equal(out[k], sd[k])


def test_dtype_convert_fp16(tmp_path):
    p, p32 = str(tmp_path / "w16.axm"), str(tmp_path / "w32.axm")
    sd = {"w": np.random.RandomState(2).randn(32, 16).astype(np.float32)}
    save_axm(sd, p, dtype="float16")
    out = load_axm(p)
    assert out["w"].dtype == np.float16
    np.testing.assert_array_equal(out["w"], sd["w"].astype(np.float16))   # one IEEE rounding
    save_axm(sd, p32)
    assert os.path.getsize(p) < os.path.getsize(p32) * 0.75


def test_reader_streaming_and_meta(tmp_path):
    p = str(tmp_path / "w.axm")
    sd = {"a": np.ones((8, 8), np.float32), "b": np.zeros((4,), np.float32)}
    save_axm(sd, p, meta={"source": "test"})
    r = AxmReader(p)
    assert sorted(r.names()) == ["a", "b"]
    assert r.meta()["source"] == "test"
    np.testing.assert_array_equal(r.get("b"), sd["b"])
    with pytest.raises(KeyError):
        r.get("missing")


def test_index_only(tmp_path):
    p = str(tmp_path / "w.axm")
    save_axm({"x": np.ones((3, 3), np.float32)}, p)
    idx, data_start = read_axm_index(p)
    assert idx["tensors"][0]["name"] == "x"
    assert data_start > 16 and data_start % 64 == 0


def test_bad_files(tmp_path):
    short = str(tmp_path / "short.bin")
    open(short, "wb").write(b"XXXX")
    with pytest.raises(ValueError):
        load_axm(short)
    bad = str(tmp_path / "bad.bin")
    open(bad, "wb").write(b"NOPE" + bytes(60))
    with pytest.raises(ValueError):
        load_axm(bad)
    ver = str(tmp_path / "ver.bin")
    open(ver, "wb").write(struct.pack("<4sHHQ", b"AXM1", 2, 0, 2) + b"{}" + bytes(46))
    with pytest.raises(ValueError):
        read_axm_index(ver)


def test_byte_layout_matches_the_documented_format(tmp_path):
    """A file assembled by hand from the format description is read back, and a file written by
    save_axm has exactly those bytes."""
    a = np.arange(5, dtype=np.float32)            # 20 bytes -> padded to 64
    b = np.arange(70, dtype=np.int64).astype(np.float16).reshape(7, 10)   # 140 bytes -> padded to 192
    index = {"tensors": [{"name": "a", "dtype": "float32", "shape": [5], "offset": 0, "size": 20},
                         {"name": "b", "dtype": "float16", "shape": [7, 10], "offset": 64, "size": 140}],
             "meta": {"k": 1}}
    ib = json.dumps(index).encode()
    blob = struct.pack("<4sHHQ", b"AXM1", 1, 0, len(ib)) + ib
    blob += bytes(-len(blob) % 64)
    blob += a.tobytes() + bytes(44) + b.tobytes() + bytes(52)
    hand = str(tmp_path / "hand.axm")
    open(hand, "wb").write(blob)
    got = load_axm(hand)
    np.testing.assert_array_equal(got["a"], a)
    np.testing.assert_array_equal(got["b"], b)
    ours = str(tmp_path / "ours.axm")
    save_axm({"a": a, "b": b}, ours, meta={"k": 1})
    assert open(ours, "rb").read() == blob


def test_mmap_false_gives_independent_arrays(tmp_path):
    p = str(tmp_path / "w.axm")
    save_axm({"x": np.arange(6, dtype=np.float32).reshape(2, 3), "empty": np.zeros((0, 4), np.float32)}, p)
    out = load_axm(p, mmap=False)
    assert not isinstance(out["x"], np.memmap)
    out["x"][0, 0] = 9.0                       # writable, not backed by the file
    assert load_axm(p)["x"][0, 0] == 0.0
    assert out["empty"].shape == (0, 4)


def test_large_roundtrip(tmp_path):
    p = str(tmp_path / "big.axm")
    big = np.random.RandomState(3).randn(1024, 6144).astype(np.float32)   # 25 MB
    save_axm({"big": big}, p)
    np.testing.assert_array_equal(load_axm(p)["big"], big)


def test_text_model_weights_roundtrip_in_reference_naming(tmp_path):
    """Fused q/k/v and gate/up are split into the reference's parameter names on save and fused
    again on load; Linear weights come back fp16, norm weights fp32."""
    from axono_amd.examples.qwen3vl_text import TextConfig, random_weights, weights_from_axm, weights_to_axm

    cfg = TextConfig(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
                     intermediate_size=96, vocab_size=50)
    w = random_weights(cfg, seed=5)
    p = str(tmp_path / "text.axm")
    weights_to_axm(w, cfg, p)
    names = AxmReader(p).names()
    assert "model.language_model.layers.0.self_attn.k_proj.weight" in names
    assert "model.language_model.layers.1.mlp.up_proj.weight" in names
    assert not any("qkv_proj" in n or "gate_up" in n for n in names)
    back = weights_from_axm(p, cfg)
    assert set(back) == set(w)
    for k in w:
        assert back[k].dtype == w[k].dtype, k
        np.testing.assert_array_equal(back[k], w[k])
