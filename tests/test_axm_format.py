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


# ---- safetensors -> AXM1 (reference: examples/vlm/qwen3vl/convert.py:32-64) ------------------------

def _write_checkpoint(dirname, tensors, filename="model.safetensors"):
    from safetensors.torch import save_file

    os.makedirs(dirname, exist_ok=True)
    save_file(tensors, os.path.join(dirname, filename), metadata={"format": "pt"})


def _fake_checkpoint():
    import torch

    g = torch.Generator().manual_seed(11)
    return {
        "model.language_model.embed_tokens.weight": torch.randn(50, 16, generator=g).to(torch.bfloat16),
        "model.language_model.layers.0.self_attn.q_proj.weight": torch.randn(32, 16, generator=g).to(torch.bfloat16),
        "model.language_model.norm.weight": torch.ones(16, dtype=torch.float16),
        "model.visual.patch_embed.proj.weight": torch.randn(8, 3, 2, 4, 4, generator=g),
        "model.visual.patch_embed.proj.bias": torch.randn(8, generator=g),
        "model.visual.blocks.0.attn.qkv.weight": torch.tensor([[1e-40, -0.0, 65504.0, 3.3895314e38]]).to(torch.bfloat16),
        "model.language_model.empty": torch.zeros(0, 4),
    }


def test_convert_safetensors_checkpoint(tmp_path):
    from axono_amd.format.convert import convert, main

    src = _fake_checkpoint()
    d = str(tmp_path / "qwen3vl-2b")
    _write_checkpoint(d, src)
    out = os.path.join(d, "model.axm")
    st = convert(d, out, None)
    assert st["n_tensors"] == len(src) and st["size_gb"] > 0
    got = load_axm(out)
    assert set(got) == set(src)
    for k, v in src.items():
        want = v.float().numpy()
        if k.endswith("patch_embed.proj.weight"):
            want = want.reshape(want.shape[0], -1)       # (out, 3*t*p*p), as the model's Linear wants it
        assert got[k].dtype == np.float32 and got[k].shape == want.shape, k
        np.testing.assert_array_equal(got[k].view(np.uint32), want.view(np.uint32), err_msg=k)  # bf16 widening is exact
    index, _ = read_axm_index(out)
    assert index["meta"]["source"] == "hf-safetensors" and index["meta"]["model_dir"] == "qwen3vl-2b"
    assert index["meta"]["dtype"] == "keep" and "converted_at" in index["meta"]
    # --dtype float16 halves the file; default output path; command line
    with np.errstate(over="ignore"):  # the largest bf16 value of the fixture is inf in fp16
        assert main(["--model", d, "--dtype", "float16", "--out", str(tmp_path / "h.axm")]) == 0
    half = load_axm(str(tmp_path / "h.axm"))
    k = "model.language_model.layers.0.self_attn.q_proj.weight"
    np.testing.assert_array_equal(half[k], src[k].float().numpy().astype(np.float16))
    assert read_axm_index(str(tmp_path / "h.axm"))[0]["meta"]["dtype"] == "float16"
    os.remove(out)
    assert main(["--model", d]) == 0 and os.path.exists(out)


def test_convert_sharded_checkpoint_and_errors(tmp_path):
    import json

    from axono_amd.format.convert import convert, read_safetensors_index

    src = _fake_checkpoint()
    names = sorted(src)
    d = str(tmp_path / "sharded")
    parts = {"model-00001-of-00002.safetensors": names[:3], "model-00002-of-00002.safetensors": names[3:]}
    for fn, ks in parts.items():
        _write_checkpoint(d, {k: src[k] for k in ks}, fn)
    with open(os.path.join(d, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {}, "weight_map": {k: fn for fn, ks in parts.items() for k in ks}}, f)
    out = str(tmp_path / "s.axm")
    assert convert(d, out, None)["n_tensors"] == len(src)
    got = load_axm(out)
    for k, v in src.items():
        np.testing.assert_array_equal(got[k].reshape(-1), v.float().numpy().reshape(-1))
    with pytest.raises(FileNotFoundError):
        convert(str(tmp_path / "nothing"), out, None)
    bad = tmp_path / "bad.safetensors"
    bad.write_bytes(b"\xff" * 16)
    with pytest.raises(ValueError):
        read_safetensors_index(str(bad))
    bad.write_bytes(b"\x01\x02")
    with pytest.raises(ValueError):
        read_safetensors_index(str(bad))
