"""Pins the CPU restatement of the decode step: decoding token S with the cache filled by a prefill
of S tokens must equal the last position of a prefill over S+1 tokens (the identity the reference's
tests/nn/test_kv_cache.py:117-148 checks for its cache), and the layer wiring is checked against a
direct NumPy evaluation of one layer."""
import numpy as np

from axono_amd.examples.qwen3vl_text import TextConfig, random_weights
from oracle.decode_step import OracleDecoder

CFG = TextConfig(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
                 intermediate_size=96, vocab_size=50, mrope_section=[4, 2, 2])


def _weights(seed=0):
    w = random_weights(CFG, seed)
    rng = np.random.default_rng(seed + 1)
    for k in w:
        if "norm" in k:
            w[k] = (1 + 0.1 * rng.standard_normal(w[k].shape)).astype(np.float32)
    return w


def test_decode_with_cache_equals_longer_prefill():
    w = _weights()
    rng = np.random.default_rng(5)
    B, S = 2, 9
    ids = rng.integers(0, CFG.vocab_size, (B, S + 1)).astype(np.int64)
    a = OracleDecoder(CFG, w, B, 32)
    a.prefill(ids[:, :S])
    logits_step, _ = a.decode_step(ids[:, S], np.full((3, B), S, np.int64))
    b = OracleDecoder(CFG, w, B, 32)
    logits_full, _ = b.prefill(ids)
    np.testing.assert_allclose(logits_step, logits_full, rtol=0, atol=1e-5)
    assert list(a.lens) == [S + 1] * B
    for i in range(CFG.num_hidden_layers):
        np.testing.assert_array_equal(a.k[i][:, :, : S + 1].view(np.uint16), b.k[i][:, :, : S + 1].view(np.uint16))


def test_single_layer_wiring_against_numpy():
    """One layer, one token, written out with plain NumPy in fp64 (fp16 rounding points included)."""
    cfg = TextConfig(num_hidden_layers=1, hidden_size=32, num_attention_heads=2, num_key_value_heads=1, head_dim=16,
                     intermediate_size=48, vocab_size=20, mrope_section=[4, 2, 2])
    w = random_weights(cfg, 3)
    rng = np.random.default_rng(4)
    for k in w:
        if "norm" in k:
            w[k] = (1 + 0.1 * rng.standard_normal(w[k].shape)).astype(np.float32)
    dec = OracleDecoder(cfg, w, 1, 8)
    tok, pos = 7, 0  # position 0: RoPE is the identity, a single key: attention returns v
    logits, _ = dec.decode_step(np.array([tok]), np.zeros((3, 1), np.int64))

    def h16(x):
        return np.asarray(x, np.float64).astype(np.float16).astype(np.float64)

    def rms(x, wt, eps=1e-6):
        return x / np.sqrt((x ** 2).mean(-1, keepdims=True) + eps) * wt

    W = {k: np.asarray(v, np.float64) for k, v in w.items()}
    h = W["embed_tokens.weight"][tok]
    xn = rms(h, W["layers.0.input_layernorm.weight"])
    qkv = h16(xn) @ W["layers.0.self_attn.qkv_proj.weight"].T
    v = h16(qkv[48:64])                      # 2 q heads (32) + 1 k head (16) precede v
    attn = np.concatenate([v, v])            # both q heads read the single kv head's only value row
    o = h16(attn) @ W["layers.0.self_attn.o_proj.weight"].T
    h = h + o
    xn2 = rms(h, W["layers.0.post_attention_layernorm.weight"])
    gu = h16(xn2) @ W["layers.0.mlp.gate_up_proj.weight"].T
    act = gu[:48] / (1 + np.exp(-gu[:48])) * gu[48:]
    h = h + h16(act) @ W["layers.0.mlp.down_proj.weight"].T
    want = h16(rms(h, W["norm.weight"])) @ W["embed_tokens.weight"].T
    np.testing.assert_allclose(logits[0], want, rtol=0, atol=2e-5)


def test_f64_operator_set_agrees_with_the_fp32_oracle_operators():
    """oracle/f64_ops.py (the float64 yardstick) against the restatement, operator by operator, on random
    inputs: they evaluate the same functions, so they agree to fp32 rounding."""
    from oracle import port
    from oracle.f64_ops import F64Ops

    f = F64Ops()
    rng = np.random.default_rng(12)
    q = rng.standard_normal((3, 4, 16)).astype(np.float32)
    k = rng.standard_normal((7, 2, 16)).astype(np.float32)
    v = rng.standard_normal((7, 2, 16)).astype(np.float32)
    for causal in (False, True):
        np.testing.assert_allclose(f.sdpa(q, k, v, causal), port.sdpa(q, k, v, causal), rtol=0, atol=2e-6)
    x = rng.standard_normal((5, 64)).astype(np.float32)
    r = rng.standard_normal((5, 64)).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(64)).astype(np.float32)
    np.testing.assert_allclose(f.rms_norm(x, w, 1e-6), port.rms_norm(x, w, 1e-6), rtol=0, atol=2e-6)
    np.testing.assert_allclose(f.rms_norm(x, None, 1e-5), port.rms_norm(x, None, 1e-5), rtol=0, atol=2e-6)
    y64, o64 = f.add_rms_norm(x, r, w, 1e-6)
    y32, o32 = port.add_rms_norm(x, r, w, 1e-6)
    np.testing.assert_allclose(y64, y32, rtol=0, atol=1e-6)
    np.testing.assert_allclose(o64, o32, rtol=0, atol=2e-6)
    np.testing.assert_allclose(f.silu_mul(x, r), port.silu_mul(x, r), rtol=0, atol=2e-6)
    wl = (0.1 * rng.standard_normal((9, 64))).astype(np.float32)
    np.testing.assert_allclose(f.linear(x, wl), port.linear(x, wl), rtol=0, atol=1e-5)
    b = rng.standard_normal(9).astype(np.float32)
    np.testing.assert_allclose(f.linear(x, wl, b), port.linear(x, wl, b), rtol=0, atol=1e-5)
    # M-RoPE with distinct (t, h, w) positions and sections that leave some channels on T
    xr = rng.standard_normal((6, 3, 16)).astype(np.float32)
    pos = rng.integers(0, 50, (3, 6)).astype(np.int64)
    inv = port.rope_inv_freq(1e4, 16)
    np.testing.assert_allclose(f.rope_thd(xr, pos, inv, [4, 2, 2]), port.rope_thd(xr, pos, inv, [4, 2, 2]), rtol=0,
                               atol=5e-6)
    ids = rng.integers(0, 5, 8)
    np.testing.assert_array_equal(f.embedding(ids, x), port.embedding(ids, x).astype(np.float64))
    np.testing.assert_array_equal(f.argmax(x), port.argmax(x))


def test_f64_decode_step_is_the_same_op_sequence():
    """The float64 evaluation of a prefill + decode step stays within fp32-rounding distance of the fp32
    restatement on a shallow model (where fp16 boundary flips have no depth to grow in), and keeps the
    cache-vs-longer-prefill identity itself."""
    from oracle.f64_ops import F64Ops

    w = _weights(2)
    rng = np.random.default_rng(6)
    B, S = 2, 7
    ids = rng.integers(0, CFG.vocab_size, (B, S + 1)).astype(np.int64)
    a32 = OracleDecoder(CFG, w, B, 32)
    a64 = OracleDecoder(CFG, w, B, 32, ops=F64Ops())
    a32.prefill(ids[:, :S])
    a64.prefill(ids[:, :S])
    pos = np.full((3, B), S, np.int64)
    l32, _ = a32.decode_step(ids[:, S], pos)
    l64, _ = a64.decode_step(ids[:, S], pos)
    assert l64.dtype == np.float64
    assert np.abs(l64 - l32).max() <= 2e-3     # two layers: at most a few fp16 flips of 1 ulp each
    b64 = OracleDecoder(CFG, w, B, 32, ops=F64Ops())
    full64, _ = b64.prefill(ids)
    np.testing.assert_allclose(l64, full64, rtol=0, atol=1e-9)
