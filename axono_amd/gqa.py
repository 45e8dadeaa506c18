"""Grouped-query decode attention (axono/python/axono/gqa.py): split-K flash-decoding over the KV
cache.  `gqa_decode_attention` is the reference's single-sequence call; `gqa_decode_attention_cache`
is the batched form over a static [B,Hkv,Lmax,D] cache with device-resident lengths."""
from . import libaxono as _l

__all__ = ["gqa_decode_attention", "gqa_decode_attention_cache"]


def gqa_decode_attention(q, k, v):
    """q (1, n_q_heads, head_dim); k / v (seq_len, n_kv_heads, head_dim) -> (1, n_q_heads, head_dim).
    Equals scaled_dot_product_attention(q, k, v, is_causal=False); scale 1/sqrt(head_dim)."""
    return _l.gqa_decode_attention(q, k, v)


def gqa_decode_attention_cache(q, k_cache, v_cache, seq_lens=None, max_len=None, out=None, workspace=None):
    return _l.gqa_decode_attention_cache(q, k_cache, v_cache, seq_lens, max_len, out, workspace)
