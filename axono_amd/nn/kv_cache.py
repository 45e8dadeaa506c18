"""KV-cache components (axono/python/axono/nn/kv_cache.py).

`KVCache` is the abstract interface; `DynamicKVCache` is the reference's default (per layer, the
full k / v tensors, grown by concat along axis 0 — a byte copy, layout (seq, n_kv_head, d_head)).
`StaticKVCache` is this build's cache for the captured decode step: one pre-allocated
[B, n_kv_head, max_len, d_head] tensor pair per layer, device-resident lengths, and an append that
writes one row per (sequence, head) instead of re-copying the cache.
"""
from __future__ import annotations

import numpy as np

from .. import libaxono as _l
from ..core.tensor import Tensor
from ..core.types import DataType


class KVCache:
    def update(self, layer_idx: int, k_new, v_new):  # pragma: no cover
        raise NotImplementedError

    def get(self, layer_idx: int):  # pragma: no cover
        raise NotImplementedError

    def reset(self):  # pragma: no cover
        raise NotImplementedError

    def __len__(self) -> int:  # pragma: no cover
        raise NotImplementedError


class DynamicKVCache(KVCache):
    def __init__(self, n_layers: int, device: str | None = None):
        self.n_layers = n_layers
        self.device = device
        self._k = [None] * n_layers
        self._v = [None] * n_layers

    def update(self, layer_idx: int, k_new, v_new) -> None:
        if self._k[layer_idx] is None:
            self._k[layer_idx] = k_new
            self._v[layer_idx] = v_new
            return
        self._k[layer_idx] = _l.concat(self._k[layer_idx], k_new, 0)
        self._v[layer_idx] = _l.concat(self._v[layer_idx], v_new, 0)

    def get(self, layer_idx: int):
        if self._k[layer_idx] is None:
            raise RuntimeError("DynamicKVCache: 尚未 update (prefill 未执行?)")
        return self._k[layer_idx], self._v[layer_idx]

    def reset(self) -> None:
        self._k = [None] * self.n_layers
        self._v = [None] * self.n_layers

    def __len__(self) -> int:
        for k in self._k:
            if k is not None:
                return int(k.shape[0])
        return 0


class StaticKVCache(KVCache):
    """Pre-allocated cache for a batch of sequences.

    k/v of layer i: Tensor [B, n_kv_head, max_len, d_head] (FLOAT16 by default).  `seq_lens` is an
    INT32 device tensor [B] holding each sequence's current length; `update` appends the new token's
    k / v (shape [B, n_kv_head, d_head]) at position seq_lens[b] of every sequence.  The lengths are
    advanced once per step with `advance()` (after the last layer), on the device, so a captured step
    can be replayed."""

    def __init__(self, n_layers: int, batch: int, n_kv_head: int, max_len: int, d_head: int,
                 dtype: DataType = DataType.FLOAT16, device: str = "hip"):
        self.n_layers, self.batch, self.n_kv_head, self.max_len, self.d_head = n_layers, batch, n_kv_head, max_len, d_head
        self.dtype, self.device = DataType(dtype), device
        shape = [batch, n_kv_head, max_len, d_head]
        self._k = [Tensor(dtype, shape, device) for _ in range(n_layers)]
        self._v = [Tensor(dtype, shape, device) for _ in range(n_layers)]
        self.seq_lens = Tensor(DataType.INT32, [batch], device)
        self._host_len = 0

    def update(self, layer_idx: int, k_new, v_new) -> None:
        _l.kv_append(k_new, v_new, self._k[layer_idx], self._v[layer_idx], self.seq_lens)

    def get(self, layer_idx: int):
        return self._k[layer_idx], self._v[layer_idx]

    def advance(self, n: int = 1) -> None:
        _l.index_add(self.seq_lens, n)
        self._host_len += n

    def set_lengths(self, lens) -> None:
        lens = np.ascontiguousarray(lens, dtype=np.int32).reshape(self.batch)
        self.seq_lens.copy_from_numpy(lens)
        self._host_len = int(lens.max()) if lens.size else 0

    def reset(self) -> None:
        self.seq_lens.fill_zero()
        self._host_len = 0

    def __len__(self) -> int:
        """Host-side view of the longest sequence (kept in step with advance/set_lengths)."""
        return self._host_len
