"""KV-cache components (axono/python/axono/nn/kv_cache.py).

`KVCache` is the abstract interface; `DynamicKVCache` is the default component (per layer, the
full k / v tensors, layout (seq, n_kv_head, d_head), grown along axis 0 by byte copies).
`PagedKVCache` grows by pages of 128 keys through a page table (memory follows the tokens that exist).
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
    """Interface of a KV-cache component (axono/python/axono/nn/kv_cache.py:41-68).  A model's attention
    layer calls `update(layer, k_new, v_new)` with the new tokens' keys / values and then
    `get(layer)` for everything cached so far; `reset()` starts a new conversation and `len()` is
    the number of cached positions.  User-written components subclass this."""

    def update(self, layer_idx: int, k_new, v_new):  # pragma: no cover - interface
        raise NotImplementedError(f"{type(self).__name__}.update")

    def get(self, layer_idx: int):  # pragma: no cover - interface
        raise NotImplementedError(f"{type(self).__name__}.get")

    def reset(self):  # pragma: no cover - interface
        raise NotImplementedError(f"{type(self).__name__}.reset")

    def __len__(self) -> int:  # pragma: no cover - interface
        raise NotImplementedError(f"{type(self).__name__}.__len__")


class _GrowableRows:
    """One tensor of rows (seq, ...) that grows along axis 0: a buffer with spare capacity plus the
    number of rows in use.  Appending copies only the new rows (byte copy at the end of the used
    part); the buffer is re-allocated with twice the capacity when it runs out, so the cost of n
    appends is O(n) rows moved instead of the O(n^2) of a concat per step."""

    __slots__ = ("buf", "rows", "row_shape")

    def __init__(self, first: Tensor, capacity: int):
        self.row_shape = first.shape[1:]
        self.rows = 0
        self.buf = Tensor(first.dtype, [capacity] + self.row_shape, first.device, _zero=False)
        self.append(first)

    def _row_bytes(self) -> int:
        return self.buf.num_bytes // self.buf.shape[0]

    def _copy_rows(self, dst: Tensor, dst_row: int, src: Tensor, n_rows: int) -> None:
        nbytes = n_rows * self._row_bytes()
        if nbytes == 0:
            return
        if dst.is_hip:
            _l.copy_bytes(dst, dst_row * self._row_bytes(), src, 0, nbytes)
        else:
            d = dst.to_numpy().reshape(-1).view(np.uint8)
            s = src.to_numpy().reshape(-1).view(np.uint8)
            d[dst_row * self._row_bytes():dst_row * self._row_bytes() + nbytes] = s[:nbytes]

    def append(self, new: Tensor) -> None:
        if new.shape[1:] != self.row_shape or new.dtype != self.buf.dtype:
            raise RuntimeError(f"KV cache append: rows of shape {new.shape[1:]} / {new.dtype.name} do not match the "
                               f"cached {self.row_shape} / {self.buf.dtype.name}")
        add = int(new.shape[0])
        cap = int(self.buf.shape[0])
        if self.rows + add > cap:
            bigger = Tensor(self.buf.dtype, [max(2 * cap, self.rows + add)] + self.row_shape, self.buf.device, _zero=False)
            self._copy_rows(bigger, 0, self.buf, self.rows)
            self.buf = bigger
        self._copy_rows(self.buf, self.rows, new, add)
        self.rows += add

    def view(self) -> Tensor:
        """The rows in use as a tensor [rows, ...] sharing the buffer's memory (a prefix of a
        contiguous row-major buffer is itself contiguous)."""
        return Tensor(self.buf.dtype, [self.rows] + self.row_shape, self.buf.device, _storage=self.buf._st)


class DynamicKVCache(KVCache):
    """The default component: per layer, all keys and all values so far as tensors
    (seq, n_kv_head, d_head); new tokens are appended along axis 0 by a byte copy, so cached values
    are bit-identical to an uncached forward (axono/python/axono/nn/kv_cache.py:71-117).

    Same observable behaviour as the reference's concat-per-step cache; the storage differs: each layer
    keeps a buffer with spare capacity and `get` returns tensors over its used prefix."""

    _FIRST_CAPACITY = 64

    def __init__(self, n_layers: int, device: str | None = None):
        self.n_layers = int(n_layers)
        self.device = device
        self._layers: dict = {}   # layer index -> (_GrowableRows for k, _GrowableRows for v)

    def _check_layer(self, layer_idx: int) -> int:
        li = int(layer_idx)
        if not 0 <= li < self.n_layers:
            raise IndexError(f"DynamicKVCache: layer {layer_idx} outside 0..{self.n_layers - 1}")
        return li

    def update(self, layer_idx: int, k_new, v_new) -> None:
        li = self._check_layer(layer_idx)
        if self.device is not None:
            k_new, v_new = k_new.to(self.device), v_new.to(self.device)
        entry = self._layers.get(li)
        if entry is None:
            cap = max(self._FIRST_CAPACITY, 2 * int(k_new.shape[0]))
            self._layers[li] = (_GrowableRows(k_new, cap), _GrowableRows(v_new, cap))
        else:
            entry[0].append(k_new)
            entry[1].append(v_new)

    def get(self, layer_idx: int):
        entry = self._layers.get(self._check_layer(layer_idx))
        if entry is None:
            raise RuntimeError(f"DynamicKVCache: layer {layer_idx} holds nothing yet (call update first, e.g. by running the prefill)")
        return entry[0].view(), entry[1].view()

    def reset(self) -> None:
        self._layers.clear()

    def __len__(self) -> int:
        """Cached positions of the lowest-numbered layer that holds any (every layer of a model is
        updated once per forward, so they agree)."""
        if not self._layers:
            return 0
        return self._layers[min(self._layers)][0].rows


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

    def note_advanced(self, n: int) -> None:
        """The device-side lengths were advanced by n outside `advance` (replays of a captured step): keeps the
        host-side view in step."""
        self._host_len += int(n)

    def reset(self) -> None:
        self.seq_lens.fill_zero()
        self._host_len = 0

    def __len__(self) -> int:
        """Host-side view of the longest sequence (kept in step with advance/set_lengths)."""
        return self._host_len


class PagedKVCache(KVCache):
    """KV cache of a batch of sequences that grows by pages of 128 keys instead of being allocated for
    batch x max_len rows up front.

    Per layer two pools [n_pages, n_kv_head, 128, d_head]; ONE page table INT32 [batch, max_pages] shared by
    all layers (page p of a sequence has the same page number in every layer's pool) and the lengths INT32
    [batch], both on the device (the attention kernel reads them) with host mirrors for the allocator.  Pages
    come from a free list; `free_sequence` returns a finished sequence's pages, so memory follows the tokens
    that exist.  `update` (one new token per sequence) and `update_rows` (many tokens of one sequence: its
    prefill) write through the page table; `attend` is decode attention over the pages, bit-identical to the
    dense cache's.  The lengths advance once per step, after the last layer (`advance`), as in
    StaticKVCache.  Page allocation uploads the page table, so inside a captured step call
    `reserve(tokens)` before capturing."""

    PAGE = _l.PAGE_KEYS

    def __init__(self, n_layers: int, batch: int, n_kv_head: int, d_head: int, n_pages: int, max_len: int,
                 dtype: DataType = DataType.FLOAT16, device: str = "hip", page_order=None):
        self.n_layers, self.batch, self.n_kv_head, self.d_head = int(n_layers), int(batch), int(n_kv_head), int(d_head)
        self.n_pages, self.max_len = int(n_pages), int(max_len)
        self.max_pages = (self.max_len + self.PAGE - 1) // self.PAGE
        self.dtype, self.device = DataType(dtype), device
        shape = [self.n_pages, self.n_kv_head, self.PAGE, self.d_head]
        self._k = [Tensor(dtype, shape, device) for _ in range(self.n_layers)]
        self._v = [Tensor(dtype, shape, device) for _ in range(self.n_layers)]
        self.page_table = Tensor(DataType.INT32, [self.batch, self.max_pages], device)
        self.seq_lens = Tensor(DataType.INT32, [self.batch], device)
        # page_order: the order in which physical pages are handed out (default 0, 1, 2, ...)
        order = list(range(self.n_pages)) if page_order is None else [int(p) for p in page_order]
        if sorted(order) != list(range(self.n_pages)):
            raise ValueError("page_order must be a permutation of range(n_pages)")
        self._order = order
        self.reset()

    # ---- page allocator (host) -----------------------------------------------------------------
    def reset(self) -> None:
        self._free = list(reversed(self._order))        # pop() hands out self._order[0] first
        self._table = np.full((self.batch, self.max_pages), -1, np.int32)
        self._lens = np.zeros(self.batch, np.int64)
        self._owned = np.zeros(self.batch, np.int64)     # pages each sequence holds
        self.page_table.copy_from_numpy(self._table)
        self.seq_lens.fill_zero()

    @property
    def pages_in_use(self) -> int:
        return self.n_pages - len(self._free)

    def reserve(self, new_tokens=1) -> None:
        """Makes sure every sequence has pages for its length + new_tokens (an int, or one int per
        sequence).  Raises MemoryError when the pool runs out (nothing is changed then)."""
        want = self._lens + np.broadcast_to(np.asarray(new_tokens, np.int64), (self.batch,))
        if np.any(want > self.max_len):
            raise ValueError(f"PagedKVCache: a sequence would exceed max_len = {self.max_len}")
        need = (want + self.PAGE - 1) // self.PAGE - self._owned
        need = np.maximum(need, 0)
        if int(need.sum()) == 0:
            return
        if int(need.sum()) > len(self._free):
            raise MemoryError(f"PagedKVCache: {int(need.sum())} pages needed, {len(self._free)} free of {self.n_pages}")
        for b in np.nonzero(need)[0]:
            for _ in range(int(need[b])):
                self._table[b, self._owned[b]] = self._free.pop()
                self._owned[b] += 1
        self.page_table.copy_from_numpy(self._table)

    def free_sequence(self, b: int) -> None:
        """Returns sequence b's pages to the free list and empties it."""
        n = int(self._owned[b])
        self._free.extend(int(p) for p in self._table[b, :n][::-1])
        self._table[b, :n] = -1
        self._owned[b] = 0
        self._lens[b] = 0
        self.page_table.copy_from_numpy(self._table)
        self.seq_lens.copy_from_numpy(self._lens.astype(np.int32))

    # ---- KVCache interface ---------------------------------------------------------------------
    def update(self, layer_idx: int, k_new, v_new) -> None:
        """One new token per sequence: k_new / v_new [batch, n_kv_head, d_head], written at each
        sequence's current length."""
        self.reserve(1)
        _l.kv_append_paged(k_new, v_new, self._k[layer_idx], self._v[layer_idx], self.page_table, self.seq_lens)

    def update_rows(self, layer_idx: int, b: int, k_rows, v_rows) -> None:
        """Many tokens of ONE sequence (its prefill): k_rows / v_rows [tokens, n_kv_head, d_head] - the
        reference cache's own layout - written from sequence b's current length on."""
        n = int(k_rows.shape[0])
        grow = np.zeros(self.batch, np.int64)
        grow[b] = n
        self.reserve(grow)
        _l.kv_append_paged(k_rows, v_rows, self._k[layer_idx], self._v[layer_idx], self.page_table, self.seq_lens,
                           tokens_per_sequence=n, table_row=b)

    def advance(self, n: int = 1) -> None:
        """Every sequence grew by n tokens (call once per step, after the last layer's update)."""
        self.reserve(max(int(n), 0))
        _l.index_add(self.seq_lens, n)
        self._lens += n

    def advance_rows(self, b: int, n: int) -> None:
        self._lens[b] += n
        self.seq_lens.copy_from_numpy(self._lens.astype(np.int32))

    def get(self, layer_idx: int):
        """(k_pool, v_pool) of the layer; together with `page_table` and `seq_lens` they are what
        gqa_decode_attention_paged takes."""
        return self._k[layer_idx], self._v[layer_idx]

    def attend(self, layer_idx: int, q, extra_tokens: int = 0, max_len: int | None = None):
        """Decode attention of q [batch, n_q_head, d_head] over the layer's cached keys (+ extra_tokens
        rows already written by `update` in this step but not yet counted by `advance`).  Everything
        runs on the device, so the call can be captured; a captured step passes `max_len`, the longest
        sequence any replay will see (the split plan is made from it), and reserves the pages for those
        tokens before capturing."""
        lens = self.seq_lens
        if extra_tokens:
            lens = Tensor(DataType.INT32, [self.batch], self.device, _zero=False)
            _l.copy_bytes(lens, 0, self.seq_lens, 0, 4 * self.batch)
            _l.index_add(lens, int(extra_tokens))
        bound = int(max_len) if max_len is not None else int(self._lens.max()) + int(extra_tokens)
        return _l.gqa_decode_attention_paged(q, self._k[layer_idx], self._v[layer_idx], self.page_table, lens,
                                             max(min(bound, self.max_len), 1))

    def set_lengths(self, lens) -> None:
        """Sets every sequence's length (pages for them must exist: `reserve` / `update_rows` first)."""
        lens = np.ascontiguousarray(lens, dtype=np.int64).reshape(self.batch)
        if np.any((lens + self.PAGE - 1) // self.PAGE > self._owned):
            raise ValueError("PagedKVCache.set_lengths: a sequence has fewer pages than its length needs")
        self._lens = lens.copy()
        self.seq_lens.copy_from_numpy(lens.astype(np.int32))

    def note_advanced(self, n: int) -> None:
        """The device-side lengths were advanced by n outside `advance` (replays of a captured step)."""
        self._lens += int(n)

    def sync_from_device(self) -> None:
        """Refreshes the host mirror of the lengths from the device tensor (after replays of a captured
        step, whose `advance` ran on the device only)."""
        self._lens = self.seq_lens.to_numpy().astype(np.int64)

    def __len__(self) -> int:
        return int(self._lens.max()) if self.batch else 0
