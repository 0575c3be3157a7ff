"""Preallocated contiguous per-layer KV cache.

The reference grows its cache by ``torch.cat`` every step and every layer
(metaseq/modules/multihead_attention.py:449-479), re-copying the whole history.  Here each
layer owns one fp16 tensor ``[2, B, H, S_cap, hd]`` (K then V) that the QKV kernel appends to
in place; ``length`` counts the valid positions (columns of the token history).  A "ragged"
cache (prefilled from right-padded prompts, or filled slot by slot) stores every row without
pads and keeps the per-row lengths in ``lens`` (int32 [B] on the device, negative = empty
slot).  The object lives inside the caller-owned
``incremental_state`` dict, as the reference's per-module buffers do
(metaseq/incremental_decoding_utils.py:30-69), and is freed with it.
"""
import weakref

import torch


class KVCache:
    def __init__(self, n_layers, batch, heads, head_dim, capacity, device):
        self.n_layers, self.batch, self.heads, self.head_dim = n_layers, batch, heads, head_dim
        self.capacity = int(capacity)
        self.length = 0
        self.device = device
        self.has_pads = False
        self.ragged = False
        self.lens = None  # int32 [B] device tensor when ragged
        self.layers = [
            torch.empty(2, batch, heads, self.capacity, head_dim, dtype=torch.float16,
                        device=device)
            for _ in range(n_layers)
        ]

    def k(self, i):
        return self.layers[i][0]

    def v(self, i):
        return self.layers[i][1]

    def rows_view(self, b0, b1):
        """Rows b0 .. b1 - 1 as a cache of their own (a decode step taken in row chunks); the
        same object for the same range, so that work buffers kept on it persist."""
        views = self.__dict__.setdefault("_row_views", {})
        if (b0, b1) not in views:
            views[(b0, b1)] = _RowsView(self, b0, b1)
        return views[(b0, b1)]

    def grow(self, new_capacity):
        """Reallocates every layer to ``new_capacity`` positions, keeping the valid prefix."""
        new_capacity = int(new_capacity)
        if new_capacity <= self.capacity:
            return
        for i, old in enumerate(self.layers):
            new = torch.empty(2, self.batch, self.heads, new_capacity, self.head_dim,
                              dtype=torch.float16, device=self.device)
            new[:, :, :, :self.length].copy_(old[:, :, :, :self.length])
            self.layers[i] = new
        self.capacity = new_capacity

    def bytes(self):
        return sum(t.numel() * 2 for t in self.layers)


class _RowsView:
    """Rows b0 .. b1 - 1 of a ``KVCache`` with what a decode step reads of a cache: ``k(i)``,
    ``v(i)`` (contiguous slices of the parent's current tensors), ``capacity``, ``device``."""

    def __init__(self, cache, b0, b1):
        # a weak reference: the cache keeps its views, and must still be freed by its last
        # outside reference going away, not by a later garbage-collection pass
        self._cache, self._b0, self._b1 = weakref.proxy(cache), b0, b1
        self.device = cache.device

    @property
    def capacity(self):
        return self._cache.capacity

    def k(self, i):
        return self._cache.layers[i][0][self._b0:self._b1]

    def v(self, i):
        return self._cache.layers[i][1][self._b0:self._b1]
