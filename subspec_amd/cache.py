"""KV caches shared by the target and the substitute draft, with the reference's
``KVManager`` interface (specdecodes/models/utils/cache_utils.py:41-60): ``seq_len``,
``get_seq_length()``, ``crop()``, ``reorder_cache_with_offset(beam_idx, new_chunk_len, offset, dim)``,
``reset()``.  ``StaticKVCache`` stands for ``TreeStaticCache`` (:113-208), ``DynamicKVCache`` for
``TreeDynamicCache`` (:62-110): no fixed length, storage grows as rows are written, and a reorder
truncates to the kept rows.

Layout: ONE tensor ``[layers, 2 (K, V), batch, kv_heads, max_cache_len, head_dim]`` so that
compaction after verification is a single kernel launch over ``layers * 2 * batch * kv_heads`` slabs
(the reference stacks and copies back every layer's full cache, cache_utils.py:199-208).  Storage
addresses never change; rows beyond the accepted block are left stale, as in the reference.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import ops


class StaticKVCache:
    growable = False

    def __init__(self, n_layers: int, n_kv_heads: int, head_dim: int, max_cache_len: int, device, dtype,
                 max_batch_size: int = 1):
        self.max_cache_len = int(max_cache_len)
        self.data = torch.zeros((n_layers, 2, max_batch_size, n_kv_heads, self.max_cache_len, head_dim),
                                device=device, dtype=dtype)

    def k(self, layer: int) -> torch.Tensor:
        return self.data[layer, 0]

    def v(self, layer: int) -> torch.Tensor:
        return self.data[layer, 1]

    def ensure(self, n_rows: int) -> None:
        """Called before a forward that touches cache rows below ``n_rows``."""
        if n_rows > self.max_cache_len:
            raise ValueError(f"the static cache holds {self.max_cache_len} rows, {n_rows} are needed")

    def write(self, layer: int, positions: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> None:
        """k, v: [B, Hkv, n, D] written at cache rows ``positions`` (int64 [n])."""
        self.data[layer, 0].index_copy_(2, positions, k)
        self.data[layer, 1].index_copy_(2, positions, v)

    contiguous = True                          # k(i) / v(i) are [B, Hkv, S, D] views the one-call layers can take

    def prefix_kv(self, layer: int, n_rows: int):
        """K and V of rows 0 .. n_rows - 1 as [B, Hkv, n_rows, D] (the causal prefill reads them)."""
        return self.data[layer, 0][:, :, :n_rows], self.data[layer, 1][:, :, :n_rows]

    def tree_attention(self, layer: int, q: torch.Tensor, anc_bits: torch.Tensor, prefix_len: int, n_tree_slots: int):
        return ops.tree_attention(q, self.k(layer), self.v(layer), anc_bits, prefix_len, n_tree_slots=n_tree_slots)

    def reset(self) -> None:
        self.data.zero_()

    def crop(self, start: int, end: Optional[int] = None, dim: int = 2) -> None:
        if end is None or end <= start:
            return
        self.data[..., start:end, :] = 0

    def reorder_cache_with_offset(self, beam_idx: torch.Tensor, new_chunk_len: int = 1, offset: int = 0, dim: int = 2,
                                  count_dev: Optional[torch.Tensor] = None) -> None:
        """rows offset+j <- offset+beam_idx[j] in every layer, K and V (cache_utils.py:166-208).
        ``beam_idx`` may live on the host (reference call style) or on the device together with a
        device-side count (no host round trip)."""
        if beam_idx.device != self.data.device:
            beam_idx = beam_idx.to(self.data.device)
        ops.kv_compact_(self.data, beam_idx.to(torch.int64).contiguous(), int(offset), count_dev=count_dev,
                        max_count=None if count_dev is None else min(int(beam_idx.numel()), ops.L.MAX_TREE_NODES))


class DynamicKVCache(StaticKVCache):
    """The same single-tensor layout without a fixed length (``TreeDynamicCache``, cache_utils.py:62-110): the
    capacity doubles whenever a forward needs more rows (one reallocation and copy, amortised), ``crop`` and
    ``reorder_cache_with_offset`` set the number of rows seen, as the reference's slicing / index_select do;
    the kernels are the static cache's.  ``max_cache_len`` is the current capacity."""

    growable = True

    def __init__(self, n_layers: int, n_kv_heads: int, head_dim: int, device, dtype, max_batch_size: int = 1,
                 initial_len: int = 1024):
        super().__init__(n_layers, n_kv_heads, head_dim, max(64, int(initial_len)), device, dtype, max_batch_size)
        self._seen_tokens = 0

    def ensure(self, n_rows: int) -> None:
        if n_rows <= self.max_cache_len:
            return
        new_len = max(2 * self.max_cache_len, (int(n_rows) + 255) // 256 * 256)
        shape = list(self.data.shape)
        shape[-2] = new_len
        grown = torch.zeros(shape, device=self.data.device, dtype=self.data.dtype)
        grown[..., :self.max_cache_len, :] = self.data
        self.data, self.max_cache_len = grown, new_len

    def get_seq_length(self) -> int:
        return self._seen_tokens

    def reset(self) -> None:
        self._seen_tokens = 0

    def crop(self, start: int, end: Optional[int] = None, dim: int = 2) -> None:
        if end is not None and start < 0:
            start = end - abs(start)
        self._seen_tokens = start                            # rows beyond are simply no longer part of the cache

    def reorder_cache_with_offset(self, beam_idx: torch.Tensor, new_chunk_len: int = 1, offset: int = 0, dim: int = 2,
                                  count_dev: Optional[torch.Tensor] = None) -> None:
        """[:offset] unchanged, rows offset + beam_idx[j] follow, everything else is dropped (:92-110)."""
        super().reorder_cache_with_offset(beam_idx, new_chunk_len, offset, dim, count_dev=count_dev)
        if count_dev is None:                                # with a device-side count the caller sets the length
            self._seen_tokens = int(offset) + int(beam_idx.numel())


class KVManager:
    def __init__(self, cache: StaticKVCache):
        self.cache = cache
        self.seq_len = 0

    def get_seq_length(self) -> int:
        return self.seq_len

    def crop(self, start: int, end: Optional[int] = None, dim: int = 2) -> None:
        self.cache.crop(start, self.get_seq_length() if end is None else end, dim)

    def reorder_cache_with_offset(self, beam_idx, new_chunk_len=1, offset=0, dim=0, count_dev=None):
        self.cache.reorder_cache_with_offset(beam_idx, new_chunk_len, offset, dim, count_dev=count_dev)

    def reset(self) -> None:
        self.cache.reset()
        self.seq_len = 0


def create_kv_cache(cache_implementation: str = "static", max_cache_len: Optional[int] = None,
                    max_batch_size: Optional[int] = 1, config=None, device="cuda:0", dtype=torch.bfloat16) -> KVManager:
    """Factory with the reference's signature (cache_utils.py:6-39).  For the dynamic cache ``max_cache_len`` is only
    the initial capacity.  ``"paged"`` (not a choice of the reference's factory, whose paged path has generators of
    its own) puts the same interface over a page pool: one request's pages, 16 tokens each."""
    if isinstance(dtype, str):
        if not hasattr(torch, dtype):
            raise ValueError(f"Unsupported dtype string: {dtype}")
        dtype = getattr(torch, dtype)
    if cache_implementation not in ("static", "dynamic", "paged"):
        raise ValueError(f"Unsupported cache_implementation: {cache_implementation}")
    if config is None:
        # the reference's dynamic cache learns its shapes from the first update; this one allocates up front
        raise ValueError("config must be provided (layer count and head shapes of the cache)")
    if cache_implementation == "dynamic":
        return KVManager(DynamicKVCache(config.num_hidden_layers, config.num_key_value_heads, config.head_dim, device, dtype,
                                        max_batch_size or 1, initial_len=max_cache_len or 1024))
    if cache_implementation == "paged":
        if max_cache_len is None:
            raise ValueError("max_cache_len must be provided for the paged cache (it sizes the page pool)")
        from .paged_cache import PagedKVCache
        return KVManager(PagedKVCache(config.num_hidden_layers, config.num_key_value_heads, config.head_dim,
                                      max_cache_len, device, dtype))
    if max_cache_len is None:
        raise ValueError("max_cache_len must be provided for static cache")
    return KVManager(StaticKVCache(config.num_hidden_layers, config.num_key_value_heads, config.head_dim,
                                   max_cache_len, device, dtype, max_batch_size or 1))
