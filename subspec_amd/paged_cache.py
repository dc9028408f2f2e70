"""Paged KV cache with the reference's pool / request interface
(specdecodes/models/utils/flashinfer/cache_manager.py:35-348): ``KvCachePool`` owns
``cache_data [layers, max_pages, 2, page_len, kv_heads, head_dim]`` and a free-page map,
``RequestKvCache`` owns one sequence's page list and length.  Same method names, argument meaning
and error behaviour; the device work goes to the paged HIP entry points:

* ``RequestKvCache.attention`` -> ``subspec_tree_attention_paged`` (the reference plans a FlashInfer
  ``BatchPrefillWithPagedKVCacheWrapper`` with a custom mask per forward);
* ``reorder_cache_with_offset`` -> ``subspec_kv_compact_paged``: one launch for all layers, rows
  addressed through the request's page table (the reference clones every layer, reorders the pool
  as if the request owned pages 0, 1, 2, ... and copies everything back).

Page bookkeeping is host-side Python, as in the reference.
"""
from __future__ import annotations

import math
from typing import List, Optional

import torch

from . import ops


class KvCachePool:
    def __init__(self, max_pages: int, num_layers: int, num_heads: int, head_dim: int, page_len: int,
                 dtype: torch.dtype, device):
        if page_len <= 0 or page_len & (page_len - 1):
            raise ValueError(f"page_len={page_len} must be a power of two (the kernels split a row index with a shift)")
        self.cache_data = torch.zeros(num_layers, max_pages, 2, page_len, num_heads, head_dim, dtype=dtype, device=device)
        self.num_layers, self.device, self.max_pages, self.page_len = num_layers, torch.device(device), max_pages, page_len
        self.free_page_mask = torch.ones(max_pages, dtype=torch.bool, device="cpu")
        self.num_heads, self.head_dims, self.dtype = num_heads, head_dim, dtype

    def reset(self) -> None:
        self.cache_data.zero_()

    def num_free_pages(self):
        return self.free_page_mask.sum()

    def allocate(self, num_pages: int) -> List[int]:
        free = self.free_page_mask.nonzero()
        assert len(free) >= num_pages, f"Out of available cache pages: asked {num_pages}, only {len(free)} free pages"
        taken = free[:num_pages]
        self.free_page_mask[taken] = False
        return taken.squeeze(1).tolist()

    def deallocate(self, kv_page_indices: List[int]) -> None:
        self.free_page_mask[kv_page_indices] = True

    def crop(self, seq_len: int) -> None:
        """Zero everything after ``seq_len`` tokens of pages 0, 1, 2, ... and free the unused pages (:83-119)."""
        if not (0 <= seq_len <= self.max_pages * self.page_len):
            raise ValueError(f"seq_len={seq_len} is outside the [0, {self.max_pages * self.page_len}] range.")
        full, rem = divmod(seq_len, self.page_len)
        keep = full + (1 if rem else 0)
        if rem:
            self.cache_data[:, full, :, rem:].zero_()
        if keep < self.max_pages:
            self.cache_data[:, keep:].zero_()
        self.free_page_mask.zero_()
        if keep < self.max_pages:
            self.free_page_mask[keep:] = True

    def reorder_cache_with_offset(self, beam_idx: torch.Tensor, offset: int = 0, num_new_tokens: int = 0,
                                  page_indices: Optional[torch.Tensor] = None, count_dev: Optional[torch.Tensor] = None) -> None:
        """Logical rows offset + j <- offset + beam_idx[j] in every layer, K and V (:120-213).  Without
        ``page_indices`` the rows are those of pages 0, 1, 2, ..., as in the reference."""
        total_pages = (offset + num_new_tokens + self.page_len - 1) // self.page_len
        if total_pages > self.max_pages:
            raise ValueError(f"Cache does not have enough pages ({self.max_pages}) for total tokens ({offset + num_new_tokens}).")
        if page_indices is None:
            need = max(1, (offset + max(int(beam_idx.numel()), num_new_tokens) + self.page_len - 1) // self.page_len)
            page_indices = torch.arange(min(need, self.max_pages), dtype=torch.int32, device=self.device)
        beam_idx = beam_idx.to(self.device).to(torch.int64).contiguous()
        ops.kv_compact_paged_(self.cache_data, page_indices, beam_idx, int(offset), count_dev=count_dev,
                              max_count=None if count_dev is None else min(int(beam_idx.numel()), ops.L.MAX_TREE_NODES))


class RequestKvCache:
    def __init__(self, kvCachePool: KvCachePool, page_len: int, seq_init_len: int):
        self.kvCachePool, self.page_len = kvCachePool, page_len
        init_num_pages = math.ceil(seq_init_len / self.page_len)
        self.kv_last_page_len = seq_init_len - (init_num_pages - 1) * self.page_len
        self.kv_page_indices = kvCachePool.allocate(init_num_pages)
        self.kv_len = seq_init_len
        self.is_released = False

    def get_seq_length(self) -> int:
        return self.kv_len

    def increment(self, num_tokens: int = 1) -> None:
        self.kv_len += num_tokens
        self.kv_last_page_len += num_tokens
        while self.kv_last_page_len > self.page_len:
            self.kv_last_page_len -= self.page_len
            self.kv_page_indices.extend(self.kvCachePool.allocate(1))

    def release(self) -> None:
        self.kvCachePool.deallocate(self.kv_page_indices)
        self.is_released = True

    def _set_len(self, kv_len: int, allow_growth: bool) -> None:
        self.kv_len = kv_len
        self.kv_last_page_len = 0 if kv_len == 0 else (kv_len - 1) % self.page_len + 1
        needed = (kv_len + self.page_len - 1) // self.page_len
        if len(self.kv_page_indices) > needed:
            self.kvCachePool.deallocate(self.kv_page_indices[needed:])
            self.kv_page_indices = self.kv_page_indices[:needed]
        elif len(self.kv_page_indices) < needed:
            self.kv_page_indices.extend(self.kvCachePool.allocate(needed - len(self.kv_page_indices)))
            if not allow_growth:
                raise ValueError("need to allocate new pages in reorder cache, should not happen")

    def decrement(self, num_tokens: int = 1) -> None:
        if num_tokens <= 0:
            return
        self._set_len(self.kv_len - min(num_tokens, self.kv_len), allow_growth=True)

    def crop(self, start: int, end: Optional[int] = None, dim: int = 0) -> None:
        if end is None:
            end = self.get_seq_length()
        if start < 0:
            start = end - abs(start)
        if end <= start:
            return
        self._set_len(start, allow_growth=False)

    # ------------------------------------------------------------------ device side
    def page_table(self, extra_tokens: int = 0) -> torch.Tensor:
        """The request's pages (int32, device), grown first so that ``extra_tokens`` more rows fit."""
        need = (self.kv_len + extra_tokens + self.page_len - 1) // self.page_len
        if need > len(self.kv_page_indices):
            self.kv_page_indices.extend(self.kvCachePool.allocate(need - len(self.kv_page_indices)))
        return torch.tensor(self.kv_page_indices, dtype=torch.int32, device=self.kvCachePool.device)

    def append(self, layer: int, k: torch.Tensor, v: torch.Tensor, first_row: Optional[int] = None) -> torch.Tensor:
        """Writes ``k``, ``v`` [n, kv_heads, head_dim] at logical rows first_row.. (default: the current length)
        of one layer, what ``flashinfer.append_paged_kv_cache`` does in the reference
        (attention_wrapper.py:235-254).  Does not change the length; returns the page table used."""
        first = self.kv_len if first_row is None else int(first_row)
        n = k.shape[0]
        table = self.page_table(max(0, first + n - self.kv_len))
        rows = torch.arange(first, first + n, device=k.device)
        pages, toks = table.long()[rows // self.page_len], rows % self.page_len
        data = self.kvCachePool.cache_data
        data[layer, pages, 0, toks] = k
        data[layer, pages, 1, toks] = v
        return table

    def attention(self, layer: int, q: torch.Tensor, anc_bits: torch.Tensor, prefix_len: int,
                  n_tree_slots: Optional[int] = None, table: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Tree attention of ``q`` [1, Hq, n, D] over this request's rows of one layer."""
        slots = q.shape[2] if n_tree_slots is None else n_tree_slots
        table = self.page_table(max(0, prefix_len + slots - self.kv_len)) if table is None else table
        return ops.tree_attention_paged(q, self.kvCachePool.cache_data[layer], table, anc_bits, prefix_len, n_tree_slots=slots)

    def reorder_cache_with_offset(self, beam_idx: torch.Tensor, offset: int = 0, num_new_tokens: int = 0) -> None:
        """Keeps rows offset + beam_idx[j] as rows offset + j and sets the length to offset + len(beam_idx).
        As in the reference (:315-318) a non-zero ``offset`` is first reduced by one: its callers pass the
        sequence length including the token whose K/V row is the root of the tree."""
        if offset != 0:
            offset -= 1
        table = self.page_table(max(0, offset + max(int(beam_idx.numel()), num_new_tokens) - self.kv_len))
        self.kvCachePool.reorder_cache_with_offset(beam_idx, offset, num_new_tokens, page_indices=table)
        self._set_len(offset + int(beam_idx.size(0)), allow_growth=False)


class PagedKVCache:
    """One sequence over a page pool behind the interface the decoder and the cycle drivers use for the static cache
    (``ensure``, ``write``, ``prefix_kv``, ``tree_attention``, ``reorder_cache_with_offset``, ``crop``, ``reset``):
    the alternative cache layout of the reference's FlashInfer path serving the same speculative cycle.  Rows are
    logical positions; pages are taken from the pool as rows are first needed, in whatever order the pool hands them
    out, and the page table goes to the kernels as it is."""
    growable = False
    contiguous = False

    def __init__(self, n_layers: int, n_kv_heads: int, head_dim: int, max_cache_len: int, device, dtype, page_len: int = 16):
        self.page_len = int(page_len)
        max_pages = (int(max_cache_len) + self.page_len - 1) // self.page_len
        self.max_cache_len = max_pages * self.page_len
        self.pool = KvCachePool(max_pages, n_layers, n_kv_heads, head_dim, self.page_len, dtype, device)
        self.request = RequestKvCache(self.pool, self.page_len, 0)
        self._table: Optional[torch.Tensor] = None

    # ---- pages
    def ensure(self, n_rows: int) -> None:
        if n_rows > self.max_cache_len:
            raise ValueError(f"the page pool holds {self.max_cache_len} rows, {n_rows} are needed")
        need = (int(n_rows) + self.page_len - 1) // self.page_len
        pages = self.request.kv_page_indices
        if need > len(pages):
            pages.extend(self.pool.allocate(need - len(pages)))
            self._table = None

    def table(self) -> torch.Tensor:
        if self._table is None or self._table.numel() != len(self.request.kv_page_indices):
            self._table = torch.tensor(self.request.kv_page_indices, dtype=torch.int32, device=self.pool.device)
        return self._table

    # ---- rows
    def write(self, layer: int, positions: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> None:
        """k, v: [1, Hkv, n, D] written at logical rows ``positions`` (int64 [n])."""
        table = self.table().long()                       # the caller has sized the cache with ensure()
        pages, toks = table[positions // self.page_len], positions % self.page_len
        data = self.pool.cache_data
        data[layer, pages, 0, toks] = k[0].transpose(0, 1)
        data[layer, pages, 1, toks] = v[0].transpose(0, 1)

    def prefix_kv(self, layer: int, n_rows: int):
        rows = torch.arange(n_rows, device=self.pool.device)
        table = self.table().long()
        pages, toks = table[rows // self.page_len], rows % self.page_len
        kv = self.pool.cache_data[layer, pages, :, toks]                  # [n_rows, 2, Hkv, D]
        return kv[:, 0].transpose(0, 1).unsqueeze(0), kv[:, 1].transpose(0, 1).unsqueeze(0)

    def tree_attention(self, layer: int, q: torch.Tensor, anc_bits: torch.Tensor, prefix_len: int, n_tree_slots: int):
        return ops.tree_attention_paged(q, self.pool.cache_data[layer], self.table(), anc_bits, prefix_len,
                                        n_tree_slots=n_tree_slots)

    def reorder_cache_with_offset(self, beam_idx: torch.Tensor, new_chunk_len: int = 1, offset: int = 0, dim: int = 2,
                                  count_dev: Optional[torch.Tensor] = None) -> None:
        self.pool.reorder_cache_with_offset(beam_idx, int(offset), 0, page_indices=self.table(), count_dev=count_dev)

    def crop(self, start: int, end: Optional[int] = None, dim: int = 2) -> None:
        """Rows from ``start`` on leave the cache: whole pages behind them go back to the pool."""
        keep = (max(int(start), 0) + self.page_len - 1) // self.page_len
        pages = self.request.kv_page_indices
        if keep < len(pages):
            self.pool.deallocate(pages[keep:])
            del pages[keep:]
            self._table = None

    def reset(self) -> None:
        self.crop(0)
