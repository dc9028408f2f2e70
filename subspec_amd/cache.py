"""Static KV cache shared by the target and the substitute draft, with the reference's
``KVManager`` interface (specdecodes/models/utils/cache_utils.py:41-60): ``seq_len``,
``get_seq_length()``, ``crop()``, ``reorder_cache_with_offset(beam_idx, new_chunk_len, offset, dim)``,
``reset()``.

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
    def __init__(self, n_layers: int, n_kv_heads: int, head_dim: int, max_cache_len: int, device, dtype,
                 max_batch_size: int = 1):
        self.max_cache_len = int(max_cache_len)
        self.data = torch.zeros((n_layers, 2, max_batch_size, n_kv_heads, self.max_cache_len, head_dim),
                                device=device, dtype=dtype)

    def k(self, layer: int) -> torch.Tensor:
        return self.data[layer, 0]

    def v(self, layer: int) -> torch.Tensor:
        return self.data[layer, 1]

    def write(self, layer: int, positions: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> None:
        """k, v: [B, Hkv, n, D] written at cache rows ``positions`` (int64 [n])."""
        self.data[layer, 0].index_copy_(2, positions, k)
        self.data[layer, 1].index_copy_(2, positions, v)

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
                        max_count=None if count_dev is None else min(int(beam_idx.numel()), 256))


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
    """Factory with the reference's signature (cache_utils.py:6-39); only the static cache exists here."""
    if isinstance(dtype, str):
        if not hasattr(torch, dtype):
            raise ValueError(f"Unsupported dtype string: {dtype}")
        dtype = getattr(torch, dtype)
    if cache_implementation != "static":
        raise ValueError(f"Unsupported cache_implementation: {cache_implementation} (this build keeps the static cache)")
    if config is None:
        raise ValueError("config must be provided for static cache")
    if max_cache_len is None:
        raise ValueError("max_cache_len must be provided for static cache")
    return KVManager(StaticKVCache(config.num_hidden_layers, config.num_key_value_heads, config.head_dim,
                                   max_cache_len, device, dtype, max_batch_size or 1))
