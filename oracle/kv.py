"""Oracle: KV-cache compaction.  Test infrastructure only.

Follows specdecodes/models/utils/cache_utils.py:166-208 (static cache: gather with index_select,
then index_copy_ into [offset, offset+L); everything else untouched) and :85-103 (dynamic cache:
the same gather, truncated to offset+L), and, for the paged pool of the FlashInfer path,
specdecodes/models/utils/flashinfer/cache_manager.py:120-213 (``KvCachePool.reorder_cache_with_offset``).
"""
import torch


def compact_static(cache: torch.Tensor, contexts, offset: int) -> torch.Tensor:
    """``cache``: [..., seq, d].  Returns a new tensor with rows offset+j <- offset+contexts[j]."""
    ctx = torch.as_tensor(contexts, dtype=torch.long)
    out = cache.clone()
    gathered = cache.index_select(-2, ctx + offset)          # temporary: sources read before any write
    out.index_copy_(-2, offset + torch.arange(ctx.numel()), gathered)
    return out


def compact_dynamic(cache: torch.Tensor, contexts, offset: int) -> torch.Tensor:
    ctx = torch.as_tensor(contexts, dtype=torch.long)
    full = torch.cat([torch.arange(offset), ctx + offset])
    return cache.index_select(-2, full)


def compact_paged_reference(pool: torch.Tensor, contexts, offset: int) -> torch.Tensor:
    """The reference's pool reorder, step by step (cache_manager.py:131-213): ``pool`` is
    [L, max_pages, 2, page_len, heads, d]; K and V planes are flattened over (page, token) as if the
    request owned pages 0, 1, 2, ..., gathered with index_select and written back with index_copy_."""
    L, max_pages, _, page_len, H, D = pool.shape
    ctx = torch.as_tensor(contexts, dtype=torch.long)
    old = ctx + offset
    new = torch.arange(offset, offset + ctx.numel())
    old_flat = (old // page_len) * page_len + old % page_len
    new_flat = (new // page_len) * page_len + new % page_len
    out = pool.clone()
    for kv in (0, 1):
        plane = pool[:, :, kv].clone().view(L, max_pages * page_len, H, D)
        plane.index_copy_(1, new_flat, plane.index_select(1, old_flat))
        out[:, :, kv] = plane.view(L, max_pages, page_len, H, D)
    return out


def compact_paged(pool: torch.Tensor, page_indices, contexts, offset: int) -> torch.Tensor:
    """The same reorder for a request whose logical row p sits in page ``page_indices[p // page_len]``:
    gather the request's rows into sequence order, compact them like the static cache, scatter them back.
    With the identity table this is ``compact_paged_reference``."""
    L, max_pages, _, page_len, H, D = pool.shape
    pages = torch.as_tensor(page_indices, dtype=torch.long)
    out = pool.clone()
    for kv in (0, 1):
        rows = pool[:, pages, kv].reshape(L, pages.numel() * page_len, H * D)          # [L, seq, H*D] in sequence order
        rows = compact_static(rows, contexts, offset)
        out[:, pages, kv] = rows.view(L, pages.numel(), page_len, H, D)
    return out


def gather_paged(pool_layer: torch.Tensor, page_indices, seq_len: int):
    """K and V of one pool layer [max_pages, 2, page_len, heads, d] as contiguous [1, heads, seq_len, d] tensors."""
    pages = torch.as_tensor(page_indices, dtype=torch.long)
    max_pages, _, page_len, H, D = pool_layer.shape
    k = pool_layer[pages, 0].reshape(-1, H, D)[:seq_len].transpose(0, 1).unsqueeze(0).contiguous()
    v = pool_layer[pages, 1].reshape(-1, H, D)[:seq_len].transpose(0, 1).unsqueeze(0).contiguous()
    return k, v
