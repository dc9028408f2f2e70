"""Oracle: KV-cache compaction.  Test infrastructure only.

Follows specdecodes/models/utils/cache_utils.py:166-208 (static cache: gather with index_select,
then index_copy_ into [offset, offset+L); everything else untouched) and :85-103 (dynamic cache:
the same gather, truncated to offset+L).
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
