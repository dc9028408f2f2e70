"""``DraftParams`` and ``invert_mask`` with the reference's definitions
(specdecodes/models/utils/utils.py:4-17)."""
from dataclasses import dataclass
from typing import Optional

import torch


def invert_mask(mask: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """bool "may attend" mask -> additive mask (0 where allowed, finfo.min where not)."""
    return (~mask).to(dtype) * torch.finfo(dtype).min


@dataclass
class DraftParams:
    temperature: float = 1
    max_depth: int = 6
    topk_len: int = 10
    max_verify_tokens: Optional[int] = None

    def __post_init__(self):
        self.max_sample_tokens = self.max_depth * self.topk_len + 1
        self.max_verify_tokens = (min(self.max_sample_tokens, self.max_verify_tokens)
                                  if self.max_verify_tokens is not None else self.max_sample_tokens)
