"""Substitute draft: the target's own weights quantized to int4, expanding a top-k tree level by
level on the device.

Keeps the method surface of the reference's draft wrapper (``speculate``, ``speculate_once``,
``topk_sampling``, ``init_postspec`` / ``postspec`` / ``update_tree_after_post``,
``set_past_key_values``; specdecodes/models/draft_models/subspec_sd.py:23-145,
classic_sd.py:10-118, base.py:268-305).  Differences in mechanism:

* softmax(logits / T) stays a torch call, the cumulative-probability product and the global top-k
  over (leaves x vocab) are one fused HIP launch (no ``[1, k, V]`` product buffer);
* the incremental ``[1, 1, k, max_cache_len]`` boolean mask of ``TreeMaskCache`` (base.py:49-117) is
  replaced by one 64-bit ancestor bitset per node, updated on the device with a gather and an OR;
* nothing is copied to the host until the tree is assembled (one small copy, as in
  ``Tree.add_nodes``).
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import ops
from .cpu_tree import Tree
from .model import Decoder
from .utils import DraftParams


class SubSpecSDDraftModel:
    def __init__(self, decoder: Decoder, eos_token_id: Optional[int] = None):
        self.model = decoder
        self.eos_token_id = eos_token_id
        self.draft_params: Optional[DraftParams] = None
        self.past_key_values = None
        self.had_first_speculate = False
        self.postspec_count = 0

    def set_past_key_values(self, past_key_values) -> None:
        self.past_key_values = past_key_values

    def get_tree(self) -> Tree:
        return self.tree

    # ------------------------------------------------------------------ sampling
    @torch.no_grad()
    def topk_sampling(self, sampled_probs: torch.Tensor, parent_probs: torch.Tensor, sample_k: int
                      ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """(token_ids, topk_probs, parent_indices), each [B, k] (draft_models/base.py:268-305)."""
        return ops.topk_expand(sampled_probs.contiguous(), parent_probs.contiguous(), sample_k)

    def _probs(self, logits: torch.Tensor) -> torch.Tensor:
        return ops.softmax_temperature(logits, self.draft_params.temperature)       # classic_sd.py:10-16

    # ------------------------------------------------------------------ tree growth
    @torch.no_grad()
    def speculate(self, input_ids: torch.Tensor, **kwargs) -> Tree:
        """``input_ids`` [1, 1]: the root token; the cache already holds everything before it."""
        assert input_ids.shape == (1, 1), "the root of the tree is a single token"
        self.had_first_speculate = True
        p = self.draft_params
        dev = self.model.device
        self.prefix_len = int(self.past_key_values.get_seq_length())
        logits = self.model.tree_forward(input_ids[0].to(dev), torch.zeros(1, dtype=torch.long, device=dev),
                                         torch.ones(1, dtype=torch.int64, device=dev), self.prefix_len)
        self.tree = Tree(input_ids[0, -1], self.model.dtype)
        self.levels = []
        self.level_bits = torch.ones(1, dtype=torch.int64, device=dev)             # root: slot 0
        self.next_slot = 1
        self.depth = 0
        self._expand(self._probs(logits).unsqueeze(0), torch.ones((1, 1), device=dev, dtype=logits.dtype))
        for _ in range(p.max_depth - 1):
            self.speculate_once()
        return self.update_tree()

    def _expand(self, sampled_probs: torch.Tensor, parent_probs: torch.Tensor) -> None:
        k = self.draft_params.topk_len
        token_ids, child_probs, parent_indices = self.topk_sampling(sampled_probs, parent_probs, k)
        self.levels.append((token_ids, child_probs, parent_indices))
        self.token_ids, self.parent_probs = token_ids, child_probs
        slots = torch.arange(self.next_slot, self.next_slot + token_ids.shape[1], device=token_ids.device)
        usable = slots < 64                                                        # one mask word per node
        self_bit = torch.where(usable, torch.ones_like(slots) << slots.clamp(max=62), torch.zeros_like(slots))
        self_bit = torch.where(slots == 63, torch.full_like(slots, -(1 << 63)), self_bit)
        self.level_bits = self.level_bits[parent_indices[0]] | self_bit
        self.first_slot = self.next_slot
        self.next_slot += token_ids.shape[1]
        self.depth += 1

    @torch.no_grad()
    def speculate_once(self, **kwargs) -> None:
        """One more level: draft forward on the newest k nodes, then top-k over (k x vocab)."""
        dev = self.model.device
        n = self.token_ids.shape[1]
        if self.first_slot + n > 64:
            raise ValueError("draft tree exceeds 64 slots (max_depth * topk_len must stay below 64 for fed levels)")
        depths = torch.full((n,), self.depth, dtype=torch.long, device=dev)
        logits = self.model.tree_forward(self.token_ids[0], depths, self.level_bits, self.prefix_len,
                                         first_slot=self.first_slot)
        self._expand(self._probs(logits).unsqueeze(0), self.parent_probs)

    def update_tree(self) -> Tree:
        tok = torch.stack([lv[0][0] for lv in self.levels]).unsqueeze(0)
        prob = torch.stack([lv[1][0] for lv in self.levels]).unsqueeze(0)
        par = torch.stack([lv[2][0] for lv in self.levels]).unsqueeze(0)
        packed = torch.stack([tok.double(), prob.double(), par.double()]).cpu()     # one device-to-host copy
        self.tree.add_nodes(packed[0].long(), packed[1].to(self.model.dtype), packed[2].long())
        self.levels = []
        cap = self.draft_params.max_verify_tokens
        if cap is not None and self.tree.size() > cap:
            self.tree.truncate(cap)
        return self.tree

    # ------------------------------------------------------------------ post-speculation hooks
    def init_postspec(self) -> None:
        self.levels = []
        self.postspec_count = 0

    @torch.no_grad()
    def postspec(self) -> None:
        if not self.had_first_speculate or self.postspec_count > (self.draft_params.max_depth - 1):
            return
        self.speculate_once()
        self.postspec_count += 1

    def update_tree_after_post(self) -> Tree:
        return self.update_tree() if self.levels else self.tree
