"""Substitute draft: the target's own weights quantized to int4, expanding a top-k tree level by
level on the device.

Keeps the method surface of the reference's draft wrapper (``speculate``, ``speculate_once``,
``topk_sampling``, ``init_postspec`` / ``postspec`` / ``update_tree_after_post``,
``set_past_key_values``; specdecodes/models/draft_models/subspec_sd.py:23-145,
classic_sd.py:10-118, base.py:268-305).  Differences in mechanism:

* softmax(logits / T) stays a torch call, the cumulative-probability product and the global top-k
  over (leaves x vocab) are one fused HIP launch (no ``[1, k, V]`` product buffer);
* the incremental ``[1, 1, k, max_cache_len]`` boolean mask of ``TreeMaskCache`` (base.py:49-117) is
  replaced by an ancestor bitset per node (eight 64-bit words: up to 512 tree slots, the 289 nodes of the
  reference's depth-48 x 6 trees plus what post-speculation adds), updated on the device with a gather
  and an OR; a forward is handed only the words its occupied slots need;
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

MAX_SLOTS = ops.L.MAX_TREE_NODES          # tree slots the attention masks describe
MASK_WORDS = MAX_SLOTS // 64


class SubSpecSDDraftModel:
    def __init__(self, decoder, eos_token_id: Optional[int] = None):
        # ``model``: a ``Decoder``, or the HuggingFace-shaped module the reference's builder quantizes in place through
        # ``draft_model.model`` (run/core/builder.py:340-341); the latter becomes a ``Decoder`` once the cache is known
        self.model = decoder
        self._decoder: Optional[Decoder] = decoder if isinstance(decoder, Decoder) else None
        self.eos_token_id = eos_token_id
        self.draft_params: Optional[DraftParams] = None
        self.past_key_values = None
        self.had_first_speculate = False
        self.postspec_count = 0
        # Graph replay of speculate(): the reference captures its draft step into a CUDA graph with device-side
        # positions (draft_models/subspec_sd_fi.py:65-179); here ALL levels of one speculation are one captured graph
        # per prefix bucket, replayed with the prefix length in device memory.  Off unless asked for.
        self.capture_graphs = False
        self.graph_bucket = 256                   # a graph serves prefixes up to the next multiple of this
        self.graph_warmup = 2                     # eager speculations before the first capture (library handles, tables)
        self.max_graphs = 8                       # captured buckets kept (each pins its level tensors and a workspace)
        self._graphs = {}
        self._eager_speculations = 0
        self.graph_replays = 0

    @classmethod
    def from_pretrained(cls, pretrained_model_name_or_path=None, *model_args, target_model=None,
                        torch_dtype=torch.float32, **model_kwargs) -> "SubSpecSDDraftModel":
        """The reference's constructor for the substitute draft (draft_models/subspec_sd.py:29-45): no checkpoint of
        its own, a second module tree over ``target_model``'s parameters (``hf_model.share_parameters``) that a
        recipe's quantizer then converts; ``eos_token_id`` and ``device_map`` are taken from the keyword arguments
        the builder passes (run/core/builder.py:119-131).  The target's dtype is kept: the shared parameters are the
        target's own tensors, so there is nothing to convert."""
        if target_model is None:
            raise ValueError("SubSpecSDDraftModel.from_pretrained needs target_model (the draft shares its weights)")
        if isinstance(target_model, Decoder):
            raise TypeError("a Decoder target has its draft built by subspec_amd.model.build_models; from_pretrained "
                            "takes the HuggingFace-shaped module the builder loads")
        from .hf_model import share_parameters
        return cls(share_parameters(target_model), eos_token_id=model_kwargs.pop("eos_token_id", None))

    @property
    def decoder(self) -> Decoder:
        if self._decoder is None:
            raise RuntimeError("the draft has no KV cache yet: call set_past_key_values(past_key_values) first "
                               "(generate() does)")
        return self._decoder

    def eval(self) -> "SubSpecSDDraftModel":
        return self

    def set_past_key_values(self, past_key_values) -> None:
        if past_key_values is not self.past_key_values:
            self._graphs.clear()                  # a captured graph holds the addresses of the cache it was recorded over
        self.past_key_values = past_key_values
        if past_key_values is not None:
            from .hf_model import as_decoder
            self._decoder = as_decoder(self.model, past_key_values)

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
    def speculate(self, input_ids: torch.Tensor, cap: bool = True, **kwargs) -> Tree:
        """``input_ids`` [1, 1]: the root token; the cache already holds everything before it.  ``cap``: cut the
        tree to ``draft_params.max_verify_tokens`` nodes (the reference never cuts; a driver that goes on extending
        the tree must not, because the draft's level state describes the uncut level)."""
        assert input_ids.shape == (1, 1), "the root of the tree is a single token"
        self.had_first_speculate = True
        dev = self.decoder.device
        self.prefix_len = int(self.past_key_values.get_seq_length())
        self.tree = Tree(input_ids[0, -1], self.decoder.dtype)
        bound = self._graph_bound() if self.capture_graphs else None
        if bound is None or self._eager_speculations < self.graph_warmup:
            self._eager_speculations += 1
            self._grow_levels(input_ids[0].to(dev), self.prefix_len, None)
        else:
            self._replay_levels(input_ids[0].to(dev), bound)
        return self.update_tree(cap=cap)

    def _grow_levels(self, root: torch.Tensor, prefix_len: int, prefix_len_dev: Optional[torch.Tensor]) -> None:
        """All levels of one speculation, device work only (nothing is read back): the root's forward, then
        ``max_depth - 1`` tree steps.  With ``prefix_len_dev`` no launch depends on the actual prefix length."""
        dev = self.decoder.device
        self._prefix_len_dev, self._prefix_bound = prefix_len_dev, prefix_len
        pos32, rows32 = self._slot_tables(prefix_len, prefix_len_dev, rebuild=True)
        logits = self.decoder.tree_forward(root, torch.zeros(1, dtype=torch.long, device=dev),
                                           torch.ones(1, dtype=torch.int64, device=dev), prefix_len,
                                           prefix_len_dev=prefix_len_dev, positions32=pos32[0:1], rows32=rows32[0:1])
        self.levels = []
        self.level_state = {}                                                      # depth -> what speculate_once needs
        self.level_bits = self._own_bits(dev)[0:1].clone()                         # root: slot 0 (no host value involved)
        self.next_slot = 1
        self.depth = 0
        self._expand(self._probs(logits).unsqueeze(0), torch.ones((1, 1), device=dev, dtype=logits.dtype))
        for _ in range(self.draft_params.max_depth - 1):
            self.speculate_once()
        self._prefix_len_dev = None

    # ------------------------------------------------------------------ graph replay
    _STATE = ("levels", "level_state", "level_bits", "next_slot", "first_slot", "depth", "token_ids", "parent_probs")

    def _graph_bound(self) -> Optional[int]:
        """Upper bound of the prefix length the graph for the current prefix is laid out for, or None when this
        speculation cannot be replayed from a graph (cache that may move or is paged, layers not one-call, tree wider
        than a launch window, no room left in the cache)."""
        dec, p = self.decoder, self.draft_params
        cache = dec.kv.cache
        slots = 1 + (p.max_depth - 1) * p.topk_len
        if cache.growable or not cache.contiguous or not (dec.use_native_layers and dec.native_layers):
            return None
        if p.topk_len > 64 or slots > MAX_SLOTS:
            return None
        bound = (self.prefix_len // self.graph_bucket + 1) * self.graph_bucket
        bound = min(bound, cache.max_cache_len - slots)
        return bound if bound >= self.prefix_len else None

    def _replay_levels(self, root: torch.Tensor, bound: int) -> None:
        """A captured graph is bound to the memory its kernels were recorded over: the KV cache storage, the decoder's
        layer workspace, the rotary tables, the weights.  The cache storage and the decoder are part of a graph's
        identity (another cache, or a cache whose storage moved, never replays it), and every entry owns its workspace and
        keeps the tensors of its capture alive, so an eager call that replaces the decoder's workspace cannot pull
        memory from under a graph."""
        dec = self.decoder
        cache = dec.kv.cache
        key = (bound, self.draft_params.max_depth, self.draft_params.topk_len, float(self.draft_params.temperature),
               id(dec), int(cache.data.data_ptr()))
        entry = self._graphs.get(key)
        if entry is None:
            dev = dec.device
            self._own_bits(dev)                                                    # tables are built outside the capture
            cache.ensure(bound + 1 + (self.draft_params.max_depth - 1) * self.draft_params.topk_len)
            dec._rope_tables(bound + 1 + (self.draft_params.max_depth - 1) * self.draft_params.topk_len + 8)
            if len(self._graphs) >= self.max_graphs:                               # oldest bucket out
                self._graphs.pop(next(iter(self._graphs)))
            entry = {"root": torch.zeros(1, dtype=torch.long, device=dev),
                     "prefix": torch.zeros(1, dtype=torch.int64, device=dev), "graph": torch.cuda.CUDAGraph(),
                     "cache_data": cache.data, "rope": (dec.cos, dec.sin)}
            entry["root"].copy_(root)
            entry["prefix"].fill_(self.prefix_len)
            shared_ws = dec._native_ws.pop("ws", None) if dec.native_layers else None
            torch.cuda.synchronize()
            try:
                with torch.cuda.graph(entry["graph"]):
                    self._grow_levels(entry["root"], bound, entry["prefix"])
                entry["ws"] = dec._native_ws.get("ws")                             # allocated under the capture: the graph's own
            finally:
                if shared_ws is not None:
                    dec._native_ws["ws"] = shared_ws
                else:
                    dec._native_ws.pop("ws", None)
            entry["state"] = {name: getattr(self, name) for name in self._STATE}
            self._graphs[key] = entry
        entry["root"].copy_(root)
        entry["prefix"].fill_(self.prefix_len)
        entry["graph"].replay()
        self.graph_replays += 1
        for name, value in entry["state"].items():                                 # what the eager code leaves on the host
            setattr(self, name, dict(value) if isinstance(value, dict) else list(value) if isinstance(value, list) else value)

    def _own_bits(self, device) -> torch.Tensor:
        """Row s: the mask words with only the bit of slot s set (word s // 64, bit s % 64; bit 63 is the sign bit of
        the signed word).  Built once, so that a level costs one slice and one OR."""
        table = getattr(self, "_own_bits_table", None)
        if table is None or table.device != torch.device(device):
            slots = torch.arange(MAX_SLOTS)
            low = slots % 64
            bit = torch.where(low == 63, torch.full_like(slots, -(1 << 63)), torch.ones_like(slots) << low.clamp(max=62))
            words = torch.arange(MASK_WORDS)
            table = torch.where((slots // 64).unsqueeze(1) == words, bit.unsqueeze(1), torch.zeros_like(bit).unsqueeze(1))
            self._own_bits_table = table = table.to(device)
        return table

    def _slot_tables(self, prefix_len: int, prefix_len_dev: Optional[torch.Tensor], rebuild: bool = False):
        """Rotary position and cache row of every tree slot, int32 [MAX_SLOTS] each, for the current prefix: slot 0 is
        the root, slot s > 0 belongs to level 1 + (s - 1) // k.  Worked out once per speculation (two small launches);
        a level takes its slice.  Per level it was five launches of a few microseconds each on the level's critical
        path (fill, add, arange, two conversions)."""
        k = self.draft_params.topk_len
        dev = self.decoder.device
        const = getattr(self, "_slot_const", None)
        if const is None or const[0] != (k, str(dev)):
            slots = torch.arange(MAX_SLOTS, dtype=torch.int32)
            depth = torch.where(slots == 0, torch.zeros_like(slots), 1 + (slots - 1) // max(k, 1))
            const = self._slot_const = ((k, str(dev)), depth.to(dev), slots.to(dev))
        key = (k, int(prefix_len)) if prefix_len_dev is None else None      # a device-side prefix: rebuilt every time
        held = getattr(self, "_slot_held", None)
        if rebuild or key is None or held is None or held[0] != key:
            if prefix_len_dev is None:
                held = (key, const[1] + int(prefix_len), const[2] + int(prefix_len))
            else:
                held = (None, (const[1] + prefix_len_dev).to(torch.int32), (const[2] + prefix_len_dev).to(torch.int32))
            self._slot_held = held
        return held[1], held[2]

    def _expand(self, sampled_probs: torch.Tensor, parent_probs: torch.Tensor) -> None:
        k = self.draft_params.topk_len
        token_ids, child_probs, parent_indices = self.topk_sampling(sampled_probs, parent_probs, k)
        self.levels.append((token_ids, child_probs, parent_indices))
        self.token_ids, self.parent_probs = token_ids, child_probs
        own = self._own_bits(token_ids.device)[self.next_slot:self.next_slot + token_ids.shape[1]]
        self.level_bits = self.level_bits[parent_indices[0]] | own
        self.first_slot = self.next_slot
        self.next_slot += token_ids.shape[1]
        self.depth += 1
        self.level_state[self.depth] = (self.first_slot, self.token_ids, self.parent_probs, self.level_bits)

    @torch.no_grad()
    def speculate_once(self, **kwargs) -> None:
        """One more level: draft forward on the newest k nodes, then top-k over (k x vocab)."""
        dev = self.decoder.device
        n = self.token_ids.shape[1]
        total = self.first_slot + n
        if total > MAX_SLOTS:
            raise ValueError(f"draft tree exceeds the {MAX_SLOTS} tree slots of the attention mask")
        bits = self.level_bits[:, 0].contiguous() if total <= 64 else self.level_bits[:, :(total + 63) // 64].contiguous()
        dyn = getattr(self, "_prefix_len_dev", None)
        # inside _grow_levels the prefix length may live on the device; prefix_len is then the bound the launches use
        prefix = self._prefix_bound if dyn is not None else self.prefix_len
        tables = {}
        if n == self.draft_params.topk_len and self.first_slot == 1 + (self.depth - 1) * n:
            # the regular tree (every level k nodes): positions and rows are slices of the speculation's tables
            pos32, rows32 = self._slot_tables(prefix, dyn)
            tables = dict(positions32=pos32[self.first_slot:total], rows32=rows32[self.first_slot:total])
        depths = None if tables else torch.full((n,), self.depth, dtype=torch.long, device=dev)
        logits = self.decoder.tree_forward(self.token_ids[0], depths, bits, prefix,
                                           first_slot=self.first_slot, prefix_len_dev=dyn, **tables)
        self._expand(self._probs(logits).unsqueeze(0), self.parent_probs)

    def update_tree(self, cap: bool = False) -> Tree:
        tok = torch.stack([lv[0][0] for lv in self.levels]).unsqueeze(0)
        prob = torch.stack([lv[1][0] for lv in self.levels]).unsqueeze(0)
        par = torch.stack([lv[2][0] for lv in self.levels]).unsqueeze(0)
        packed = torch.stack([tok.double(), prob.double(), par.double()]).cpu()     # one device-to-host copy
        self.tree.add_nodes(packed[0].long(), packed[1].to(self.decoder.dtype), packed[2].long())
        self.levels = []
        limit = self.draft_params.max_verify_tokens if cap else None
        if limit is not None and self.tree.size() > limit:
            self.tree.truncate(limit)
        return self.tree

    # ------------------------------------------------------------------ post-speculation hooks
    def init_postspec(self, keep_pending: bool = False) -> None:
        """Start counting post-speculation steps; levels not yet attached to the tree are dropped unless kept."""
        if not keep_pending:
            self.levels = []
        self.postspec_count = 0

    @torch.no_grad()
    def prefeed(self) -> bool:
        """Runs the deepest level of the tree through the draft now and keeps the level it yields pending.  Done before
        the target decodes that level: a post-speculation step that fed it later would overwrite, in the layers the
        target has already passed, the target's K / V rows of nodes that may be accepted."""
        if not self._room_for_level():
            return False
        self.speculate_once()
        return True

    def _room_for_level(self) -> bool:
        """One more level needs tree slots (the masks describe ``MAX_SLOTS``) and, once it is decoded, cache rows."""
        n = self.token_ids.shape[1]
        if self.first_slot + n > MAX_SLOTS or self.next_slot + n > MAX_SLOTS:
            return False
        cache = self.decoder.kv.cache
        return cache.growable or self.prefix_len + self.next_slot + n <= cache.max_cache_len

    @torch.no_grad()
    def postspec(self) -> None:
        """One more level while the target is busy (subspec_sd.py:133-140); also a no-op once the tree slots
        the masks can describe, or the rows of a fixed-length cache, are used up."""
        if not self.had_first_speculate or self.postspec_count > (self.draft_params.max_depth - 1):
            return
        if not self._room_for_level():
            return
        self.speculate_once()
        self.postspec_count += 1

    def resync_to_depth(self, depth: int) -> None:
        """After the tree was pruned to ``depth``: continue from that level (its tokens, cumulative probabilities,
        masks and slots) instead of from the deeper level that no longer exists, and make exactly that level the
        tree's expandable frontier."""
        first, tokens, probs, bits = self.level_state[int(depth)]
        self.token_ids, self.parent_probs, self.level_bits = tokens, probs, bits
        self.first_slot, self.next_slot, self.depth = first, first + tokens.shape[1], int(depth)
        self.level_state = {d: v for d, v in self.level_state.items() if d <= depth}
        self.levels = []
        self.tree.available_leaves = list(range(first, first + tokens.shape[1]))

    def update_tree_after_post(self) -> Tree:
        return self.update_tree() if self.levels else self.tree
