"""Cycle driver with post-speculation: while the target forward waits for streamed weights, the draft keeps
extending the tree; when the target ends up accepting a whole root-to-leaf path AND its bonus token is one of
the extension's nodes, the next cycle does not speculate from scratch but verifies the extension
(``SubSpecSDGeneratorBase._generate`` / ``_post_verify`` of specdecodes/models/generators/subspec_sd_v2.py:32-55,157-262,
driven by the wait hooks of specdecodes/helpers/offloaders/prefetch_offloader_postspec.py:193-232).

Same surface as the v1 driver (``generate``, ``generator_kwargs``, metrics) plus ``post_verify_count`` /
``speculate_count``.  What carries over from the reference exactly: the order of the steps, ``skip_nodes`` =
size of the part of the tree already verified, verification of tree nodes ``skip_nodes ..`` against logits of
those nodes only, ``root_ind = find_child_index(last accepted node, bonus token)``, KV compaction delayed until
a cycle fails to continue (or generation ends) with the accepted node indices accumulated, and ``_post_verify``:
the draft scores the extension once more, walks it greedily, the tree is pruned to the depth that walk
reaches and refilled to ``max_depth`` more levels.

Three things are not carried over as they are, and are decided here:

* How many post-speculation steps fit into a target forward depends, in the reference, on a host-side poll of the
  copy event -- on timing.  The same poll is used here (``generator_kwargs["postspec_steps"] = None``); an
  integer forces that many steps per target forward, which makes runs reproducible.  Whatever the number, the
  emitted tokens are the target's own greedy (or sampled) continuation: the extension only changes how many of
  them one cycle yields.
* The reference's first post-speculation step feeds the deepest level of the tree to the draft while the target is
  decoding the same nodes; draft and target share the cache, so in the layers the target has already passed the
  draft's K / V rows replace the target's for nodes that may be accepted.  Here that level is fed BEFORE the target
  forward (``prefeed``: one draft step that is not overlapped), every later step only touches rows of extension
  nodes, and the cache keeps exactly the target's rows.
* After ``prune_to_depth`` removed levels, the reference keeps expanding from the draft state of the removed
  deepest level and attaches the new nodes to whatever leaves come first in index order.  Here the draft state is
  first set back to the deepest level that survived (``resync_to_depth``), so new levels hang below it.

Tree and extension together may occupy 512 tree slots (eight mask words per row); once they are used up, or a
fixed-length cache has no rows left, post-speculation simply stops adding levels.
"""
from __future__ import annotations

import time
from typing import Optional

import torch

from . import ops
from .cache import KVManager
from .generator import SubSpecSDGenerator
from .lossy_diagnostics import record_lossy_diagnostics
from .wandb_logger import wandb_logger


class SubSpecSDGeneratorV2(SubSpecSDGenerator):
    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        steps = self.generator_kwargs.get("postspec_steps")
        self.postspec_steps: Optional[int] = None if steps is None else int(steps)
        self.post_verify_count = 0
        self.speculate_count = 0

    # ------------------------------------------------------------------ pieces
    def _speculate(self, input_ids):
        # No cut to max_verify_tokens here (subspec_sd_v2.py never prunes the fresh tree): the draft keeps extending
        # this tree from its deepest level, whose tokens, slots and masks describe the whole level.  A tree of more
        # than 64 nodes is decoded by the target module by module instead of through the one-call layers.
        return self.draft_model.speculate(input_ids, cap=False)

    def _window_forward(self, model, tree, position_offset: int, skip_nodes: int) -> torch.Tensor:
        """Forward of tree nodes ``skip_nodes ..`` (their cache rows are position_offset + node index)."""
        packed = tree.packed()
        anc = ops.ancestor_bits_tensor(packed["parent_indices"].tolist())          # [n] or [n, 2] above 64 nodes
        s = int(skip_nodes)
        dev = model.device
        return model.tree_forward(packed["token_ids"][s:].long().to(dev), packed["depths"][s:].long().to(dev),
                                  anc[s:].contiguous().to(dev), position_offset, first_slot=s, n_tree_slots=tree.size())

    def _postspec_while_copying(self, copy_done: torch.cuda.Event) -> None:
        """Idle hook of the layer streamer: draft levels into the gap before a slab arrives."""
        if self.postspec_steps is not None:
            return                                           # forced mode runs its steps elsewhere
        limit = self.draft_params.max_depth
        while self.draft_model.postspec_count < limit and not copy_done.query():
            before = self.draft_model.postspec_count
            self.draft_model.postspec()
            if self.draft_model.postspec_count == before:    # no room left for another level
                break

    def _target_decode(self, tree, position_offset: int, skip_nodes: int) -> torch.Tensor:
        self.draft_model.init_postspec(keep_pending=True)        # the prefed level is the first level of the extension
        streamer = getattr(self.target_model, "streamer", None)
        if streamer is not None:
            streamer.idle_hook = self._postspec_while_copying
        try:
            logits = self._window_forward(self.target_model, tree, position_offset, skip_nodes)
        finally:
            if streamer is not None:
                streamer.idle_hook = None
        if self.postspec_steps is not None:
            for _ in range(self.postspec_steps):
                self.draft_model.postspec()
        return logits

    def _verified(self, tree, root_ind: int, logits, logits_processor, do_sample: bool, skip_nodes: int):
        """(tokens, contexts, accept_len) on the host; one small device-to-host copy."""
        out = self._verify(tree, root_ind, logits, logits_processor, do_sample, skip_nodes=skip_nodes)
        n = tree.size()
        host = torch.cat([out["counts"][0].long(), out["tokens"][0], out["contexts"][0]]).cpu()
        emitted, accept, _, status = (int(v) for v in host[:4])
        if status:
            raise RuntimeError(f"verifier reported a malformed tree (status {status})")
        tokens, contexts = host[4:4 + emitted], host[5 + n:5 + n + emitted]
        if self.generator_kwargs.get("verify_method") == "lossy":
            vk = dict(self.generator_kwargs.get("verify_kwargs") or {})
            record_lossy_diagnostics(
                tree=tree, skip_nodes=int(skip_nodes), target=out["target"][0].cpu(), entropy=out["entropy"][0].cpu(),
                child_prob=out["child_prob"][0].cpu(), tokens=tokens, contexts=contexts, accept_len=accept,
                eos_token_id=self.eos_token_id, threshold=float(vk.get("threshold", 0.0)),
                window_size=int(vk.get("window_size", 1)),
                threshold_method=str(vk.get("threshold_method", "prob") or "prob").strip().lower())
        return tokens, contexts, accept

    def _post_verify(self, tree, root_ind: int, position_offset: int, last_tree_depth: int, skip_nodes: int):
        """subspec_sd_v2.py:32-55: the draft verifies the extension itself, the tree keeps the depth that walk reaches
        and is refilled."""
        draft = self.draft_model
        logits = self._window_forward(draft.decoder, tree, position_offset, skip_nodes)
        tokens, _, _ = self._verified(tree, root_ind, logits, None, False, skip_nodes)
        accepted_len = int(tokens.numel())
        tree.prune_to_depth(last_tree_depth + accepted_len)
        refill = self.draft_params.max_depth - accepted_len
        if refill > 0:
            depth = int(tree.get_depth())
            if depth != draft.depth:
                draft.resync_to_depth(depth)
            draft.init_postspec()
            for _ in range(refill):
                draft.postspec()
            tree = draft.update_tree_after_post()
        if self.postspec_steps != 0:
            draft.prefeed()
        return tree

    # ------------------------------------------------------------------ the loop
    def _generate(self, input_ids, max_length: Optional[int], past_key_values: KVManager, stream_callback=None,
                  logits_processor=None, do_sample: bool = False):
        p = self.draft_params
        if 1 + p.max_depth * p.topk_len > ops.L.MAX_TREE_NODES:
            raise ValueError(f"1 + max_depth * topk_len must not exceed the {ops.L.MAX_TREE_NODES} tree slots of the masks")
        self._bind(past_key_values)
        dev = self.target_model.device
        input_ids = input_ids.to(dev)
        ev = lambda: torch.cuda.Event(enable_timing=True)
        phases = {"draft": [], "target": [], "verify": []}
        t_start = time.perf_counter()
        org_len = input_ids.shape[1]

        logits = self._chunked_prefill_forward(input_ids, past_key_values)
        sampled = self._sample_token(logits.view(1, 1, -1), logits_processor, do_sample).view(1, 1)
        input_ids = torch.cat([input_ids, sampled], dim=-1)
        position_offset = input_ids.shape[1] - 1
        if stream_callback is not None:
            stream_callback(sampled)

        self.post_verify_count = self.speculate_count = 0
        n_iter = sampled_count = 0
        finished = self._hit_stop(input_ids, sampled, max_length)[0]
        is_prev_accepted = False
        hidden_cache: Optional[torch.Tensor] = None
        tree, root_ind = None, 0
        last_tree_size = last_tree_depth = 0
        while not finished:
            e = [ev() for _ in range(4)]
            e[0].record()
            if is_prev_accepted:
                self.post_verify_count += 1
                skip_nodes = last_tree_size
                tree = self._post_verify(tree, root_ind, position_offset, last_tree_depth, skip_nodes)
            else:
                self.speculate_count += 1
                tree = self._speculate(sampled[:, -1:].clone())
                if self.postspec_steps != 0:
                    self.draft_model.prefeed()
                skip_nodes = 0
                position_offset = input_ids.shape[1] - 1
            last_tree_size, last_tree_depth = tree.size(), int(tree.get_depth())
            e[1].record()
            logits = self._target_decode(tree, position_offset, skip_nodes)
            tree = self.draft_model.update_tree_after_post()
            e[2].record()
            root = root_ind if is_prev_accepted else 0
            tokens, contexts, _ = self._verified(tree, root, logits, logits_processor, do_sample, skip_nodes)
            e[3].record()
            last_accepted, bonus = int(contexts[-1]), int(tokens[-1])
            hidden_cache = torch.cat([hidden_cache, contexts]) if is_prev_accepted else contexts
            root_ind = tree.find_child_index(last_accepted, bonus)
            is_prev_accepted = root_ind >= 0

            sampled = tokens.view(1, -1).to(dev)
            input_ids = torch.cat([input_ids, sampled], dim=-1)
            finished, input_ids, kept, prune_tokens = self._hit_stop(input_ids, sampled, max_length, host_tokens=tokens.tolist())
            if stream_callback is not None and kept.numel() > 0:
                stream_callback(kept)
            if not is_prev_accepted or finished:
                # rows of every node accepted since the last speculation move up behind the prefix
                past_key_values.reorder_cache_with_offset(hidden_cache.to(dev), new_chunk_len=last_tree_size,
                                                          offset=past_key_values.get_seq_length(), dim=2)
                past_key_values.seq_len += int(hidden_cache.numel())
                if finished:
                    past_key_values.seq_len -= prune_tokens
            n_iter += 1
            sampled_count += int(tokens.numel())
            if self.profiling:
                phases["draft"].append((e[0], e[1]))
                phases["target"].append((e[1], e[2]))
                phases["verify"].append((e[2], e[3]))

        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t_start
        n_tokens = int(input_ids.shape[1] - org_len)
        log = wandb_logger.log_data
        log.update({"n_iter": n_iter, "n_tokens": n_tokens, "elapsed_time": elapsed,
                    "tput": n_tokens / elapsed if elapsed > 0 else 0.0,
                    "avg_sampled": sampled_count / n_iter if n_iter else 0.0,
                    "post_verify_count": self.post_verify_count, "speculate_count": self.speculate_count,
                    "post_verify_rate": (self.post_verify_count / (self.post_verify_count + self.speculate_count)
                                         if self.post_verify_count + self.speculate_count else 0.0)})   # mixin.py:341-347
        if self.profiling:
            for name, pairs in phases.items():
                log[f"avg_{name}_time"] = (sum(a.elapsed_time(b) for a, b in pairs) / len(pairs) / 1e3) if pairs else 0.0
        return input_ids
