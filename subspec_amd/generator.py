"""Cycle driver: speculate -> tree decode -> verify -> KV compaction.

Keeps the reference's generator surface (specdecodes/models/generators/base.py:156-197 ``generate``,
classic_sd.py:12-134 ``ClassicSDGeneratorBase`` incl. ``generator_kwargs = {prefill_chunk_size,
verify_method, verify_kwargs}``, subspec_sd.py:10-126 ``_generate``) for the greedy and the sampling
target (``do_sample``, ``temperature``, ``top_k``, ``top_p``: base.py:42-64,156-197), and the
metrics contract of ``SDProfilingMixin`` (specdecodes/models/utils/mixin.py:181-224,267-269,318-349:
``avg_draft_time``, ``avg_target_time``, ``avg_verify_time``, ``avg_sampled``, ``n_iter``,
``n_tokens``, ``elapsed_time``, ``tput``).

Per cycle the host synchronises once, to read the few accepted tokens it needs for the stop
criteria; verification and KV compaction are queued back to back on the device (the compaction
kernel reads the accepted-row count from device memory).
"""
from __future__ import annotations

import time
from typing import Any, Optional

import torch

from . import ops
from .cache import DynamicKVCache, KVManager
from .lossy_diagnostics import record_lossy_diagnostics
from .tree_verify import SampleStream, sample_token, verify_tree_device
from .utils import DraftParams
from .wandb_logger import wandb_logger


class SubSpecSDGenerator:
    def __init__(self, target_model, tokenizer=None, draft_model=None, draft_params: Optional[DraftParams] = None,
                 cache_implementation: str = "static", profiling: bool = True, profiling_verbose: bool = False,
                 generator_kwargs: Optional[dict] = None, eos_token_id: Optional[int] = None):
        self.target_model, self.tokenizer, self.draft_model = target_model, tokenizer, draft_model
        self.draft_params = draft_params or DraftParams()
        self.draft_model.draft_params = self.draft_params
        if cache_implementation not in ("static", "dynamic", "paged"):
            raise ValueError(f"Unsupported cache_implementation: {cache_implementation}")
        self.cache_implementation = cache_implementation
        self.profiling = profiling
        self.generator_kwargs = generator_kwargs or {}
        self.prefill_chunk_size = self.generator_kwargs.get("prefill_chunk_size", None)
        self.eos_token_id = eos_token_id if eos_token_id is not None else getattr(tokenizer, "eos_token_id", None)
        self.draft_model.eos_token_id = self.eos_token_id
        if "draft_graph" in self.generator_kwargs:       # replay each speculation from a captured graph (static cache)
            self.draft_model.capture_graphs = bool(self.generator_kwargs["draft_graph"])
        # Philox stream of the sampling target; generator_kwargs["seed"] fixes it, else torch's seed
        self.sample_stream = SampleStream(self.generator_kwargs.get("seed"))
        self._stop_strings = None                # HuggingFace StopStringCriteria of the current generate() call

    def eval(self) -> "SubSpecSDGenerator":
        """The reference's generators are ``nn.Module``s and the builder calls ``generator.eval()``
        (run/core/builder.py:359); nothing here has a training mode."""
        return self

    def _bind(self, past_key_values: KVManager) -> None:
        """Models handed over by the reference's builder are HuggingFace-shaped modules (quantized / offloaded by the
        recipe); they become ``Decoder``s over the cache of this call.  ``Decoder``s are re-bound to it."""
        from .hf_model import as_decoder
        self.target_model = as_decoder(self.target_model, past_key_values)
        self.draft_model.set_past_key_values(past_key_values)

    # ------------------------------------------------------------------ pieces of one cycle
    def _speculate(self, input_ids):
        return self.draft_model.speculate(input_ids)

    def _tree_decoding(self, tree, past_key_values: KVManager, position_offset: int):
        dev = self.target_model.device
        packed = tree.packed()
        anc = ops.ancestor_bits_tensor(packed["parent_indices"].tolist())
        n = anc.shape[0]
        # one host-to-device copy: token ids, depths and the mask words of every node side by side
        both = torch.cat([packed["token_ids"].long().view(n, 1), packed["depths"].long().view(n, 1), anc.view(n, -1)],
                         dim=1).to(dev, non_blocking=True)
        bits = both[:, 2].contiguous() if both.shape[1] == 3 else both[:, 2:].contiguous()
        return self.target_model.tree_forward(both[:, 0].contiguous(), both[:, 1].contiguous(), bits, position_offset)

    def _get_logits_processor(self, temperature: float = 1.0, top_k: Optional[int] = None, top_p: Optional[float] = None):
        """The HuggingFace warpers of multinomial sampling, in the reference's order and under its
        conditions (generators/base.py:42-64): temperature unless None or 1, top-k unless None or
        0, top-p unless None or >= 1."""
        from transformers.generation.logits_process import (LogitsProcessorList, TemperatureLogitsWarper,
                                                            TopKLogitsWarper, TopPLogitsWarper)
        warpers = LogitsProcessorList()
        if temperature is not None and temperature != 1.0:
            warpers.append(TemperatureLogitsWarper(temperature))
        if top_k is not None and top_k != 0:
            warpers.append(TopKLogitsWarper(top_k=top_k))
        if top_p is not None and top_p < 1.0:
            warpers.append(TopPLogitsWarper(top_p=top_p))
        return warpers

    def _sample_token(self, logits, logits_processor, do_sample: bool, return_probs: bool = False):
        return sample_token(logits, logits_processor, do_sample, return_probs, stream=self.sample_stream)

    def _verify(self, tree, root_ind, logits, logits_processor=None, do_sample=False, skip_nodes=0):
        method = str(self.generator_kwargs.get("verify_method", "exact") or "exact").strip().lower()
        if method not in ("exact", "lossy"):
            raise ValueError(f"Unsupported verify_method: {method!r} (supported: 'exact', 'lossy')")
        return verify_tree_device(tree=tree, root_ind=int(root_ind), logits=logits, eos_token_id=self.eos_token_id,
                                  skip_nodes=int(skip_nodes), verify_method=method,
                                  verify_kwargs=dict(self.generator_kwargs.get("verify_kwargs") or {}),
                                  logits_processor=logits_processor, do_sample=bool(do_sample),
                                  stream=self.sample_stream)

    def _chunked_prefill_forward(self, input_ids: torch.Tensor, past_key_values: KVManager):
        """Prefill in chunks of ``prefill_chunk_size`` (generators/base.py:204-263); returns the last logits."""
        start = past_key_values.get_seq_length()
        todo = input_ids[0, start:]
        chunk = todo.numel() if self.prefill_chunk_size is None else min(todo.numel(), int(self.prefill_chunk_size))
        logits = None
        for s in range(0, todo.numel(), chunk):
            piece = todo[s:s + chunk]
            logits = self.target_model.prefill(piece, past_key_values.get_seq_length())
            past_key_values.seq_len += piece.numel()
        return logits

    # ------------------------------------------------------------------ public API
    @torch.no_grad()
    def generate(self, input_ids: torch.LongTensor, temperature=None, top_p=None, top_k=None, max_new_tokens=None,
                 max_length=None, do_sample=False, stop_strings=None, stream_callback=None, **model_kwargs):
        self._stop_strings = None
        if stop_strings is not None:                          # generators/base.py:94-101
            if self.tokenizer is None:
                raise ValueError("There are one or more stop strings in the arguments to `generate`, but the generator has "
                                 "no tokenizer: pass the model's tokenizer to the generator when generating with stop strings.")
            from transformers.generation.stopping_criteria import StopStringCriteria
            self._stop_strings = StopStringCriteria(stop_strings=stop_strings, tokenizer=self.tokenizer)
        if max_new_tokens is not None:
            max_length = input_ids.shape[1] + int(max_new_tokens)
        past_key_values = model_kwargs.get("past_key_values")
        if max_length is None and (self.cache_implementation == "static" or
                                   not isinstance(getattr(past_key_values, "cache", None), DynamicKVCache)):
            raise ValueError("max_length is not set. Only 'dynamic' kv-cache is supported when max_length is unspecified.")
        if past_key_values is None:
            raise ValueError("past_key_values is not provided")
        assert input_ids.shape[0] == 1, "Only support batch_size=1 for now."
        logits_processor = (self._get_logits_processor(temperature=temperature, top_p=top_p, top_k=top_k)
                            if do_sample else None)
        return self._generate(input_ids.clone(), None if max_length is None else int(max_length), past_key_values, stream_callback,
                              logits_processor=logits_processor, do_sample=bool(do_sample))

    def _generate(self, input_ids, max_length: Optional[int], past_key_values: KVManager, stream_callback=None,
                  logits_processor=None, do_sample: bool = False):
        self._bind(past_key_values)
        dev = self.target_model.device
        input_ids = input_ids.to(dev)
        p = self.draft_params
        ev = lambda: torch.cuda.Event(enable_timing=True)
        phases = {"draft": [], "target": [], "verify": []}
        t_start = time.perf_counter()
        org_len = input_ids.shape[1]

        logits = self._chunked_prefill_forward(input_ids, past_key_values)
        sampled = self._sample_token(logits.view(1, 1, -1), logits_processor, do_sample).view(1, 1)
        input_ids = torch.cat([input_ids, sampled], dim=-1)
        if stream_callback is not None:
            stream_callback(sampled)

        n_iter = sampled_count = 0
        finished = self._hit_stop(input_ids, sampled, max_length)[0]
        while not finished:
            e = [ev() for _ in range(4)]
            e[0].record()
            tree = self._speculate(sampled[:, -1:].clone())
            e[1].record()
            prev_kv_len = past_key_values.get_seq_length()
            logits = self._tree_decoding(tree, past_key_values, position_offset=input_ids.shape[1] - 1)
            e[2].record()
            out = self._verify(tree, 0, logits, logits_processor, do_sample)
            # KV rows of the accepted path move up right behind the verifier, count read on the device
            past_key_values.reorder_cache_with_offset(out["contexts"][0], new_chunk_len=p.max_verify_tokens,
                                                      offset=prev_kv_len, dim=2, count_dev=out["counts"][0, 0:1])
            e[3].record()
            host = torch.cat([out["counts"][0].long(), out["tokens"][0], out["contexts"][0]]).cpu()   # the one sync
            emitted, accept, _, status = (int(v) for v in host[:4])
            if status:
                raise RuntimeError(f"verifier reported a malformed tree (status {status})")
            n = tree.size()
            sampled = host[4:4 + emitted].view(1, -1).to(dev)
            if self.generator_kwargs.get("verify_method") == "lossy":
                vk = dict(self.generator_kwargs.get("verify_kwargs") or {})
                record_lossy_diagnostics(
                    tree=tree, skip_nodes=0, target=out["target"][0].cpu(), entropy=out["entropy"][0].cpu(),
                    child_prob=out["child_prob"][0].cpu(), tokens=host[4:4 + emitted],
                    contexts=host[5 + n:5 + n + emitted], accept_len=accept, eos_token_id=self.eos_token_id,
                    threshold=float(vk.get("threshold", 0.0)), window_size=int(vk.get("window_size", 1)),
                    threshold_method=str(vk.get("threshold_method", "prob") or "prob").strip().lower())
            input_ids = torch.cat([input_ids, sampled], dim=-1)
            finished, input_ids, kept, prune_tokens = self._hit_stop(input_ids, sampled, max_length,
                                                                     host_tokens=host[4:4 + emitted].tolist())
            if stream_callback is not None and kept.numel() > 0:
                stream_callback(kept)
            past_key_values.seq_len += emitted
            if finished:
                past_key_values.seq_len -= prune_tokens
            n_iter += 1
            sampled_count += emitted
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
                    "avg_sampled": sampled_count / n_iter if n_iter else 0.0})
        if self.profiling:
            for name, pairs in phases.items():
                log[f"avg_{name}_time"] = (sum(a.elapsed_time(b) for a, b in pairs) / len(pairs) / 1e3) if pairs else 0.0
        return input_ids

    def _hit_stop(self, input_ids, sampled_tokens, max_length: int, host_tokens=None):
        """Token-by-token stop check over the new block (generators/base.py:265-299): returns
        (finished, input_ids cut after the stop, kept tokens, number of pruned tokens).  ``host_tokens``: the same
        tokens as a host-side list, when the caller has them (saves a device synchronisation per cycle)."""
        base = input_ids.shape[1] - sampled_tokens.shape[1]
        toks = sampled_tokens[0].tolist() if host_tokens is None else list(host_tokens)
        for j, t in enumerate(toks):
            cur_len = base + j + 1
            stop = (max_length is not None and cur_len >= max_length) or \
                (self.eos_token_id is not None and t == int(self.eos_token_id))
            if not stop and getattr(self, "_stop_strings", None) is not None:
                stop = bool(self._stop_strings(input_ids[:, :cur_len], None).any())    # the text so far ends in a stop string
            if stop:
                prune = len(toks) - j - 1
                if prune > 0:
                    input_ids = input_ids[:, :-prune]
                return True, input_ids, sampled_tokens[:, :len(toks) - prune], prune
        return False, input_ids, sampled_tokens, 0
