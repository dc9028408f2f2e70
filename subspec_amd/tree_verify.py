"""``verify_tree`` with the reference's signature, backed by the fused HIP verifier.

Mirrors specdecodes/models/utils/tree_verify.py:8-163: same keyword arguments, same return value
``(sampled_tokens [1, L] cpu int64, hidden_indices [L] cpu int64, (total_len, accept_len))`` and
the same ``ValueError`` for an unknown ``verify_method`` / ``threshold_method``.  Differences:

* logits go straight to the device kernels; the ``[rows, V]`` probability tensor is never
  materialised nor copied to the host (the reference's dominant verify cost);
* with ``do_sample=True`` the target token of every scored row is drawn on the device by the
  verifier's Philox race (one draw per context, as in the reference's walk) instead of
  ``torch.multinomial`` on the host.  A lone ``TemperatureLogitsWarper`` is fused into the
  kernels; any other HuggingFace warper in ``logits_processor`` (top-k, top-p) is applied to the
  logits with its own device ops first.  ``sample_token_fn`` / ``verify_step_fn`` are accepted
  for signature compatibility and not called.

``verify_tree_device`` is the non-blocking form used by the cycle driver: it returns device
tensors so that KV compaction can be queued behind the verifier without a host round trip.
"""
from __future__ import annotations

from typing import Any, Dict, Optional, Tuple

import torch

from . import ops
from .lossy_diagnostics import record_lossy_diagnostics


def _tree_arrays(tree, device) -> Tuple[torch.Tensor, torch.Tensor]:
    if hasattr(tree, "packed"):
        d = tree.packed()
        tok, par = d["token_ids"], d["parent_indices"]
    else:                                   # any object with the reference Tree's get_tree_data()
        d = tree.get_tree_data()
        tok, par = d["token_ids"].to(torch.int32), d["parent_indices"].to(torch.int32)
    both = torch.stack([tok, par]).to(device, non_blocking=True)
    return both[0], both[1]


class SampleStream:
    """Seed and running offset of the verifier's Philox stream: every sampling call takes the next
    offset, so one seed reproduces a whole generation."""

    def __init__(self, seed: Optional[int] = None):
        self.seed = int(torch.initial_seed() if seed is None else seed)
        self.offset = 0

    def next(self) -> Tuple[int, int]:
        self.offset += 1
        return self.seed, self.offset - 1


_default_stream: Optional[SampleStream] = None


def default_stream() -> SampleStream:
    global _default_stream
    if _default_stream is None:
        _default_stream = SampleStream()
    return _default_stream


def split_warpers(logits_processor, logits: torch.Tensor) -> Tuple[torch.Tensor, float]:
    """(scores, temperature) for the sampling kernels: a processor list that only holds a
    ``TemperatureLogitsWarper`` (or nothing) is fused as the temperature; otherwise the whole list
    runs on the device as the reference runs it (generators/base.py:121-126) and the temperature
    left for the kernels is 1."""
    procs = list(logits_processor or [])
    if not procs:
        return logits, 1.0
    if len(procs) == 1 and type(procs[0]).__name__ == "TemperatureLogitsWarper":
        return logits, float(procs[0].temperature)
    flat = logits.reshape(-1, logits.shape[-1])
    return logits_processor(None, flat).reshape(logits.shape), 1.0


def sample_token(logits: torch.Tensor, logits_processor, do_sample: bool, return_probs: bool = False,
                 stream: Optional[SampleStream] = None) -> torch.Tensor:
    """``GeneratorBase._sample_token`` (generators/base.py:110-138) for ``logits [B, S, V]`` on the
    device: argmax, or one Philox draw per row."""
    if return_probs:
        if not do_sample:
            return torch.softmax(logits, dim=-1)
        scores, t = split_warpers(logits_processor, logits)
        return ops.softmax_temperature(scores, t) if t != 1.0 else torch.softmax(scores, dim=-1)
    if not do_sample:
        return torch.argmax(logits, dim=-1)
    scores, t = split_warpers(logits_processor, logits)
    seed, offset = (stream or default_stream()).next()
    return ops.sample_tokens(scores, t, seed, offset).view(logits.shape[:-1])


def verify_tree_device(*, tree, root_ind: int, logits: torch.Tensor, eos_token_id: Optional[int],
                       skip_nodes: int = 0, verify_method: str = "exact",
                       verify_kwargs: Optional[dict] = None, exact_entropy: bool = False,
                       workspace: Optional[torch.Tensor] = None, logits_processor=None, do_sample: bool = False,
                       stream: Optional[SampleStream] = None) -> Dict[str, torch.Tensor]:
    vk: dict[str, Any] = dict(verify_kwargs or {})
    tok, par = _tree_arrays(tree, logits.device)
    lg = logits[0] if logits.dim() == 3 else logits
    sampling = {}
    if do_sample:
        lg, t = split_warpers(logits_processor, lg)
        seed, offset = (stream or default_stream()).next()
        sampling = dict(do_sample=True, temperature=t, seed=seed, offset=offset)
    return ops.tree_verify(
        lg, tok, par, root=int(root_ind), skip_nodes=int(skip_nodes), eos_token_id=eos_token_id,
        verify_method=verify_method,
        threshold_method=str(vk.get("threshold_method", "prob") or "prob"),
        threshold=float(vk.get("threshold", 0.0)), window_size=int(vk.get("window_size", 1)),
        exact_entropy=exact_entropy, workspace=workspace, **sampling)


@torch.no_grad()
def verify_tree(*, tree, root_ind: int, logits: torch.Tensor, sample_token_fn=None, verify_step_fn=None,
                eos_token_id: Optional[int], logits_processor=None, do_sample: bool = False,
                skip_nodes: int = 0, verify_method: str = "exact",
                verify_kwargs: Optional[dict[str, Any]] = None, stream: Optional[SampleStream] = None):
    method = str(verify_method or "exact").strip().lower()
    if method not in ("exact", "lossy"):
        raise ValueError(f"Unsupported verify_method: {verify_method!r} (supported: 'exact', 'lossy')")
    out = verify_tree_device(tree=tree, root_ind=root_ind, logits=logits, eos_token_id=eos_token_id,
                             skip_nodes=skip_nodes, verify_method=method, verify_kwargs=verify_kwargs,
                             logits_processor=logits_processor, do_sample=bool(do_sample), stream=stream)
    # one small device-to-host copy: the host needs the tokens before the stop criteria run
    counts = out["counts"][0].cpu()
    emitted, accept, total, status = (int(v) for v in counts)
    if status & 1:
        raise IndexError("verify_tree: the walk reached a node whose logits row was not scored")
    if status & 2:
        raise ValueError("verify_tree: tree nodes must be ordered so that parents precede children")
    host = torch.stack([out["tokens"][0, :emitted], out["contexts"][0, :emitted]]).cpu()
    if method == "lossy":
        vk = dict(verify_kwargs or {})
        record_lossy_diagnostics(
            tree=tree, skip_nodes=int(skip_nodes), target=out["target"][0].cpu(), entropy=out["entropy"][0].cpu(),
            child_prob=out["child_prob"][0].cpu(), tokens=host[0], contexts=host[1], accept_len=accept,
            eos_token_id=eos_token_id, threshold=float(vk.get("threshold", 0.0)),
            window_size=int(vk.get("window_size", 1)),
            threshold_method=str(vk.get("threshold_method", "prob") or "prob").strip().lower())
    return host[0].unsqueeze(0), host[1], (total, accept)
