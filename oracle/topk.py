"""Oracle: top-k draft-tree expansion.  Test infrastructure only.

Follows DraftModelBase._topk_flatten (specdecodes/models/draft_models/base.py:281-305):
``buf = sampled_probs * parent_probs[..., None]`` (rounded to the tensor dtype),
``topk(buf.view(B, L*V), min(k, V), sorted=True)``, ``token = idx % V``, ``parent = idx // V``.

``torch.topk`` does not define the order of equal values, so the canonical answer is defined by a
stable descending sort (value descending, flat index ascending); ``topk_expand_torch`` is the
reference's literal call sequence, used to check that the canonical values equal ``torch.topk``'s
bit for bit and that any index difference stays inside a group of equal values (the tie-tolerant
rule of the reference's analysis/bench_topk_sampling.py:146-163).
"""
import torch


def topk_expand(sampled_probs: torch.Tensor, parent_probs: torch.Tensor, k: int):
    B, L, V = sampled_probs.shape
    k = min(int(k), int(V))
    buf = torch.mul(sampled_probs, parent_probs.unsqueeze(-1)).view(B, -1)
    order = torch.sort(buf.float(), dim=1, descending=True, stable=True).indices[:, :k]
    vals = torch.gather(buf, 1, order)
    return (order % V).long(), vals, (order // V).long()


def topk_expand_torch(sampled_probs: torch.Tensor, parent_probs: torch.Tensor, k: int):
    B, L, V = sampled_probs.shape
    k = min(int(k), int(V))
    buf = torch.mul(sampled_probs, parent_probs.unsqueeze(-1)).view(B, -1)
    vals, idx = torch.topk(buf, k, dim=1, sorted=True)
    return (idx % V).long(), vals, (idx // V).long()


def topk_brute_force(sampled_probs: torch.Tensor, parent_probs: torch.Tensor, k: int):
    """Python-loop selection for tiny inputs: repeatedly take the best remaining (value, -index)."""
    B, L, V = sampled_probs.shape
    k = min(int(k), int(V))
    buf = torch.mul(sampled_probs, parent_probs.unsqueeze(-1)).view(B, -1)
    out = []
    for b in range(B):
        items = [(float(v), -i) for i, v in enumerate(buf[b])]
        items.sort(reverse=True)
        out.append([(-i) for _, i in items[:k]])
    idx = torch.tensor(out)
    return (idx % V).long(), torch.gather(buf, 1, idx), (idx // V).long()


def draft_probs(logits: torch.Tensor, temperature: float) -> torch.Tensor:
    """The draft's probability rows: ``torch.softmax(logits / temperature, dim=-1)`` in the logits dtype
    (specdecodes/models/draft_models/classic_sd.py:10-16).  Pinned by the library routine itself; the
    quotient is a tensor op and therefore rounded to the dtype before the softmax."""
    return torch.softmax(logits / temperature, dim=-1)
