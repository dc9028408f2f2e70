"""Synthetic inputs of the benchmark configurations (seeded, shapes of Qwen2.5-7B).

Used by the tests, the smoke run and bench.py so that all three exercise identical data.
Nothing here computes an expected answer; that is the oracle's job.
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch

QWEN_VOCAB = 152064


def random_tree(gen: torch.Generator, n: int = 64, max_depth: int = 8, max_children: int = 4,
                vocab: int = QWEN_VOCAB, chain_depth: int = 0) -> Tuple[List[int], List[int], List[int]]:
    """Random tree in level order (parent < child, depth non-decreasing with the index).

    Returns (parents, token_ids, depths); siblings carry distinct tokens.  ``chain_depth`` > 0
    first lays down one root path of that many edges so that deep acceptances are possible.
    """
    parents, depths, kids = [-1], [0], [0]
    tip = 0
    for _ in range(min(chain_depth, n - 1)):
        parents.append(tip)
        depths.append(depths[tip] + 1)
        kids[tip] += 1
        kids.append(0)
        tip = len(parents) - 1
    while len(parents) < n:
        open_nodes = [i for i in range(len(parents)) if depths[i] < max_depth and kids[i] < max_children]
        p = open_nodes[int(torch.randint(0, len(open_nodes), (1,), generator=gen))]
        parents.append(p)
        depths.append(depths[p] + 1)
        kids[p] += 1
        kids.append(0)
    order = sorted(range(n), key=lambda i: (depths[i], i))       # level order, stable
    new_of = {old: new for new, old in enumerate(order)}
    parents = [(-1 if parents[o] < 0 else new_of[parents[o]]) for o in order]
    depths = [depths[o] for o in order]
    tokens: List[int] = []
    for i in range(n):
        used = {tokens[j] for j in range(i) if parents[j] == parents[i]}
        while True:
            t = int(torch.randint(0, vocab, (1,), generator=gen))
            if t not in used:
                break
        tokens.append(t)
    return parents, tokens, depths


def children_of(parents: List[int]) -> List[List[int]]:
    kids: List[List[int]] = [[] for _ in parents]
    for i, p in enumerate(parents):
        if p >= 0:
            kids[p].append(i)
    return kids


def deepest_path(parents: List[int], depths: List[int], gen: Optional[torch.Generator] = None) -> List[int]:
    """Node indices root..leaf of one maximal-depth path (random among them when ``gen`` is given)."""
    dmax = max(depths)
    leaves = [i for i, d in enumerate(depths) if d == dmax]
    leaf = leaves[int(torch.randint(0, len(leaves), (1,), generator=gen))] if gen is not None else leaves[0]
    path = [leaf]
    while parents[path[-1]] >= 0:
        path.append(parents[path[-1]])
    return path[::-1]


def plant_exact(logits: torch.Tensor, ctx: int, token: int, delta: float = 1.0) -> None:
    """Make ``token`` the argmax of row ``ctx``."""
    logits[ctx, token] = logits[ctx].float().max() + delta


def greedy_config(seed: int = 0, n: int = 64, vocab: int = QWEN_VOCAB, device="cpu", path_len: int = 5):
    """Config 1: fp32 logits [n, V] ~ N(0, sigma=2) with the target argmax planted along the first
    ``path_len`` edges of a random root-to-leaf path; the next context's argmax is not a child."""
    gen = torch.Generator().manual_seed(seed)
    parents, tokens, depths = random_tree(gen, n, vocab=vocab, chain_depth=path_len + 1)
    dgen = torch.Generator(device=device).manual_seed(seed)
    logits = torch.randn(n, vocab, generator=dgen, device=device, dtype=torch.float32) * 2.0
    path = deepest_path(parents, depths, gen)
    kids = children_of(parents)
    for u, c in list(zip(path, path[1:]))[:path_len]:
        plant_exact(logits, u, tokens[c])
    stop = path[min(path_len, len(path) - 1)]
    if kids[stop]:
        banned = {tokens[c] for c in kids[stop]}
        t = next(t for t in range(vocab) if t not in banned)
        plant_exact(logits, stop, t)
    return dict(logits=logits, parents=parents, tokens=tokens, depths=depths, path=path[: path_len + 1])


def lossy_config(seed: int = 0, batch: int = 32, n: int = 64, vocab: int = QWEN_VOCAB, device="cpu",
                 dtype=torch.bfloat16, window: int = 6):
    """Config 2: ``batch`` independent 64-node trees (depth <= 8) with logits [batch, n, V] drawn
    N(0,1) and scaled per row by U[0.5, 3].  Pure Gaussian rows have normalized entropy >= 0.55, so
    the 0.3 gate would never open; each tree therefore gets a planted depth-8 path in one of five
    flavours (all exact / low-entropy mismatch at edge 0 or 1 / high-entropy mismatch / nothing
    planted), which exercises exact chains, lossy accepts and gate rejections."""
    gen = torch.Generator().manual_seed(1000 + seed)
    dgen = torch.Generator(device=device).manual_seed(1000 + seed)
    logits = torch.randn(batch, n, vocab, generator=dgen, device=device, dtype=torch.float32)
    scale = torch.rand(batch, n, 1, generator=dgen, device=device) * 2.5 + 0.5
    logits = (logits * scale).to(dtype)
    all_parents, all_tokens, flavours = [], [], []
    for b in range(batch):
        parents, tokens, depths = random_tree(gen, n, vocab=vocab, chain_depth=8)
        path = deepest_path(parents, depths, gen)
        kids = children_of(parents)
        flavour = b % 5
        edges = list(zip(path, path[1:]))
        for e, (u, c) in enumerate(edges):
            lossy_edge = (flavour in (1, 3) and e == 0) or (flavour == 2 and e == 1)
            if flavour == 4:
                break
            if not lossy_edge:
                plant_exact(logits[b], u, tokens[c], delta=2.0)
                continue
            banned = {tokens[k] for k in kids[u]}
            t = next(t for t in range(7, vocab) if t not in banned)
            # +14 above the row maximum -> one dominant token, entropy far below 0.3;
            # +0.5 -> a mismatch whose entropy stays high, so the gate must block it
            plant_exact(logits[b], u, t, delta=14.0 if flavour in (1, 2) else 0.5)
        all_parents.append(parents)
        all_tokens.append(tokens)
        flavours.append(flavour)
    return dict(logits=logits, parents=all_parents, tokens=all_tokens, flavours=flavours,
                threshold=0.3, window_size=window, threshold_method="entropy")
