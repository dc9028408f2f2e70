"""Oracle: tree verification (greedy exact walk and lossy bottom-up DP).  Test infrastructure only.

Follows (reference paths):
  * target probabilities   specdecodes/models/generators/base.py:135-137  (softmax in logits dtype)
  * exact walk             specdecodes/models/utils/tree_verify.py:49-106 and
                           specdecodes/models/generators/classic_sd.py:111-116 (_verify_step)
  * lossy prelude          specdecodes/models/utils/tree_verify.py:111-163
  * lossy DP + extraction  specdecodes/models/utils/lossy_tree_verify.py:9-343

All functions take CPU tensors / python lists and are written for clarity, not speed.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence, Tuple

import torch


def children_from_parents(parents: Sequence[int]) -> List[List[int]]:
    """Children lists in ascending index order from a parent array (root parent = -1)."""
    kids: List[List[int]] = [[] for _ in parents]
    for i, p in enumerate(parents):
        if p is not None and 0 <= int(p) < len(parents) and int(p) != i:
            kids[int(p)].append(i)
    return kids


def target_probs(logits: torch.Tensor) -> torch.Tensor:
    """softmax over the vocabulary in the logits' own dtype (generators/base.py:135-137)."""
    return torch.softmax(logits.cpu(), dim=-1)


def normalized_entropy(probs: torch.Tensor) -> List[float]:
    """sum(entr(p)) / ln V per row, evaluated in the dtype of ``probs``
    (lossy_tree_verify.py:66-72).  Returned as python floats, as ``.tolist()`` does."""
    vocab = int(probs.shape[1])
    denom = math.log(vocab) if vocab > 1 else 1.0
    return (torch.special.entr(probs).sum(dim=-1) / denom).tolist()


def exact_verify(
    probs: torch.Tensor,
    token_ids: Sequence[int],
    children: Sequence[Sequence[int]],
    root: int = 0,
    eos_token_id: Optional[int] = None,
    skip_nodes: int = 0,
    target_tokens: Optional[Sequence[int]] = None,
) -> Tuple[List[int], List[int], Tuple[int, int]]:
    """Walk from the root (tree_verify.py:49-106).  The target token of a context is the argmax of
    its row, or, for a sampling target, ``target_tokens[row]``: the reference draws
    ``p.multinomial(1)`` once per visited context (classic_sd.py:112; the bonus draw of :99-100 is
    taken only for a context that has not been drawn yet), so one pre-drawn token per row
    restates it.

    ``token_ids``/``children`` use ORIGINAL node indexing for the whole tree;
    ``probs[r]`` is the distribution at original node ``r + skip_nodes``.
    Returns (sampled_tokens, hidden_indices (original indexing), (total_len, accept_len)).
    """
    rows = int(probs.shape[0])
    target = (lambda r: int(probs[r].argmax())) if target_tokens is None else (lambda r: int(target_tokens[r]))
    cur = int(root)
    out_tok: List[int] = []
    out_ctx: List[int] = []
    total = accept = 0
    bonus: Optional[int] = None
    kids = list(children[cur])
    while kids:
        total += 1
        t = target(cur - skip_nodes)                        # classic_sd.py:112
        match = [c for c in kids if int(token_ids[c]) == t]
        if not match:                                       # classic_sd.py:115-116
            bonus = t
            break
        bonus = None
        accept += 1
        out_tok.append(t)
        out_ctx.append(cur)
        if eos_token_id is not None and t == int(eos_token_id):   # tree_verify.py:82-83
            break
        cur = match[0]                                      # siblings carry distinct tokens
        kids = list(children[cur])
        if not kids:                                        # tree_verify.py:89-90
            break
        if min(kids) - skip_nodes >= rows:                  # tree_verify.py:91-92
            break
    if (not out_tok) or eos_token_id is None or out_tok[-1] != int(eos_token_id):  # :97
        if bonus is None:
            bonus = target(cur - skip_nodes)
        out_tok.append(bonus)
        out_ctx.append(cur)
    return out_tok, out_ctx, (total, accept)


def _welford_push(store: Dict[str, dict], key: str, x: float) -> None:
    st = store.get(key) or {"n": 0, "mean": 0.0, "M2": 0.0}
    n = st["n"] + 1
    d = x - st["mean"]
    mean = st["mean"] + d / n
    store[key] = {"n": n, "mean": mean, "M2": st["M2"] + d * (x - mean)}


def _welford_read(store: Dict[str, dict], key: str) -> Tuple[float, float]:
    st = store.get(key)
    if not st or st["n"] <= 0:
        return 0.0, 0.0
    return float(st["mean"]), float(max(st["M2"] / st["n"], 0.0) ** 0.5)


def lossy_verify(
    probs: torch.Tensor,
    token_ids: Sequence[int],
    children: Sequence[Sequence[int]],
    root: int = 0,
    eos_token_id: Optional[int] = None,
    threshold: float = 0.0,
    window_size: int = 1,
    threshold_method: str = "prob",
    internal: Optional[dict] = None,
    log: Optional[dict] = None,
    target_tokens: Optional[Sequence[int]] = None,
) -> Tuple[List[int], List[int], int]:
    """Bottom-up DP verifier in LOCAL indexing (lossy_tree_verify.py:9-343).  ``target_tokens`` (one per
    row) stands for the ``torch.multinomial`` draw of a sampling target (:75-77); None = argmax.

    ``internal``/``log`` play the role of ``wandb_logger.internal_data`` / ``.log_data``
    (running accumulators and exported metrics); pass the same dicts across calls to accumulate.
    """
    method = str(threshold_method or "entropy").strip().lower()
    if method not in ("entropy", "prob"):
        raise ValueError(f"Unsupported threshold_method: {threshold_method!r}")
    use_entropy = method == "entropy"
    theta = float(threshold)
    need = max(0, int(window_size))
    n = int(probs.shape[0])
    tok = [int(t) for t in token_ids]
    tgt = probs.argmax(dim=-1).tolist() if target_tokens is None else [int(t) for t in target_tokens]   # :75-77
    h = normalized_entropy(probs) if use_entropy else None               # :103-105

    mismatch = [bool(children[u]) and all(tok[c] != tgt[u] for c in children[u]) for u in range(n)]

    best_len = [0] * n
    best_next = [-1] * n
    exact_after = [0] * n
    for u in range(n - 1, -1, -1):                                       # :112
        kids = children[u]
        if not kids:
            continue
        hits = [exact_after[c] for c in kids if tok[c] == tgt[u]]
        if hits:
            exact_after[u] = 1 + max(hits)                               # :118-120
        pick, pick_len, pick_exact, pick_p = -1, 0, False, -1.0
        for c in kids:
            is_exact = tok[c] == tgt[u]
            if is_exact:
                p = -1.0
            else:
                if exact_after[c] < need:                                # :139-140
                    continue
                if use_entropy and h[u] >= theta:                        # :141-142
                    continue
                p = float(probs[u, tok[c]])
                if (not use_entropy) and p < theta:                      # :144-145
                    continue
            length = 1 + best_len[c]
            if length > pick_len:
                pick, pick_len, pick_exact, pick_p = c, length, is_exact, p
            elif length == pick_len:
                if is_exact and not pick_exact:
                    pick, pick_exact, pick_p = c, True, p
                elif (not is_exact) and (not pick_exact) and p > pick_p:
                    pick, pick_p = c, p
        if pick >= 0 and pick_len > 0:
            best_next[u], best_len[u] = pick, pick_len

    # gate value a window-eligible mismatch context would have to pass (:170-195)
    gate_val: List[Optional[float]] = [None] * n
    for u in range(n):
        if not children[u] or not mismatch[u]:
            continue
        if use_entropy:
            if any(exact_after[c] >= need for c in children[u]):
                gate_val[u] = float(h[u])
        else:
            ps = [float(probs[u, tok[c]]) for c in children[u] if exact_after[c] >= need]
            gate_val[u] = max(ps) if ps else None

    internal = internal if internal is not None else {}
    log = log if log is not None else {}
    blocks = (lambda v: v >= theta) if use_entropy else (lambda v: v < theta)

    out_tok: List[int] = []
    out_ctx: List[int] = []
    ctx = int(root)
    mm_ctx = mm_elig = mm_drop = mm_acc = mm_acc_nomatch = 0
    while True:                                                           # :247-286
        if mismatch[ctx]:
            mm_ctx += 1
            g = gate_val[ctx]
            if g is not None:
                mm_elig += 1
                _welford_push(internal, "lossy/window_ok_gate", g)
                if blocks(g):
                    mm_drop += 1
                    _welford_push(internal, "lossy/window_ok_drop_gate", g)
        nxt = best_next[ctx]
        if nxt < 0:
            break
        t = tok[nxt]
        out_tok.append(t)
        out_ctx.append(ctx)
        if t != tgt[ctx]:
            mm_acc += 1
            p = float(probs[ctx, t])
            _welford_push(internal, "verify/mm_acc_p", p)
            _welford_push(internal, "lossy/accept_gate", float(h[ctx]) if use_entropy else p)
            if mismatch[ctx]:
                mm_acc_nomatch += 1
        if eos_token_id is not None and t == int(eos_token_id):
            break
        ctx = nxt
    accept_len = len(out_tok)
    if (not out_tok) or eos_token_id is None or out_tok[-1] != int(eos_token_id):   # :289-291
        out_tok.append(int(tgt[ctx]))
        out_ctx.append(ctx)

    for key, val in (("lossy/accept_tokens", accept_len), ("lossy/mm_ctx", mm_ctx),
                     ("lossy/mm_elig_ctx", mm_elig), ("lossy/mm_drop_ctx", mm_drop),
                     ("lossy/mm_acc_steps", mm_acc), ("lossy/mm_acc_nomatch_steps", mm_acc_nomatch)):
        internal[key] = float(internal.get(key, 0.0)) + float(val)
    acc = internal["lossy/accept_tokens"]
    log["verify_accept_tokens"] = acc
    log["verify_lossy_accept_tokens"] = internal["lossy/mm_acc_steps"]
    log["verify_lossy_accept_rate"] = internal["lossy/mm_acc_steps"] / acc if acc > 0 else 0.0
    e = internal["lossy/mm_elig_ctx"]
    log["lossy_window_ok_drop_rate"] = internal["lossy/mm_drop_ctx"] / e if e > 0 else 0.0
    m = internal["lossy/mm_ctx"]
    log["lossy_accept_rate_when_no_match"] = internal["lossy/mm_acc_nomatch_steps"] / m if m > 0 else 0.0
    for name, key in (("lossy_window_ok_gate", "lossy/window_ok_gate"),
                      ("lossy_window_ok_drop_gate", "lossy/window_ok_drop_gate"),
                      ("lossy_accepted_prob", "verify/mm_acc_p"),
                      ("lossy_accepted_gate", "lossy/accept_gate")):
        log[name + "_mean"], log[name + "_std"] = _welford_read(internal, key)
    log["lossy_threshold_method"] = "entropy" if use_entropy else "prob"
    return out_tok, out_ctx, accept_len


def verify_logits(
    logits: torch.Tensor,
    token_ids: Sequence[int],
    parents: Sequence[int],
    root: int = 0,
    eos_token_id: Optional[int] = None,
    skip_nodes: int = 0,
    verify_method: str = "exact",
    verify_kwargs: Optional[dict] = None,
    internal: Optional[dict] = None,
    log: Optional[dict] = None,
    temperature: Optional[float] = None,
    target_tokens: Optional[Sequence[int]] = None,
):
    """``verify_tree`` restated on plain arrays (tree_verify.py:8-163).  Greedy target by default; for a
    sampling target pass the warper's ``temperature`` and one pre-drawn token per row
    (``oracle.sampling.draw_tokens`` on ``oracle.sampling.warp_probs``).

    ``token_ids``/``parents`` describe the WHOLE tree in original indexing, ``logits`` is
    ``[rows, V]`` for original nodes ``skip_nodes .. skip_nodes+rows-1``.
    Returns (sampled_tokens, hidden_indices(original), (total_len, accept_len)).
    """
    method = str(verify_method or "exact").strip().lower()
    vk = dict(verify_kwargs or {})
    if temperature is not None and float(temperature) != 1.0:
        logits = logits.cpu() / float(temperature)                        # generators/base.py:57-58
    probs = target_probs(logits)
    kids_all = children_from_parents(parents)
    if method == "exact":
        return exact_verify(probs, token_ids, kids_all, root, eos_token_id, skip_nodes, target_tokens)
    if method != "lossy":
        raise ValueError(f"Unsupported verify_method: {verify_method!r} (supported: 'exact', 'lossy')")
    rows = int(probs.shape[0])
    tok_local = list(token_ids[skip_nodes:])[:rows]                       # tree_verify.py:122-123
    n_local = len(tok_local)
    root_local = int(root) - int(skip_nodes)
    if root_local < 0 or root_local >= n_local:                           # :133-135
        root_local = 0
    kids_local: List[List[int]] = [[] for _ in range(n_local)]
    for v in range(skip_nodes, skip_nodes + n_local):                     # :137-145
        for c in kids_all[v]:
            cl = c - skip_nodes
            if 0 <= cl < n_local:
                kids_local[v - skip_nodes].append(cl)
    toks, ctx_local, acc = lossy_verify(
        probs, tok_local, kids_local, root_local, eos_token_id,
        threshold=float(vk.get("threshold", 0.0)),
        window_size=int(vk.get("window_size", 1)),
        threshold_method=str(vk.get("threshold_method", "prob") or "prob").strip().lower(),
        internal=internal, log=log, target_tokens=target_tokens,
    )
    return toks, [c + skip_nodes for c in ctx_local], (len(toks), acc)


def brute_force_lossy_len(probs, token_ids, children, root, threshold, window_size, threshold_method,
                          target_tokens=None):
    """Independent check: longest admissible root path by exhaustive recursion (tiny trees only).

    Admissibility of an edge u->c (lossy_tree_verify.py:135-146): exact if tok[c]==argmax p[u];
    otherwise needs ``exact_chain(c) >= window`` and the gate.  ``exact_chain(c)`` is the longest
    run of exact edges below c.
    """
    tok = [int(t) for t in token_ids]
    tgt = probs.argmax(dim=-1).tolist() if target_tokens is None else [int(t) for t in target_tokens]
    h = normalized_entropy(probs)
    use_entropy = threshold_method == "entropy"

    def exact_chain(u):
        best = 0
        for c in children[u]:
            if tok[c] == tgt[u]:
                best = max(best, 1 + exact_chain(c))
        return best

    def admissible(u, c):
        if tok[c] == tgt[u]:
            return True
        if exact_chain(c) < max(0, window_size):
            return False
        if use_entropy:
            return not (h[u] >= threshold)
        return not (float(probs[u, tok[c]]) < threshold)

    def longest(u):
        best = 0
        for c in children[u]:
            if admissible(u, c):
                best = max(best, 1 + longest(c))
        return best

    return longest(root)
