"""Host-side diagnostics of the lossy verifier, computed from the small per-node arrays the
device returns (argmax token, normalized entropy, p[parent, token]) instead of the full
probability matrix.  Produces the ``wandb_logger`` keys of
specdecodes/models/utils/lossy_tree_verify.py:170-337 (window-eligible gate statistics, lossy accept
counts and rates) with the same running mean / std accumulators."""
from __future__ import annotations

from typing import List, Optional

from .wandb_logger import wandb_logger


def _push(key: str, x: float) -> None:
    st = wandb_logger.internal_data.get(key) or {"n": 0, "mean": 0.0, "M2": 0.0}
    n = int(st["n"]) + 1
    delta = x - float(st["mean"])
    mean = float(st["mean"]) + delta / n
    wandb_logger.internal_data[key] = {"n": n, "mean": mean, "M2": float(st["M2"]) + delta * (x - mean)}


def _mean_std(key: str):
    st = wandb_logger.internal_data.get(key)
    if not st or int(st.get("n", 0)) <= 0:
        return 0.0, 0.0
    return float(st["mean"]), float(max(float(st["M2"]) / int(st["n"]), 0.0) ** 0.5)


def record_lossy_diagnostics(*, tree, skip_nodes: int, target, entropy, child_prob, tokens, contexts,
                             accept_len: int, eos_token_id: Optional[int], threshold: float, window_size: int,
                             threshold_method: str) -> None:
    use_entropy = threshold_method == "entropy"
    need = max(0, int(window_size))
    tgt: List[int] = [int(v) for v in target.tolist()]
    ent: List[float] = entropy.tolist()
    cp: List[float] = child_prob.tolist()
    d = tree.get_tree_data(skip_nodes=skip_nodes)
    n = min(len(tgt), int(d["token_ids"].numel()))
    tok = d["token_ids"].tolist()[:n]
    par = [int(p) - skip_nodes for p in d["parent_indices"].tolist()[:n]]
    kids: List[List[int]] = [[] for _ in range(n)]
    for i, p in enumerate(par):
        if 0 <= p < n and p != i:
            kids[p].append(i)
    exact_after = [0] * n
    for u in range(n - 1, -1, -1):
        hits = [exact_after[c] for c in kids[u] if tok[c] == tgt[u]]
        if hits:
            exact_after[u] = 1 + max(hits)
    mismatch = [bool(kids[u]) and all(tok[c] != tgt[u] for c in kids[u]) for u in range(n)]

    def gate_value(u: int) -> Optional[float]:
        ok = [c for c in kids[u] if exact_after[c] >= need]
        if not ok:
            return None
        return float(ent[u]) if use_entropy else max(float(cp[c]) for c in ok)

    blocks = (lambda v: v >= threshold) if use_entropy else (lambda v: v < threshold)
    toks = [int(t) for t in tokens.tolist()]
    ctxs = [int(c) - skip_nodes for c in contexts.tolist()]
    mm_ctx = mm_elig = mm_drop = mm_acc = mm_acc_nomatch = 0
    for step, ctx in enumerate(ctxs):
        if not 0 <= ctx < n:
            continue
        if mismatch[ctx]:
            mm_ctx += 1
            g = gate_value(ctx)
            if g is not None:
                mm_elig += 1
                _push("lossy/window_ok_gate", g)
                if blocks(g):
                    mm_drop += 1
                    _push("lossy/window_ok_drop_gate", g)
        if step < accept_len and toks[step] != tgt[ctx]:
            mm_acc += 1
            if step + 1 < len(ctxs):
                nxt = ctxs[step + 1]
            else:                       # path ended on EOS: no following context, find the child by token
                nxt = next(c for c in kids[ctx] if tok[c] == toks[step])
            p = float(cp[nxt])
            _push("verify/mm_acc_p", p)
            _push("lossy/accept_gate", float(ent[ctx]) if use_entropy else p)
            if mismatch[ctx]:
                mm_acc_nomatch += 1

    store = wandb_logger.internal_data
    for key, val in (("lossy/accept_tokens", accept_len), ("lossy/mm_ctx", mm_ctx), ("lossy/mm_elig_ctx", mm_elig),
                     ("lossy/mm_drop_ctx", mm_drop), ("lossy/mm_acc_steps", mm_acc),
                     ("lossy/mm_acc_nomatch_steps", mm_acc_nomatch)):
        store[key] = float(store.get(key, 0.0)) + float(val)
    log = wandb_logger.log_data
    acc = store["lossy/accept_tokens"]
    log["verify_accept_tokens"] = acc
    log["verify_lossy_accept_tokens"] = store["lossy/mm_acc_steps"]
    log["verify_lossy_accept_rate"] = store["lossy/mm_acc_steps"] / acc if acc > 0 else 0.0
    log["lossy_window_ok_drop_rate"] = store["lossy/mm_drop_ctx"] / store["lossy/mm_elig_ctx"] if store["lossy/mm_elig_ctx"] > 0 else 0.0
    log["lossy_accept_rate_when_no_match"] = store["lossy/mm_acc_nomatch_steps"] / store["lossy/mm_ctx"] if store["lossy/mm_ctx"] > 0 else 0.0
    for name, key in (("lossy_window_ok_gate", "lossy/window_ok_gate"), ("lossy_window_ok_drop_gate", "lossy/window_ok_drop_gate"),
                      ("lossy_accepted_prob", "verify/mm_acc_p"), ("lossy_accepted_gate", "lossy/accept_gate")):
        log[name + "_mean"], log[name + "_std"] = _mean_std(key)
    log["lossy_threshold_method"] = "entropy" if use_entropy else "prob"
