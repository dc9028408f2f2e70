"""Writes tests/golden/reference_vectors.json by running the reference's pure-torch tree/verify code.

Run in the BUILD container only (needs /root/reference, which never travels):

    python tests/golden/make_reference_vectors.py

Covers what the reference's own tests leave open: the lossy verifier with the *entropy* gate on
random trees (tie order among equal-length children, EOS, window sizes), ``verify_tree`` with
``skip_nodes`` > 0 in both modes, and the ``Tree`` re-indexing helpers (``prune_to_depth``,
``prune_to_top_n``, ``create_attention_mask``, ``get_tree_data``).  Inputs are small (V <= 40) and
stored explicitly, so the fixture is data only.
"""
import json
import os
import sys

import torch

REF = os.environ.get("SUBSPEC_REFERENCE", "/root/reference")
sys.path.insert(0, REF)

from specdecodes.models.utils.cpu_tree import Tree  # noqa: E402
from specdecodes.models.utils.lossy_tree_verify import lossy_bottom_up_verify  # noqa: E402
from specdecodes.models.utils.tree_verify import verify_tree  # noqa: E402
from specdecodes.models.utils.wandb_logger import wandb_logger  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.json")


def greedy_probs(logits, logits_processor, do_sample, return_probs=False):
    # greedy branch of the generator's sampler: softmax in the logits' dtype
    return torch.softmax(logits, dim=-1) if return_probs else torch.argmax(logits, dim=-1)


def greedy_step(p, token_ids, logits_processor, do_sample):
    t = p.argmax()
    return (t, None) if torch.any(t == token_ids) else (None, t)


def random_level_tree(g, depth, k, vocab):
    """Level-order tree as the drafter builds it: k nodes per level, parents among the previous
    level's nodes, distinct tokens among siblings.  Returns per-level (tokens, probs, local parents)."""
    levels = []
    prev = 1
    for d in range(depth):
        parents = torch.randint(0, prev, (k,), generator=g).sort().values.tolist()
        toks = []
        for j, p in enumerate(parents):
            used = {toks[i] for i in range(j) if parents[i] == p}
            while True:
                t = int(torch.randint(0, vocab, (1,), generator=g))
                if t not in used:
                    break
            toks.append(t)
        probs = torch.rand(k, generator=g).sort(descending=True).values.tolist()
        levels.append((toks, probs, parents))
        prev = k
    return levels


def build_tree(levels, root_token, dtype=torch.float32):
    tree = Tree(torch.tensor(root_token), dtype)
    tok = torch.tensor([[lv[0] for lv in levels]])
    pr = torch.tensor([[lv[1] for lv in levels]], dtype=dtype)
    par = torch.tensor([[lv[2] for lv in levels]])
    tree.add_nodes(tok, pr, par)
    return tree


def plant_logits(g, tree, vocab, dtype, scale):
    """Random logits with planted structure so that exact chains, low-entropy mismatch contexts
    and ties all occur."""
    n = tree.size()
    logits = torch.randn(n, vocab, generator=g) * scale
    for u in range(n):
        kids = tree.nodes[u].children
        r = float(torch.rand(1, generator=g))
        if kids and r < 0.55:
            c = kids[int(torch.randint(0, len(kids), (1,), generator=g))]
            logits[u, tree.nodes[c].token_id] = logits[u].max() + 1.0 + 6.0 * float(torch.rand(1, generator=g))
        elif r < 0.8:
            t = int(torch.randint(0, vocab, (1,), generator=g))
            logits[u, t] = logits[u].max() + 4.0 + 8.0 * float(torch.rand(1, generator=g))
    return logits.to(dtype)


def tree_arrays(tree):
    d = tree.get_tree_data()
    return d["token_ids"].tolist(), d["parent_indices"].tolist()


def main():
    g = torch.Generator().manual_seed(20240607)
    doc = {"lossy": [], "verify_tree": [], "tree": []}

    # --- lossy_bottom_up_verify, both gates, random trees --------------------------------
    for case in range(40):
        depth = int(torch.randint(2, 8, (1,), generator=g))
        k = int(torch.randint(1, 5, (1,), generator=g))
        vocab = int(torch.randint(12, 41, (1,), generator=g))
        dtype = [torch.float32, torch.bfloat16, torch.float16][case % 3]
        tree = build_tree(random_level_tree(g, depth, k, vocab), root_token=1)
        logits = plant_logits(g, tree, vocab, dtype, scale=[0.5, 1.0, 3.0][case % 3])
        probs = torch.softmax(logits, dim=-1)
        toks, parents = tree_arrays(tree)
        kids = [list(nd.children) for nd in tree.nodes]
        method = "entropy" if case % 4 != 3 else "prob"
        theta = [0.3, 0.6, 0.9, 0.15][case % 4] if method == "entropy" else [0.05, 0.2][case % 2]
        window = [0, 1, 2, 6][(case // 2) % 4]
        eos = None if case % 5 else toks[min(len(toks) - 1, 3)]
        wandb_logger.clear_log_data()
        s, hidx, acc = lossy_bottom_up_verify(
            probs=probs, token_ids=torch.tensor(toks), parent_indices=torch.tensor(parents),
            children_lists=kids, root_index=0, eos_token_id=eos, do_sample=False,
            threshold=theta, window_size=window, threshold_method=method)
        doc["lossy"].append(dict(
            dtype=str(dtype).split(".")[-1], logits=logits.float().tolist(), token_ids=toks, parents=parents,
            eos_token_id=eos, threshold=theta, window_size=window, threshold_method=method,
            sampled=s.tolist(), hidden=hidx.tolist(), accept_len=int(acc),
            log={k_: v for k_, v in wandb_logger.log_data.items()}))

    # --- verify_tree incl. skip_nodes (v2 post-verify indexing) ----------------------------
    for case in range(24):
        depth = int(torch.randint(3, 8, (1,), generator=g))
        k = int(torch.randint(2, 5, (1,), generator=g))
        vocab = int(torch.randint(16, 41, (1,), generator=g))
        dtype = [torch.float32, torch.bfloat16][case % 2]
        tree = build_tree(random_level_tree(g, depth, k, vocab), root_token=2)
        n = tree.size()
        full = plant_logits(g, tree, vocab, dtype, scale=1.5)
        toks, parents = tree_arrays(tree)
        if case % 3 == 0:
            skip, root = 0, 0
        else:
            # v2: the first `skip` nodes were scored earlier; root is an already-accepted node
            skip = 1 + k * int(torch.randint(1, max(2, depth - 1), (1,), generator=g))
            skip = min(skip, n - k)
            cands = [i for i in range(skip) if any(c >= skip for c in tree.nodes[i].children)]
            root = cands[int(torch.randint(0, len(cands), (1,), generator=g))] if cands else 0
        logits = full[skip:].unsqueeze(0)
        method = ["exact", "lossy"][(case // 2) % 2]
        vk = dict(threshold=[0.3, 0.7][case % 2], window_size=[1, 2, 0][case % 3],
                  threshold_method=["entropy", "prob"][(case // 4) % 2])
        eos = None if case % 4 else toks[min(n - 1, skip + 1)]
        wandb_logger.clear_log_data()
        try:
            s, hidx, (total, acc) = verify_tree(
                tree=tree, root_ind=root, logits=logits, sample_token_fn=greedy_probs,
                verify_step_fn=greedy_step, eos_token_id=eos, logits_processor=None, do_sample=False,
                skip_nodes=skip, verify_method=method, verify_kwargs=vk)
        except (IndexError, RuntimeError):
            # exact walk from a root whose row was not scored in this call: outside the contract
            continue
        doc["verify_tree"].append(dict(
            dtype=str(dtype).split(".")[-1], logits=logits[0].float().tolist(), token_ids=toks, parents=parents,
            root=root, skip_nodes=skip, eos_token_id=eos, verify_method=method, verify_kwargs=vk,
            sampled=s[0].tolist(), hidden=hidx.tolist(), total_len=int(total), accept_len=int(acc)))

    # --- Tree helpers -------------------------------------------------------------------------
    for case in range(12):
        depth = int(torch.randint(2, 7, (1,), generator=g))
        k = int(torch.randint(1, 6, (1,), generator=g))
        levels = random_level_tree(g, depth, k, 50)
        rec = dict(levels=[dict(tokens=a, probs=b, parents=c) for a, b, c in levels], root_token=7)
        tree = build_tree(levels, 7)
        d = tree.get_tree_data()
        rec["tree_data"] = {k_: v.tolist() for k_, v in d.items()}
        rec["children"] = [list(nd.children) for nd in tree.nodes]
        rec["mask_prefix3"] = tree.create_attention_mask(3)[0, 0].int().tolist()
        sk = min(2, tree.size() - 1)
        rec["mask_prefix2_skip"] = dict(skip=sk, mask=tree.create_attention_mask(2, sk)[0, 0].int().tolist())
        rec["depth"] = int(tree.get_depth())
        rec["find_child"] = [[u, t, tree.find_child_index(u, t)] for u in range(tree.size())
                             for t in ([tree.nodes[c].token_id for c in tree.nodes[u].children][:1] + [49])]
        md = int(torch.randint(0, depth + 1, (1,), generator=g))
        t2 = build_tree(levels, 7)
        keep = t2.prune_to_depth(md)
        rec["prune_to_depth"] = dict(max_depth=md, keep=keep.tolist(),
                                     tree_data={k_: v.tolist() for k_, v in t2.get_tree_data().items()},
                                     children=[list(nd.children) for nd in t2.nodes],
                                     available_leaves=list(t2.available_leaves))
        # distinct cumulative probabilities that decrease down the tree, so top-n keeps parents
        t3 = build_tree(levels, 7)
        for i, nd in enumerate(t3.nodes):
            nd.cumulative_probability = 1.0 / (1.0 + i)
        topn = max(1, t3.size() // 2)
        keep3 = t3.prune_to_top_n(topn)
        rec["prune_to_top_n"] = dict(n=topn, keep=keep3.tolist(),
                                     tree_data={k_: v.tolist() for k_, v in t3.get_tree_data().items()},
                                     children=[list(nd.children) for nd in t3.nodes],
                                     available_leaves=list(t3.available_leaves))
        doc["tree"].append(rec)

    with open(OUT, "w") as f:
        json.dump(doc, f)
    print("wrote", OUT, {k_: len(v) for k_, v in doc.items()}, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
