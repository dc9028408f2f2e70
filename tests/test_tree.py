"""Host tree (subspec_amd.cpu_tree.Tree) against reference-written golden vectors and a
brute-force ancestor closure.  No GPU."""
import json
import os

import pytest
import torch

from subspec_amd.cpu_tree import Tree

GOLD = os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")


def _cases():
    with open(GOLD) as f:
        return json.load(f)["tree"]


def _build(rec):
    t = Tree(torch.tensor(rec["root_token"]))
    lv = rec["levels"]
    t.add_nodes(torch.tensor([[l["tokens"] for l in lv]]),
                torch.tensor([[l["probs"] for l in lv]]),
                torch.tensor([[l["parents"] for l in lv]]))
    return t


def _data(t):
    return {k: v.tolist() for k, v in t.get_tree_data().items()}


@pytest.mark.parametrize("idx", range(12))
def test_tree_matches_reference(idx):
    rec = _cases()[idx]
    t = _build(rec)
    assert _data(t) == rec["tree_data"]
    assert [list(nd.children) for nd in t.nodes] == rec["children"]
    assert t.create_attention_mask(3)[0, 0].int().tolist() == rec["mask_prefix3"]
    ms = rec["mask_prefix2_skip"]
    assert t.create_attention_mask(2, ms["skip"])[0, 0].int().tolist() == ms["mask"]
    assert int(t.get_depth()) == rec["depth"]
    for u, tok, exp in rec["find_child"]:
        assert t.find_child_index(u, tok) == exp
    # parents precede children (level order)
    par = rec["tree_data"]["parent_indices"]
    assert all(p < i for i, p in enumerate(par))

    pd = rec["prune_to_depth"]
    t2 = _build(rec)
    assert t2.prune_to_depth(pd["max_depth"]).tolist() == pd["keep"]
    assert _data(t2) == pd["tree_data"]
    assert [list(nd.children) for nd in t2.nodes] == pd["children"]
    assert list(t2.available_leaves) == pd["available_leaves"]

    pn = rec["prune_to_top_n"]
    t3 = _build(rec)
    for i, nd in enumerate(t3.nodes):
        nd.cumulative_probability = 1.0 / (1.0 + i)
    assert t3.prune_to_top_n(pn["n"]).tolist() == pn["keep"]
    assert _data(t3) == pn["tree_data"]
    assert [list(nd.children) for nd in t3.nodes] == pn["children"]
    assert list(t3.available_leaves) == pn["available_leaves"]


def test_ancestor_bits_brute_force():
    rec = _cases()[3]
    t = _build(rec)
    par = rec["tree_data"]["parent_indices"]
    for i, b in enumerate(t.ancestor_bits()):
        anc, p = {i}, par[i]
        while p >= 0:
            anc.add(p)
            p = par[p]
        assert {j for j in range(t.size()) if (b >> j) & 1} == anc


def test_tree_errors():
    t = Tree(torch.tensor(1))
    with pytest.raises(ValueError):
        t.prune_to_depth(-1)
    with pytest.raises(IndexError):
        t.get_node(5)
    with pytest.raises(AssertionError):
        t.add_nodes(torch.zeros(2, 1, 1, dtype=torch.long), torch.zeros(2, 1, 1), torch.zeros(2, 1, 1, dtype=torch.long))
