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


def test_dynamic_cache_bookkeeping_on_the_host():
    import torch
    from subspec_amd.cache import DynamicKVCache, create_kv_cache
    from subspec_amd.model import DecoderConfig
    cfg = DecoderConfig(num_hidden_layers=2, hidden_size=256, num_attention_heads=2, num_key_value_heads=1, head_dim=128,
                        intermediate_size=512, vocab_size=64)
    kv = create_kv_cache("dynamic", max_cache_len=None, config=cfg, device="cpu", dtype=torch.float32)
    c = kv.cache
    assert isinstance(c, DynamicKVCache) and c.max_cache_len == 1024 and c.get_seq_length() == 0
    c.data[..., :10, :] = 1.0
    c.ensure(1000)
    assert c.max_cache_len == 1024
    c.ensure(1025)
    assert c.max_cache_len == 2048 and c.data.shape[-2] == 2048
    assert float(c.data[..., :10, :].min()) == 1.0 and float(c.data[..., 10:, :].abs().max()) == 0.0   # contents carried over
    c.ensure(10000)
    assert c.max_cache_len == 10240
    c.crop(7)
    assert c.get_seq_length() == 7
    kv.reset()
    assert c.get_seq_length() == 0 and kv.get_seq_length() == 0
    import pytest
    with pytest.raises(ValueError):
        create_kv_cache("paged", config=cfg)
    with pytest.raises(ValueError):
        create_kv_cache("dynamic", config=None)
    static = create_kv_cache("static", max_cache_len=32, config=cfg, device="cpu", dtype=torch.float32)
    static.cache.ensure(32)
    with pytest.raises(ValueError):
        static.cache.ensure(33)


def _two_level_tree():
    t = Tree(torch.tensor(7))
    t.add_nodes(torch.tensor([[[10, 11, 12, 13], [20, 21, 22, 23]]]),
                torch.tensor([[[.4, .3, .2, .1], [.2, .15, .1, .05]]]),
                torch.tensor([[[0, 0, 0, 0], [0, 0, 1, 2]]]))
    return t


def test_truncate_keeps_the_frontier_positions_for_later_levels():
    """A tree cut to its first n nodes and extended afterwards: the new level names its parents by position in the
    level that was cut, so surviving positions must keep their nodes and cut positions must be refused -- not
    re-mapped onto whatever childless nodes remain."""
    t = _two_level_tree()                       # 9 nodes: root, level 1 = 1..4, level 2 = 5..8 (parents 1, 1, 2, 3)
    t.truncate(7)                               # drops nodes 7 and 8 (positions 2 and 3 of the frontier)
    assert t.size() == 7 and t.available_leaves == [5, 6]
    t.add_nodes(torch.tensor([[[30, 31]]]), torch.tensor([[[.1, .05]]]), torch.tensor([[[1, 0]]]))
    d = _data(t)
    assert d["parent_indices"][7:] == [6, 5] and d["depths"][7:] == [3, 3]
    # a parent position that was cut off is an error, not a silent re-parenting to a shallower node
    t2 = _two_level_tree()
    t2.truncate(7)
    with pytest.raises(ValueError, match="truncate"):
        t2.add_nodes(torch.tensor([[[30]]]), torch.tensor([[[.1]]]), torch.tensor([[[3]]]))
    # cutting nothing changes nothing
    t3 = _two_level_tree()
    t3.truncate(9)
    assert t3.available_leaves == [5, 6, 7, 8]
    # cutting the whole last level leaves NO frontier: the childless nodes of level 1 do not become expandable
    for n in (5, 3, 1):
        t4 = _two_level_tree()
        t4.truncate(n)
        assert t4.size() == n and t4.available_leaves == []
        with pytest.raises(ValueError, match="truncate"):
            t4.add_nodes(torch.tensor([[[30]]]), torch.tensor([[[.1]]]), torch.tensor([[[0]]]))
