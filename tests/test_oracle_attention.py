"""Pins the attention oracle: explicit softmax(QK^T)V == F.scaled_dot_product_attention with the
additive mask; mask == the host tree's create_attention_mask; single-key special case.  No GPU."""
import pytest
import torch

from oracle import attention as oa
from subspec_amd import ops, workloads as W
from subspec_amd.cpu_tree import Tree


def test_explicit_equals_sdpa_and_mask_properties():
    g = torch.Generator().manual_seed(0)
    parents, _, _ = W.random_tree(g, n=12, max_depth=4, max_children=3, vocab=100)
    B, Hq, Hkv, n, D, P, S = 2, 4, 2, 12, 16, 20, 40
    q = torch.randn(B, Hq, n, D, generator=g).to(torch.bfloat16)
    k = torch.randn(B, Hkv, S, D, generator=g).to(torch.bfloat16)
    v = torch.randn(B, Hkv, S, D, generator=g).to(torch.bfloat16)
    a = oa.tree_attention(q, k, v, parents, P)
    b = oa.tree_attention_sdpa(q, k, v, parents, P)
    assert torch.allclose(a, b, rtol=1e-5, atol=1e-5)
    # rows beyond prefix+n never matter: poison them
    k2, v2 = k.clone(), v.clone()
    k2[:, :, P + n:] = 1e4
    v2[:, :, P + n:] = -1e4
    assert torch.allclose(oa.tree_attention(q, k2, v2, parents, P), a)
    # node 0 (root) with an empty prefix attends to itself only -> output is its own V row
    o0 = oa.tree_attention(q, k, v, parents, 0)
    assert torch.allclose(o0[:, 0].view(B, Hq, D), v[:, :, 0].float().repeat_interleave(2, dim=1), atol=1e-6)


def test_mask_matches_host_tree_and_bitsets():
    t = Tree(torch.tensor(1))
    t.add_nodes(torch.tensor([[[5, 6, 7], [8, 9, 10]]]), torch.rand(1, 2, 3), torch.tensor([[[0, 0, 0], [0, 0, 2]]]))
    parents = t.get_tree_data()["parent_indices"].tolist()
    m = oa.allowed_mask(parents, 3, 3 + t.size())
    assert torch.equal(m, t.create_attention_mask(3)[0, 0])
    bits = ops.ancestor_bits_tensor(parents).tolist()
    assert bits == t.ancestor_bits()
    for i, w in enumerate(bits):
        assert [bool((w >> j) & 1) for j in range(t.size())] == m[i, 3:].tolist()


def test_mask_words_of_large_trees():
    """Trees beyond 64 nodes: word w of row i holds the slots 64 w .. 64 w + 63 (as signed 64-bit integers) of the
    same ancestor-or-self relation the dense mask of the oracle describes."""
    from subspec_amd import workloads as W
    for n, depth in ((65, 10), (289, 48), (512, 60)):
        parents, _, _ = W.random_tree(torch.Generator().manual_seed(n), n=n, max_depth=depth, max_children=6, vocab=1000,
                                      chain_depth=depth)
        words = ops.ancestor_bits_tensor(parents)
        assert words.shape == (n, (n + 63) // 64) and words.dtype == torch.int64
        m = oa.allowed_mask(parents, 0, n)
        for i in (0, 1, 63, 64, n // 2, n - 1):
            row = [bool((int(words[i, j // 64]) >> (j % 64)) & 1) for j in range(n)]
            assert row == m[i].tolist(), (n, i)
    with pytest.raises(ValueError):
        ops.ancestor_bits_tensor([-1] + list(range(512)))
