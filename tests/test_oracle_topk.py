"""Pins the top-k oracle: brute force on tiny inputs, torch.topk values bit for bit, tie rule.  No GPU."""
import pytest
import torch

from oracle import topk as ot


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_canonical_topk_matches_brute_force_and_torch_values(dtype):
    g = torch.Generator().manual_seed(4)
    for B, L, V, k in ((2, 3, 17, 5), (1, 1, 9, 9), (3, 4, 33, 40)):
        probs = torch.softmax(torch.randn(B, L, V, generator=g) * 2, -1).to(dtype)
        parent = torch.rand(B, L, generator=g).to(dtype)
        tok, val, par = ot.topk_expand(probs, parent, k)
        tok_b, val_b, par_b = ot.topk_brute_force(probs, parent, k)
        assert torch.equal(tok, tok_b) and torch.equal(par, par_b) and torch.equal(val, val_b)
        tok_t, val_t, par_t = ot.topk_expand_torch(probs, parent, k)
        assert torch.equal(val, val_t)                               # values bit-exact
        assert tok.shape == (B, min(k, V))


def test_ties_resolve_to_lowest_flat_index():
    probs = torch.zeros(1, 2, 8)
    probs[0, 0, 5] = probs[0, 1, 2] = probs[0, 0, 1] = 0.25
    parent = torch.ones(1, 2)
    tok, val, par = ot.topk_expand(probs, parent, 5)
    assert tok.tolist() == [[1, 5, 2, 0, 2]] and par.tolist() == [[0, 0, 1, 0, 0]]
    assert val.tolist() == [[0.25, 0.25, 0.25, 0.0, 0.0]]


def test_bf16_full_vocab_values_equal_torch_topk():
    g = torch.Generator().manual_seed(9)
    V = 152064
    probs = torch.softmax(torch.randn(4, 1, V, generator=g).to(torch.bfloat16), -1)
    parent = torch.rand(4, 1, generator=g).to(torch.bfloat16)
    tok, val, par = ot.topk_expand(probs, parent, 16)
    tok_t, val_t, par_t = ot.topk_expand_torch(probs, parent, 16)
    assert torch.equal(val, val_t)
    buf = (probs * parent.unsqueeze(-1)).view(4, -1)
    flat, flat_t = par * V + tok, par_t * V + tok_t
    assert torch.equal(torch.gather(buf, 1, flat_t), val)            # torch's picks carry the same values
    # canonical order: within equal values the flat index increases
    for b in range(4):
        for i in range(15):
            assert val[b, i] > val[b, i + 1] or flat[b, i] < flat[b, i + 1]
