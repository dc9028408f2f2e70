"""Pins the CPU oracle's verifiers: reference known-answer cases, reference-written golden
vectors, brute force on tiny trees, and invariants.  No GPU."""
import json
import os

import pytest
import torch

from oracle import verify as ov

GOLD = os.path.join(os.path.dirname(__file__), "golden")
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}


def _kat_cases():
    with open(os.path.join(GOLD, "lossy_kat.json")) as f:
        return json.load(f)["cases"]


def _gold():
    with open(os.path.join(GOLD, "reference_vectors.json")) as f:
        return json.load(f)


@pytest.mark.parametrize("case", _kat_cases(), ids=lambda c: c["name"])
def test_lossy_known_answers(case):
    rows = torch.tensor(case["rows"], dtype=torch.float32)
    probs = rows / rows.sum(dim=-1, keepdim=True)
    internal, log = {}, {}
    toks, ctx, acc = ov.lossy_verify(
        probs, case["token_ids"], case["children"], 0, case["eos_token_id"],
        threshold=case["threshold"], window_size=case["window_size"],
        threshold_method=case["threshold_method"], internal=internal, log=log)
    exp = case["expect"]
    assert acc == exp["accept_len"]
    if "sampled" in exp:
        assert toks == exp["sampled"]
    if "hidden" in exp:
        assert ctx == exp["hidden"]
    if "sampled_prefix" in exp:
        assert toks[: len(exp["sampled_prefix"])] == exp["sampled_prefix"]
    if "hidden_prefix" in exp:
        assert ctx[: len(exp["hidden_prefix"])] == exp["hidden_prefix"]
    if "sampled_last" in exp:
        assert toks[-1] == exp["sampled_last"]
    for key, val in exp.get("log", {}).items():
        assert abs(log[key] - val) < 1e-6, key
    # children lists derived from the parent array agree with the hand-written ones
    assert ov.children_from_parents(case["parents"]) == case["children"]


@pytest.mark.parametrize("idx", range(40))
def test_lossy_reference_vectors(idx):
    c = _gold()["lossy"][idx]
    logits = torch.tensor(c["logits"]).to(DT[c["dtype"]])
    probs = torch.softmax(logits, dim=-1)
    internal, log = {}, {}
    toks, ctx, acc = ov.lossy_verify(
        probs, c["token_ids"], ov.children_from_parents(c["parents"]), 0, c["eos_token_id"],
        threshold=c["threshold"], window_size=c["window_size"],
        threshold_method=c["threshold_method"], internal=internal, log=log)
    assert (toks, ctx, acc) == (c["sampled"], c["hidden"], c["accept_len"])
    for key, val in c["log"].items():
        if isinstance(val, str):
            assert log[key] == val
        else:
            assert abs(log[key] - val) < 1e-9, key


@pytest.mark.parametrize("idx", range(len(_gold()["verify_tree"])))
def test_verify_tree_reference_vectors(idx):
    c = _gold()["verify_tree"][idx]
    logits = torch.tensor(c["logits"]).to(DT[c["dtype"]])
    toks, ctx, (total, acc) = ov.verify_logits(
        logits, c["token_ids"], c["parents"], c["root"], c["eos_token_id"], c["skip_nodes"],
        c["verify_method"], c["verify_kwargs"])
    assert toks == c["sampled"]
    assert ctx == c["hidden"]
    assert (total, acc) == (c["total_len"], c["accept_len"])


def _random_tree(g, n, max_kids, vocab):
    parents, toks, nk = [-1], [0], [0]
    for i in range(1, n):
        while True:
            p = int(torch.randint(0, i, (1,), generator=g))
            if nk[p] < max_kids:
                break
        nk[p] += 1
        nk.append(0)
        sib = {toks[j] for j in range(1, i) if parents[j] == p}
        while True:
            t = int(torch.randint(0, vocab, (1,), generator=g))
            if t not in sib:
                break
        parents.append(p)
        toks.append(t)
    return parents, toks


@pytest.mark.parametrize("seed", range(30))
def test_lossy_matches_brute_force_and_exact(seed):
    g = torch.Generator().manual_seed(seed)
    n, vocab = 9, 7
    parents, toks = _random_tree(g, n, 3, vocab)
    kids = ov.children_from_parents(parents)
    logits = torch.randn(n, vocab, generator=g) * 2.5
    for u in range(n):               # plant some exact edges so chains exist
        if kids[u] and float(torch.rand(1, generator=g)) < 0.6:
            logits[u, toks[kids[u][0]]] += 6.0
    probs = torch.softmax(logits, -1)
    for method, theta in (("entropy", 0.5), ("prob", 0.1), ("entropy", 2.0), ("prob", 0.0)):
        for window in (0, 1, 2):
            _, ctx, acc = ov.lossy_verify(probs, toks, kids, 0, None, theta, window, method)
            assert acc == ov.brute_force_lossy_len(probs, toks, kids, 0, theta, window, method)
            assert len(ctx) == acc + 1 and ctx[0] == 0
            for a, b in zip(ctx, ctx[1:]):
                assert parents[b] == a                      # a root path
    # theta = 0 with the entropy gate blocks every lossy edge -> identical to the exact walk
    t_l, c_l, a_l = ov.lossy_verify(probs, toks, kids, 0, None, 0.0, 3, "entropy")
    t_e, c_e, (_, a_e) = ov.exact_verify(probs, toks, kids, 0, None)
    assert (t_l, c_l, a_l) == (t_e, c_e, a_e)


def test_exact_planted_path_and_eos():
    g = torch.Generator().manual_seed(5)
    parents = [-1, 0, 0, 1, 1, 3, 3, 5]
    toks = [9, 4, 6, 2, 8, 1, 3, 7]
    kids = ov.children_from_parents(parents)
    logits = torch.randn(8, 12, generator=g)
    for u, c in ((0, 1), (1, 3), (3, 5)):      # planted path 0->1->3->5, stop at 5 (argmax 11)
        logits[u, toks[c]] = 9.0
    logits[5, 11] = 9.0
    probs = torch.softmax(logits, -1)
    t, c, (total, acc) = ov.exact_verify(probs, toks, kids, 0, None)
    assert t == [4, 2, 1, 11] and c == [0, 1, 3, 5] and (total, acc) == (4, 3)
    # EOS inside the path stops the walk and suppresses the bonus token
    t, c, (total, acc) = ov.exact_verify(probs, toks, kids, 0, eos_token_id=2)
    assert t == [4, 2] and c == [0, 1] and (total, acc) == (2, 2)


def test_entropy_closed_form_and_errors():
    p = torch.full((1, 16), 1 / 16.0)
    assert abs(ov.normalized_entropy(p)[0] - 1.0) < 1e-6        # uniform -> 1
    q = torch.zeros(1, 16)
    q[0, 3] = 1.0
    assert ov.normalized_entropy(q)[0] == 0.0                   # one-hot -> 0
    with pytest.raises(ValueError):
        ov.lossy_verify(p, [0], [[]], 0, None, 0.1, 1, "bogus")
    with pytest.raises(ValueError):
        ov.verify_logits(torch.zeros(1, 4), [0], [-1], verify_method="nope")
