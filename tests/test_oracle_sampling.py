"""Pins the sampling part of the CPU oracle: Philox4x32-10 against Random123's known-answer
vectors, the exponential race against a per-element loop and against the distribution it must
reproduce, and the verifiers with pre-drawn target tokens against brute force and closed cases.
No GPU."""
import math

import numpy as np
import pytest
import torch

from oracle import sampling as osamp
from oracle import verify as ov
from test_oracle_verify import _random_tree

# Random123 (philox.h, kat_vectors): counter, key -> output, Philox4x32 with 10 rounds
PHILOX_KAT = [
    ((0x00000000,) * 4, (0x00000000,) * 2, (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
    ((0xffffffff,) * 4, (0xffffffff,) * 2, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
    ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
     (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)),
]


@pytest.mark.parametrize("ctr,key,out", PHILOX_KAT)
def test_philox_known_answers(ctr, key, out):
    got = osamp.philox4x32_10(np.array(ctr), np.array(key))
    assert [int(x) for x in got] == list(out)


def test_philox_is_vectorised_consistently():
    ctr = np.array([k[0] for k in PHILOX_KAT])
    key = np.array([k[1] for k in PHILOX_KAT])
    got = osamp.philox4x32_10(ctr, key)
    assert got.tolist() == [list(k[2]) for k in PHILOX_KAT]


def test_uniforms_layout_and_range():
    u = osamp.race_uniforms(row=5, vocab=11, seed=0x1234567890abcdef, offset=(7 << 32) | 3)
    assert u.shape == (11,) and (u > 0).all() and (u < 1).all()
    assert (u.astype(np.float32).astype(np.float64) == u).all()          # exact in fp32
    # element i is word i % 4 of the block with counter (i // 4, row, offset lo, offset hi)
    for i in (0, 3, 4, 10):
        w = osamp.philox4x32_10(np.array([i // 4, 5, 3, 7]), np.array([0x90abcdef, 0x12345678]))
        assert u[i] == ((int(w[i % 4]) >> 9) + 0.5) * 2.0 ** -23
    # rows, offsets and seeds give different streams
    base = osamp.race_uniforms(0, 64, 1, 0)
    for other in (osamp.race_uniforms(1, 64, 1, 0), osamp.race_uniforms(0, 64, 2, 0), osamp.race_uniforms(0, 64, 1, 1)):
        assert (base != other).mean() > 0.9


def test_draw_matches_elementwise_loop():
    g = torch.Generator().manual_seed(0)
    probs = torch.softmax(torch.randn(6, 13, generator=g) * 2, -1)
    toks, margins = osamp.draw_tokens(probs, seed=99, offset=4, first_row=2)
    for r in range(6):
        u = osamp.race_uniforms(2 + r, 13, 99, 4)
        best, arg = -1.0, -1
        for i in range(13):
            key = float(probs[r, i]) / -math.log(u[i])
            if key > best:
                best, arg = key, i
        assert toks[r] == arg
        assert 0.0 < margins[r] <= 1.0


def test_draw_frequencies_follow_the_probabilities():
    # chi-square of 64 x 400 draws against an 8-way distribution (fixed seed: deterministic)
    p = torch.tensor([0.30, 0.22, 0.17, 0.12, 0.09, 0.05, 0.04, 0.01], dtype=torch.float64)
    counts = np.zeros(8)
    n_rows = 64
    for off in range(400):
        toks, _ = osamp.draw_tokens(p.expand(n_rows, 8), seed=2024, offset=off)
        counts += np.bincount(toks, minlength=8)
    n = counts.sum()
    chi2 = float((((counts - n * p.numpy()) ** 2) / (n * p.numpy())).sum())
    assert chi2 < 24.3                                   # 99.9 % quantile of chi-square with 7 dof
    # zero-probability entries are never drawn
    q = torch.tensor([[0.0, 0.5, 0.0, 0.5]] * 50, dtype=torch.float64)
    toks, _ = osamp.draw_tokens(q, seed=3)
    assert set(toks) <= {1, 3}


def test_warp_probs_rounds_the_quotient_first():
    g = torch.Generator().manual_seed(1)
    lg = (torch.randn(3, 40, generator=g) * 3).to(torch.bfloat16)
    got = osamp.warp_probs(lg, 0.7)
    want = torch.softmax((lg.float() / 0.7).to(torch.bfloat16), -1)      # quotient rounded to bf16, then softmax
    assert torch.equal(got, want)
    assert torch.equal(osamp.warp_probs(lg, 1.0), torch.softmax(lg, -1))


def test_exact_walk_follows_the_drawn_tokens():
    parents = [-1, 0, 0, 1, 1, 3, 3, 5]
    toks = [9, 4, 6, 2, 8, 1, 3, 7]
    kids = ov.children_from_parents(parents)
    probs = torch.full((8, 12), 1.0 / 12)
    drawn = [6, 0, 0, 0, 0, 0, 0, 0]                     # root draws node 2's token; node 2 is a leaf
    t, c, (total, acc) = ov.exact_verify(probs, toks, kids, 0, None, target_tokens=drawn)
    assert t == [6, 0] and c == [0, 2] and (total, acc) == (1, 1)
    drawn = [4, 2, 0, 1, 0, 10, 0, 0]                    # path 0 -> 1 -> 3 -> 5, node 5 draws a token no child has
    t, c, (total, acc) = ov.exact_verify(probs, toks, kids, 0, None, target_tokens=drawn)
    assert t == [4, 2, 1, 10] and c == [0, 1, 3, 5] and (total, acc) == (4, 3)
    drawn = [11] + [0] * 7                               # first draw matches no child: the draw is the bonus token
    t, c, (total, acc) = ov.exact_verify(probs, toks, kids, 0, None, target_tokens=drawn)
    assert t == [11] and c == [0] and (total, acc) == (1, 0)
    # the argmax as "draw" is the greedy walk
    g = torch.Generator().manual_seed(3)
    probs = torch.softmax(torch.randn(8, 12, generator=g) * 3, -1)
    assert ov.exact_verify(probs, toks, kids, 0, None, target_tokens=probs.argmax(-1).tolist()) == \
        ov.exact_verify(probs, toks, kids, 0, None)


@pytest.mark.parametrize("seed", range(20))
def test_lossy_with_drawn_targets_matches_brute_force(seed):
    g = torch.Generator().manual_seed(100 + seed)
    n, vocab = 9, 7
    parents, toks = _random_tree(g, n, 3, vocab)
    kids = ov.children_from_parents(parents)
    probs = torch.softmax(torch.randn(n, vocab, generator=g) * 2.0, -1)
    drawn, _ = osamp.draw_tokens(probs, seed=seed, offset=1)
    for u in range(n):                                   # make some draws hit a child so chains exist
        if kids[u] and float(torch.rand(1, generator=g)) < 0.5:
            drawn[u] = toks[kids[u][0]]
    for method, theta in (("entropy", 0.9), ("prob", 0.1), ("prob", 0.0)):
        for window in (0, 1, 2):
            out, ctx, acc = ov.lossy_verify(probs, toks, kids, 0, None, theta, window, method, target_tokens=drawn)
            assert acc == ov.brute_force_lossy_len(probs, toks, kids, 0, theta, window, method, target_tokens=drawn)
            assert out[-1] == drawn[ctx[-1]]             # the bonus token is the last context's draw
    # an entropy gate that blocks everything reduces the DP to the exact walk with the same draws
    t_l, c_l, a_l = ov.lossy_verify(probs, toks, kids, 0, None, 0.0, 3, "entropy", target_tokens=drawn)
    t_e, c_e, (_, a_e) = ov.exact_verify(probs, toks, kids, 0, None, target_tokens=drawn)
    assert (t_l, c_l, a_l) == (t_e, c_e, a_e)
