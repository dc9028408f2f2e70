"""GPU parity of the sampling verifier (through the C ABI) against the CPU oracle.

Bar: the race is evaluated in fp32 on the device and in float64 by the oracle, and the device
rounds its own softmax; a drawn token may therefore differ from the oracle's only where the
oracle's two best race keys are closer than the rounding of one probability (2^-6 relative for
bf16 rows, 2^-9 for fp16 rows, 1e-5 for fp32 rows), and the device's token must then be that runner-up class: its
key is within the same margin of the best.  Given the drawn tokens, the accepted tokens, contexts
and counts of the walk / DP are bit-exact."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import sampling as osamp
from oracle import verify as ov
from subspec_amd import ops
from test_oracle_verify import _random_tree

DEV = "cuda:0"
MARGIN = {torch.float32: 1e-5, torch.bfloat16: 2.0 ** -6, torch.float16: 2.0 ** -9}


def _check_draws(logits, temperature, got, seed, offset, first_row=0):
    """got: device draws for the rows of ``logits`` (cpu tensor).  Returns the number of near-tie rows."""
    probs = osamp.warp_probs(logits, temperature)
    want, margins = osamp.draw_tokens(probs, seed, offset, first_row)
    tol = MARGIN[logits.dtype]
    near = 0
    for r, (g, w, m) in enumerate(zip(got.tolist(), want, margins)):
        if g == w:
            continue
        near += 1
        assert m < tol, (r, g, w, m)
        u = osamp.race_uniforms(first_row + r, probs.shape[1], seed, offset)
        keys = probs[r].double().numpy() / -np.log(u)
        assert keys[g] >= keys[w] * (1 - 2 * tol), (r, g, w)
    return near


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("vocab", [1000, 4099, 32000, 152064])
def test_draws_match_oracle(dtype, vocab):
    g = torch.Generator().manual_seed(vocab)
    rows = 24
    print("draws", dtype, vocab, flush=True)
    logits = (torch.randn(rows, vocab, generator=g) * 3).to(dtype)
    logits[3, 17] = 25.0                                  # a peaked row
    near = 0
    for temperature, seed, offset in ((1.0, 7, 0), (0.7, 7, 1), (0.2, 2 ** 63 + 5, 2 ** 40 + 3)):
        got = ops.sample_tokens(logits.to(DEV), temperature, seed, offset).cpu()
        near += _check_draws(logits, temperature, got, seed, offset)
    assert near <= 4


def test_draw_frequencies_on_device():
    # 256 rows x 300 offsets of one 16-way distribution: chi-square against the rounded probabilities
    p = torch.tensor([0.25, 0.18, 0.14, 0.10, 0.08, 0.06, 0.05, 0.04, 0.03, 0.02, 0.02, 0.01, 0.01, 0.005, 0.003, 0.002])
    logits = p.log().to(torch.bfloat16).expand(256, 16).contiguous().to(DEV)
    counts = torch.zeros(16, dtype=torch.int64, device=DEV)
    for off in range(300):
        counts += torch.bincount(ops.sample_tokens(logits, 1.0, 11, off), minlength=16)
    probs = torch.softmax(logits[0].cpu(), -1).double()
    probs = probs / probs.sum()
    n = float(counts.sum())
    chi2 = float((((counts.cpu().double() - n * probs) ** 2) / (n * probs)).sum())
    print("chi2", chi2, flush=True)
    assert chi2 < 37.7                                    # 99.9 % quantile, 15 degrees of freedom


def _verify_case(seed, dtype, method, vk, skip, temperature):
    g = torch.Generator().manual_seed(seed)
    n, vocab = 40, 515
    parents, toks = _random_tree(g, n, 4, vocab)
    rows = n - skip
    logits = (torch.randn(rows, vocab, generator=g) * 2.5).to(dtype)
    kids = ov.children_from_parents(parents)
    for u in range(skip, n):                              # make the drafted children likely draws
        for c in kids[u]:
            logits[u - skip, toks[c]] += 5.0
    sd, off = 1000 + seed, seed
    out = ops.tree_verify(logits.to(DEV), torch.tensor(toks, dtype=torch.int32, device=DEV),
                          torch.tensor(parents, dtype=torch.int32, device=DEV), root=skip, skip_nodes=skip,
                          verify_method=method, threshold_method=vk.get("threshold_method", "prob"),
                          threshold=vk.get("threshold", 0.0), window_size=vk.get("window_size", 1),
                          exact_entropy=True, do_sample=True, temperature=temperature, seed=sd, offset=off)
    torch.cuda.synchronize()
    out = {k: v.cpu() for k, v in out.items()}
    drawn = out["target"][0]
    _check_draws(logits, temperature, drawn, sd, off)
    emitted, accept, total, status = out["counts"][0].tolist()
    assert status == 0
    want_t, want_c, (want_total, want_acc) = ov.verify_logits(
        logits, toks, parents, root=skip, skip_nodes=skip, verify_method=method, verify_kwargs=vk,
        temperature=temperature, target_tokens=drawn.tolist())
    assert out["tokens"][0, :emitted].tolist() == want_t
    assert out["contexts"][0, :emitted].tolist() == want_c
    assert (total, accept) == (want_total, want_acc)
    # the child probabilities refer to the warped rows
    probs = osamp.warp_probs(logits, temperature)
    for i in range(skip, n):
        pr = parents[i] - skip
        if 0 <= pr < rows:
            assert float(out["child_prob"][0, i - skip]) == float(probs[pr, toks[i]]) or \
                abs(float(out["child_prob"][0, i - skip]) - float(probs[pr, toks[i]])) <= 2.0 ** -7 * float(probs[pr, toks[i]])
    return accept


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_sampling_verify_matches_oracle(dtype):
    accepted = 0
    for seed in range(6):
        for method, vk in (("exact", {}),
                           ("lossy", {"threshold_method": "prob", "threshold": 0.05, "window_size": 1}),
                           ("lossy", {"threshold_method": "entropy", "threshold": 0.6, "window_size": 0})):
            for skip, temperature in ((0, 0.7), (3, 1.0), (0, 0.2)):
                print("sampling verify", dtype, seed, method, vk, skip, temperature, flush=True)
                accepted += _verify_case(seed, dtype, method, vk, skip, temperature)
    assert accepted > 0                                   # the cases do walk into the tree


def test_sampling_is_reproducible_and_offsets_differ():
    g = torch.Generator().manual_seed(0)
    logits = (torch.randn(64, 32000, generator=g) * 2).to(torch.bfloat16).to(DEV)
    a = ops.sample_tokens(logits, 0.8, 5, 9)
    b = ops.sample_tokens(logits, 0.8, 5, 9)
    c = ops.sample_tokens(logits, 0.8, 5, 10)
    assert torch.equal(a, b)
    assert (a != c).float().mean().item() > 0.5


def test_sampling_argument_errors():
    logits = torch.zeros(2, 16, device=DEV)
    tok = torch.zeros(2, dtype=torch.int32, device=DEV)
    par = torch.tensor([-1, 0], dtype=torch.int32, device=DEV)
    for bad in (0.0, -1.0, float("inf"), float("nan")):
        with pytest.raises(ValueError):
            ops.tree_verify(logits, tok, par, do_sample=True, temperature=bad)


def test_warpers_restrict_the_draw():
    """top-k / top-p go through HuggingFace's own warpers on the device; the draw must respect them."""
    from transformers.generation.logits_process import (LogitsProcessorList, TemperatureLogitsWarper,
                                                        TopKLogitsWarper, TopPLogitsWarper)
    from subspec_amd.tree_verify import SampleStream, sample_token
    g = torch.Generator().manual_seed(8)
    logits = (torch.randn(1, 48, 4096, generator=g) * 2).to(torch.bfloat16)
    top = logits.float().argmax(-1)
    logits.scatter_(-1, top.unsqueeze(-1), 12.0)           # a unique maximum per row
    dev = logits.to(DEV)
    st = SampleStream(3)
    # top_k = 1 leaves one token per row: whatever the noise, the draw is the argmax
    got = sample_token(dev, LogitsProcessorList([TopKLogitsWarper(top_k=1)]), True, stream=st)
    assert torch.equal(got.cpu(), top)
    # top_k = 5 after a temperature: every draw lies in the row's five best
    flat = (torch.randn(1, 48, 4096, generator=g) * 0.5).to(torch.bfloat16)
    procs = LogitsProcessorList([TemperatureLogitsWarper(1.5), TopKLogitsWarper(top_k=5)])
    best5 = (flat.float() / 1.5).to(torch.bfloat16).float().topk(5, -1)
    kth = best5.values[..., -1:]
    for _ in range(5):
        got = sample_token(flat.to(DEV), procs, True, stream=st).cpu()
        val = torch.gather((flat.float() / 1.5).to(torch.bfloat16).float(), -1, got.unsqueeze(-1))
        assert (val >= kth).all()
    # top_p keeps the smallest head of the sorted distribution whose mass reaches p
    procs = LogitsProcessorList([TopPLogitsWarper(top_p=0.5)])
    probs = torch.softmax(flat.float(), -1)
    sp, si = probs.sort(-1, descending=True)
    keep = (sp.cumsum(-1) - sp) < 0.5 + 1e-3               # tokens whose preceding mass is below p (with slack)
    allowed = torch.zeros_like(probs, dtype=torch.bool).scatter(-1, si, keep)
    for _ in range(5):
        got = sample_token(flat.to(DEV), procs, True, stream=st).cpu()
        assert torch.gather(allowed, -1, got.unsqueeze(-1)).all()
    assert st.offset == 11                                 # one stream position per sampling call


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_temperature_quotient_is_the_ieee_quotient(dtype):
    """The kernels divide with a reciprocal and one correction step; the result must be the correctly
    rounded quotient that ``tensor / T`` gives on the CPU.  Exhaustive over all 16-bit patterns,
    4M random values of mixed magnitude for fp32; nonzero inputs below 1e-30 in magnitude are left
    out (the residual of the correction step must itself be a normal fp32 number; logits that
    small do not occur)."""
    if dtype == torch.float32:
        g = torch.Generator().manual_seed(0)
        x = torch.randn(1 << 22, generator=g) * torch.exp(torch.randn(1 << 22, generator=g) * 6)
        x = torch.cat([x, torch.tensor([0.0, -0.0, float("inf"), float("-inf"), 1.0, -1.0, 3.4e38, 1.2e-38])])
    else:
        x = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype)
    x = x[~x.float().isnan() & ((x.float().abs() >= 1e-30) | (x.float() == 0))]
    for t in (0.2, 0.7, 0.5, 1.5, 3.0, 0.01, 1.0 / 3.0, 100.0, 1e-3, 0.9999999, 1.0000001):
        got = ops.temperature_warp(x.to(DEV), t).cpu()
        want = x / t
        ok = (got == want) | (got.isnan() & want.isnan())
        bad = (~ok).nonzero().flatten()
        assert bad.numel() == 0, (dtype, t, x[bad[:4]].tolist(), got[bad[:4]].tolist(), want[bad[:4]].tolist())
