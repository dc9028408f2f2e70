"""GPU parity: fused HIP verifier and KV compaction (through the C ABI) against the CPU oracle,
the reference's known-answer cases and the reference-written golden vectors.

Bar: accepted tokens, contexts, counts, argmax tokens and compacted KV are bit-exact; the
normalized entropy is bit-exact for 16-bit rows when evaluated with per-element rounding and
within 1e-5 relative for fp32 rows (fp32 sums depend on the summation order)."""
import json
import math
import os

import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import kv as okv
from oracle import verify as ov
from subspec_amd import ops, workloads as W
from subspec_amd.cpu_tree import Tree
from subspec_amd.tree_verify import verify_tree
from subspec_amd.wandb_logger import wandb_logger

GOLD = os.path.join(os.path.dirname(__file__), "golden")
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}
DEV = "cuda:0"


def _gold():
    with open(os.path.join(GOLD, "reference_vectors.json")) as f:
        return json.load(f)


def _run(logits, tokens, parents, **kw):
    out = ops.tree_verify(logits.to(DEV), torch.tensor(tokens, dtype=torch.int32, device=DEV),
                          torch.tensor(parents, dtype=torch.int32, device=DEV), **kw)
    torch.cuda.synchronize()
    return {k: v.cpu() for k, v in out.items()}


def _assert_entropy_matches(got, ref, tag):
    # Per-element rounding reproduced on the device: the values are the reference's own, except
    # that torch's CPU softmax accumulates sum(exp) in 16 fp32 lanes and the lane that holds a
    # dominant logit drops its small addends, which shifts S by up to ~3e-4 and can move the
    # rounded maximum probability (and with it the entropy of a peaked row) by one step.
    same = (got == ref).float().mean().item()
    assert same >= 0.95, (tag, same)
    assert torch.allclose(got, ref, rtol=2e-2, atol=1e-4), tag


def _unpack(out, b=0):
    emitted, accept, total, status = out["counts"][b].tolist()
    assert status == 0
    return out["tokens"][b, :emitted].tolist(), out["contexts"][b, :emitted].tolist(), (total, accept)


def test_known_answer_cases():
    with open(os.path.join(GOLD, "lossy_kat.json")) as f:
        cases = json.load(f)["cases"]
    for c in cases:
        print("KAT", c["name"], flush=True)
        rows = torch.tensor(c["rows"], dtype=torch.float32)
        probs = rows / rows.sum(-1, keepdim=True)
        logits = probs.log()                       # zeros become -inf: softmax(log p) == p
        out = _run(logits, c["token_ids"], c["parents"], verify_method="lossy", threshold_method="prob",
                   threshold=c["threshold"], window_size=c["window_size"])
        toks, ctx, (total, acc) = _unpack(out)
        exp = c["expect"]
        assert acc == exp["accept_len"]
        for key, got in (("sampled", toks), ("hidden", ctx)):
            if key in exp:
                assert got == exp[key]
            if key + "_prefix" in exp:
                assert got[: len(exp[key + "_prefix"])] == exp[key + "_prefix"]
        if "sampled_last" in exp:
            assert toks[-1] == exp["sampled_last"]


def test_reference_vectors_lossy():
    for i, c in enumerate(_gold()["lossy"]):
        print("gold lossy", i, c["dtype"], c["threshold_method"], flush=True)
        logits = torch.tensor(c["logits"]).to(DT[c["dtype"]])
        out = _run(logits, c["token_ids"], c["parents"], eos_token_id=c["eos_token_id"], verify_method="lossy",
                   threshold_method=c["threshold_method"], threshold=c["threshold"], window_size=c["window_size"],
                   exact_entropy=True)
        toks, ctx, (total, acc) = _unpack(out)
        assert (toks, ctx, acc) == (c["sampled"], c["hidden"], c["accept_len"]), i
        probs = torch.softmax(logits, -1)
        assert out["target"][0].tolist() == probs.argmax(-1).tolist()
        if c["threshold_method"] == "entropy":
            ref_h = torch.tensor(ov.normalized_entropy(probs))
            if c["dtype"] == "float32":
                assert torch.allclose(out["entropy"][0], ref_h, rtol=1e-5, atol=1e-6)
            else:
                assert torch.equal(out["entropy"][0], ref_h), i


def test_reference_vectors_verify_tree_with_skip_nodes():
    for i, c in enumerate(_gold()["verify_tree"]):
        print("gold verify_tree", i, c["verify_method"], c["skip_nodes"], flush=True)
        logits = torch.tensor(c["logits"]).to(DT[c["dtype"]])
        vk = c["verify_kwargs"]
        out = _run(logits, c["token_ids"], c["parents"], root=c["root"], skip_nodes=c["skip_nodes"],
                   eos_token_id=c["eos_token_id"], verify_method=c["verify_method"],
                   threshold_method=vk["threshold_method"], threshold=vk["threshold"], window_size=vk["window_size"],
                   exact_entropy=True)
        toks, ctx, (total, acc) = _unpack(out)
        assert toks == c["sampled"] and ctx == c["hidden"], i
        assert (total, acc) == (c["total_len"], c["accept_len"]), i


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_config1_greedy_fp32_full_vocab(seed):
    cfg = W.greedy_config(seed)
    exp_t, exp_c, exp_n = ov.verify_logits(cfg["logits"], cfg["tokens"], cfg["parents"])
    assert exp_c == cfg["path"]                                    # planted path, known by design
    out = _run(cfg["logits"], cfg["tokens"], cfg["parents"])
    assert _unpack(out) == (exp_t, exp_c, exp_n)
    assert out["target"][0].tolist() == torch.softmax(cfg["logits"], -1).argmax(-1).tolist()


def test_prepared_call_follows_its_tensors():
    """A prepared call launches on the tensors it was made with: new inputs are written INTO them, the outputs are
    the same dictionary every time, and every call agrees with the oracle and with a plain tree_verify call."""
    cfgs = [W.greedy_config(seed) for seed in (3, 4)]
    logits = cfgs[0]["logits"].to(DEV).clone()
    tok = torch.tensor(cfgs[0]["tokens"], dtype=torch.int32, device=DEV)
    par = torch.tensor(cfgs[0]["parents"], dtype=torch.int32, device=DEV)
    prepared = ops.PreparedTreeVerify(logits, tok, par)
    for cfg in cfgs + cfgs[:1]:
        logits.copy_(cfg["logits"])
        tok.copy_(torch.tensor(cfg["tokens"], dtype=torch.int32))
        par.copy_(torch.tensor(cfg["parents"], dtype=torch.int32))
        out = prepared()
        assert out is prepared.out
        torch.cuda.synchronize()
        got = {k: v.cpu() for k, v in out.items()}
        assert _unpack(got) == ov.verify_logits(cfg["logits"], cfg["tokens"], cfg["parents"])
        plain = _run(cfg["logits"], cfg["tokens"], cfg["parents"])
        for key in ("tokens", "contexts"):
            n = got["counts"][0, 0].item()
            assert torch.equal(got[key][0, :n], plain[key][0, :n]), key
        for key in ("counts", "target", "entropy", "child_prob"):
            assert torch.equal(got[key], plain[key]), key
    with pytest.raises(ValueError):
        ops.PreparedTreeVerify(logits, tok.to(torch.int64), par)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_config2_lossy_entropy_full_vocab(dtype):
    cfg = W.lossy_config(seed=3, batch=5, dtype=dtype)
    vk = dict(threshold=cfg["threshold"], window_size=cfg["window_size"], threshold_method="entropy")
    for exact_entropy in (False, True):
        out = _run(cfg["logits"], cfg["tokens"], cfg["parents"], verify_method="lossy", threshold_method="entropy",
                   threshold=cfg["threshold"], window_size=cfg["window_size"], exact_entropy=exact_entropy)
        for b in range(5):
            probs = torch.softmax(cfg["logits"][b], -1)
            exp = ov.verify_logits(cfg["logits"][b], cfg["tokens"][b], cfg["parents"][b], verify_method="lossy",
                                   verify_kwargs=vk)
            assert _unpack(out, b) == exp, (b, exact_entropy)
            assert out["target"][b].tolist() == probs.argmax(-1).tolist()
            ref_h = torch.tensor(ov.normalized_entropy(probs))
            if exact_entropy or dtype == torch.float16:
                _assert_entropy_matches(out["entropy"][b], ref_h, b)
            else:
                # single fp32 pass away from the threshold: the entropy sum and the quotient are each
                # rounded once to bf16, so the value lies within two bf16 steps of the reference's
                assert torch.allclose(out["entropy"][b], ref_h, rtol=2 ** -6, atol=1e-3), b
            # gate decisions agree everywhere
            assert torch.equal(out["entropy"][b] >= cfg["threshold"], ref_h >= cfg["threshold"])
    # accepted lengths cover exact chains, lossy accepts and gate rejections
    accepts = sorted({int(a) for a in out["counts"][:, 1]})
    assert accepts[0] == 0 and accepts[-1] == 8


def test_near_threshold_rows_take_the_rounded_path():
    # rows whose entropy sits right at the threshold: decisions must still equal the oracle's
    torch.manual_seed(7)
    V, n = 4096, 64
    logits = (torch.randn(n, V) * torch.linspace(2.6, 3.4, n).unsqueeze(1)).to(torch.bfloat16)
    probs = torch.softmax(logits, -1)
    ref_h = torch.tensor(ov.normalized_entropy(probs))
    theta = float(ref_h.median())
    parents = [-1] + [0] * (n - 1)
    tokens = list(range(n))
    out = _run(logits, tokens, parents, verify_method="lossy", threshold_method="entropy", threshold=theta,
               window_size=0)
    assert torch.equal(out["entropy"][0] >= theta, ref_h >= theta)
    near = (ref_h - theta).abs() <= 0.01 * theta
    assert near.sum() >= 3
    assert torch.equal(out["entropy"][0][near], ref_h[near])


# the long vocabularies are cut into slices (few rows): without the entropy gate the acceptance kernel then looks for
# ties of the rounded probabilities itself, with it the exact pass is a launch of its own
@pytest.mark.parametrize("dtype,vocab", [(torch.float16, 1001), (torch.float32, 777), (torch.bfloat16, 50257),
                                         (torch.bfloat16, 65536), (torch.float16, 40000), (torch.float32, 32768)])
def test_ragged_vocab_and_ties(dtype, vocab):
    torch.manual_seed(11)
    n = 9
    parents, tokens = [-1, 0, 0, 1, 1, 2, 3, 3, 6], [1, 5, 9, 2, 7, 3, 4, 8, 6]
    logits = (torch.randn(n, vocab) * 0.3).to(dtype)       # small maxima: rounded probabilities tie
    logits[2] = 0.0                                        # a constant row: argmax must be index 0
    logits[4, 100] = logits[4, 40] = logits[4].max() + 1   # duplicated maximum: first index wins
    # the maximum logit near the end of the row and, in the first slice, logits one and two steps of the dtype below it:
    # whether their probabilities round to the maximum's is the reference's rounding to decide; the index that wins lies
    # slices away from the maximum
    for r, steps in ((5, 1), (6, 2), (7, 1)):
        top = (logits[r].float().max() + 0.25).to(dtype)
        below = top.clone()
        for _ in range(steps):
            below = torch.nextafter(below, torch.tensor(-10.0, dtype=dtype))
        logits[r, vocab - 3] = top
        logits[r, 7 + r] = below
        if r == 7:
            logits[r, vocab // 2] = below
    probs = torch.softmax(logits, -1)
    for method, kw in (("exact", {}), ("lossy", dict(threshold_method="prob", threshold=0.0005, window_size=0)),
                       ("lossy", dict(threshold_method="entropy", threshold=0.99, window_size=1))):
        exp = ov.verify_logits(logits, tokens, parents, verify_method=method, verify_kwargs=kw)
        out = _run(logits, tokens, parents, verify_method=method, exact_entropy=True, **kw)
        assert _unpack(out) == exp
        assert out["target"][0].tolist() == probs.argmax(-1).tolist()


def test_masked_logits_and_single_node_tree():
    logits = torch.full((1, 4096), float("-inf"), dtype=torch.bfloat16)
    logits[0, 1234] = 0.5
    out = _run(logits, [3], [-1], verify_method="lossy", threshold_method="entropy", threshold=0.3, window_size=1)
    assert _unpack(out) == ([1234], [0], (1, 0))
    assert out["entropy"][0, 0] == 0.0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("rows,vocab", [(5, 70000), (300, 152064), (3, 8200)])
def test_mostly_masked_rows(dtype, rows, vocab):
    """Rows in which almost every logit is -inf (a constrained vocabulary): whole slices and whole trips of a slice
    hold nothing but -inf, the few finite logits sit in different slices, some next to the slice ends.  Few rows
    split a row over many workgroups, many rows take one workgroup per row (the long-slice variant of the pass)."""
    g = torch.Generator().manual_seed(rows + vocab)
    parents, toks, _ = W.random_tree(g, n=rows, max_depth=6, max_children=4, vocab=vocab, chain_depth=4)
    kids = ov.children_from_parents(parents)
    logits = torch.full((rows, vocab), float("-inf"))
    for r in range(rows):
        live = torch.randint(0, vocab, (4,), generator=g).tolist() + [0, vocab - 1] + [toks[c] for c in kids[r]]
        logits[r, live] = torch.randn(len(live), generator=g) * 3
        if kids[r] and r % 2 == 0:
            logits[r, toks[kids[r][0]]] = 9.0                      # drafted child wins: walks go deep
    logits = logits.to(dtype)
    for method, vk in (("exact", {}), ("lossy", {"threshold_method": "entropy", "threshold": 0.3, "window_size": 2}),
                       ("lossy", {"threshold_method": "prob", "threshold": 0.05, "window_size": 1})):
        print("masked rows", dtype, rows, vocab, method, flush=True)
        out = _run(logits, toks, parents, verify_method=method, exact_entropy=True,
                   threshold_method=vk.get("threshold_method", "prob"), threshold=vk.get("threshold", 0.0),
                   window_size=vk.get("window_size", 1))
        want = ov.verify_logits(logits, toks, parents, verify_method=method, verify_kwargs=vk)
        assert _unpack(out) == (want[0], want[1], want[2]), (rows, vocab, method)
        assert out["target"][0].tolist() == ov.target_probs(logits).argmax(-1).tolist()
        if vk.get("threshold_method") == "entropy":
            ref_h = torch.tensor(ov.normalized_entropy(ov.target_probs(logits)))
            if dtype == torch.float32:                       # one fp32 pass against torch's: equal up to summation order
                assert torch.allclose(out["entropy"][0], ref_h, rtol=1e-4, atol=1e-6)
            else:
                _assert_entropy_matches(out["entropy"][0], ref_h, "masked")


def test_verify_tree_host_interface_and_errors():
    cfg = W.greedy_config(5)
    tree = Tree(torch.tensor(cfg["tokens"][0]))
    # rebuild the random tree level by level through add_nodes is not possible for ragged levels;
    # use a tiny regular tree instead
    tree.add_nodes(torch.tensor([[[11, 12], [13, 14]]]), torch.tensor([[[0.6, 0.3], [0.5, 0.2]]]),
                   torch.tensor([[[0, 0], [0, 1]]]))
    logits = torch.randn(1, 5, 64)
    logits[0, 0, 11] = 9.0
    logits[0, 1, 13] = 9.0
    logits[0, 3, 40] = 9.0
    wandb_logger.clear_log_data()
    toks, ctx, (total, acc) = verify_tree(tree=tree, root_ind=0, logits=logits.to(DEV), eos_token_id=None,
                                          verify_method="exact")
    assert toks.tolist() == [[11, 13, 40]] and ctx.tolist() == [0, 1, 3] and (total, acc) == (2, 2)
    assert toks.device.type == "cpu" and toks.dtype == torch.int64
    toks, ctx, (total, acc) = verify_tree(tree=tree, root_ind=0, logits=logits.to(DEV), eos_token_id=None,
                                          verify_method="lossy", verify_kwargs=dict(threshold=0.3, window_size=1,
                                                                                    threshold_method="entropy"))
    assert toks.tolist() == [[11, 13, 40]] and (total, acc) == (3, 2)
    assert wandb_logger.log_data["verify_accept_tokens"] == 2.0
    with pytest.raises(ValueError):
        verify_tree(tree=tree, root_ind=0, logits=logits.to(DEV), eos_token_id=None, verify_method="bogus")
    with pytest.raises(ValueError):
        verify_tree(tree=tree, root_ind=0, logits=logits.to(DEV), eos_token_id=None, verify_method="lossy",
                    verify_kwargs=dict(threshold_method="bogus"))
    # sampling target through the same interface: the planted logits (+9 over N(0,1) rows) make the
    # drafted path the overwhelmingly likely draw at a low temperature
    from subspec_amd.tree_verify import SampleStream
    from transformers.generation.logits_process import LogitsProcessorList, TemperatureLogitsWarper
    toks, ctx, (total, acc) = verify_tree(tree=tree, root_ind=0, logits=logits.to(DEV), eos_token_id=None,
                                          logits_processor=LogitsProcessorList([TemperatureLogitsWarper(0.25)]),
                                          do_sample=True, stream=SampleStream(1))
    assert toks.tolist() == [[11, 13, 40]] and ctx.tolist() == [0, 1, 3] and (total, acc) == (2, 2)
    with pytest.raises(ValueError):            # more nodes than the kernels are built for
        ops.tree_verify(torch.zeros(513, 64, device=DEV), torch.zeros(513, dtype=torch.int32, device=DEV),
                        torch.zeros(513, dtype=torch.int32, device=DEV))
    # caller-provided outputs of the right shape but a narrower element type would be overrun by the kernels: refused
    lg = torch.zeros(5, 64, device=DEV)
    tk, pr = torch.zeros(5, dtype=torch.int32, device=DEV), torch.tensor([-1, 0, 0, 1, 1], dtype=torch.int32, device=DEV)
    good = ops.tree_verify(lg, tk, pr)
    for key, dtype in (("tokens", torch.int32), ("contexts", torch.int32), ("target", torch.int32), ("counts", torch.int64),
                       ("entropy", torch.bfloat16), ("child_prob", torch.float16)):
        bad = dict(good)
        bad[key] = torch.zeros_like(good[key], dtype=dtype)
        with pytest.raises(ValueError, match=key):
            ops.tree_verify(lg, tk, pr, out=bad)
    ops.tree_verify(lg, tk, pr, out=good)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_kv_compaction_bit_exact(dtype):
    torch.manual_seed(3)
    layers, heads, seq, hd = 6, 4, 300, 128
    cache = torch.randn(layers, 2, 1, heads, seq, hd).to(dtype)
    for ctx, offset in (([0, 1, 4, 10, 19, 27, 40, 55, 63], 200), ([0], 17), ([3, 2, 1, 0, 5], 100),
                        (list(range(0, 64, 1)), 236)):
        exp = okv.compact_static(cache, ctx, offset)
        dev = cache.to(DEV)
        ops.kv_compact_(dev, torch.tensor(ctx, dtype=torch.int64, device=DEV), offset)
        torch.cuda.synchronize()
        got = dev.cpu()
        assert torch.equal(got, exp)
        assert torch.equal(got[..., :offset, :], cache[..., :offset, :])                 # prefix untouched
        assert torch.equal(got[..., offset + len(ctx):, :], cache[..., offset + len(ctx):, :])   # tail stale
        # dynamic-cache view: the first offset+L rows equal the reference's truncated gather
        assert torch.equal(got[..., : offset + len(ctx), :], okv.compact_dynamic(cache, ctx, offset))


@pytest.mark.parametrize("count", [257, 300, 512])
def test_kv_compaction_of_long_paths(count):
    """More rows than a 256-node tree could accept: the accumulated contexts of consecutive post-verified cycles."""
    g = torch.Generator().manual_seed(count)
    cache = torch.randn(2, 2, 1, 2, 1200, 128, generator=g).to(torch.bfloat16)
    ctx = sorted(torch.randperm(1000, generator=g)[:count].tolist())
    exp = okv.compact_static(cache, ctx, 150)
    dev = cache.to(DEV)
    ops.kv_compact_(dev, torch.tensor(ctx, dtype=torch.int64, device=DEV), 150)
    torch.cuda.synchronize()
    assert torch.equal(dev.cpu(), exp)


def test_kv_compaction_count_from_device_follows_verifier():
    cfg = W.greedy_config(9)
    out = ops.tree_verify(cfg["logits"].to(DEV), torch.tensor(cfg["tokens"], dtype=torch.int32, device=DEV),
                          torch.tensor(cfg["parents"], dtype=torch.int32, device=DEV))
    cache = torch.randn(2, 2, 1, 4, 2048 + 64, 128).to(torch.bfloat16)
    dev = cache.to(DEV)
    ops.kv_compact_(dev, out["contexts"][0], 2048, count_dev=out["counts"][0, 0:1], max_count=65)
    torch.cuda.synchronize()
    emitted = int(out["counts"][0, 0])
    ctx = out["contexts"][0, :emitted].tolist()
    assert ctx == cfg["path"]
    assert torch.equal(dev.cpu(), okv.compact_static(cache, ctx, 2048))
    with pytest.raises(ValueError):
        ops.kv_compact_(dev[..., :7], out["contexts"][0], 0)                 # non-contiguous


@pytest.mark.parametrize("n", [65, 128, 129, 200, 256, 257, 289, 512])
def test_large_trees_up_to_the_node_limit(n):
    """Trees beyond one node per lane (2, 4 and 8 nodes per lane in the acceptance step; 289 = the reference's
    depth-48 x 6 tree), greedy and sampled targets, exact walk and both lossy gates, against the oracle; rows may be
    fewer than nodes."""
    g = torch.Generator().manual_seed(n)
    vocab = 777
    deep = n > 256
    parents, toks, depths = W.random_tree(g, n=n, max_depth=48 if deep else 12, max_children=6 if deep else 4, vocab=vocab,
                                          chain_depth=40 if deep else 10)
    kids = ov.children_from_parents(parents)
    for rows, dtype in ((n, torch.bfloat16), (n, torch.float32), (max(1, n - 40), torch.bfloat16)):
        logits = (torch.randn(rows, vocab, generator=g) * 2).to(dtype)
        for u in range(rows):                              # make drafted children frequent targets: deep walks
            if kids[u] and float(torch.rand(1, generator=g)) < 0.8:
                pick = kids[u][int(torch.randint(0, len(kids[u]), (1,), generator=g))]
                logits[u, toks[pick]] += 8.0
        for method, vk in (("exact", {}),
                           ("lossy", {"threshold_method": "prob", "threshold": 0.02, "window_size": 1}),
                           ("lossy", {"threshold_method": "entropy", "threshold": 0.7, "window_size": 2})):
            print("large tree", n, rows, dtype, method, vk, flush=True)
            out = _run(logits, toks, parents, verify_method=method, exact_entropy=True,
                       threshold_method=vk.get("threshold_method", "prob"), threshold=vk.get("threshold", 0.0),
                       window_size=vk.get("window_size", 1))
            want = ov.verify_logits(logits, toks, parents, verify_method=method, verify_kwargs=vk)
            got_t, got_c, got_m = _unpack(out)
            assert (got_t, got_c, got_m) == (want[0], want[1], want[2]), (n, rows, method)
            assert out["target"][0].tolist() == ov.target_probs(logits).argmax(-1).tolist()
            # sampled target: the walk / DP must follow the device's own draws exactly
            smp = _run(logits, toks, parents, verify_method=method, exact_entropy=True,
                       threshold_method=vk.get("threshold_method", "prob"), threshold=vk.get("threshold", 0.0),
                       window_size=vk.get("window_size", 1), do_sample=True, temperature=0.9, seed=n, offset=rows)
            drawn = smp["target"][0].tolist()
            want = ov.verify_logits(logits, toks, parents, verify_method=method, verify_kwargs=vk, temperature=0.9,
                                    target_tokens=drawn)
            got_t, got_c, got_m = _unpack(smp)
            assert (got_t, got_c, got_m) == (want[0], want[1], want[2]), (n, rows, method, "sampled")
