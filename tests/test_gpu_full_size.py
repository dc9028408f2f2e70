"""GPU: the benchmark workload at its FULL size (32 trees x 64 nodes x 152064 bf16 logits, top-16 of
2048 x 152064 bf16 rows), checked through properties that do not need the CPU oracle at that size:

  * batch independence: a tree verified inside the 32-tree batch gives exactly what it gives alone,
    and a sample of trees equals the oracle;
  * determinism: a second launch is bit-identical;
  * permutation: reordering the trees reorders the outputs;
  * planted flavours: trees built with an all-exact depth-8 path accept all 8 draft tokens, trees
    with nothing planted accept none;
  * sampling verifier at the same size: seeded draws are reproducible, a tree's draws do not depend
    on the trees around it once its global row numbers are the same, every emitted token of the
    exact verifier is the draw of its context, a sample of rows equals the oracle's draws, and the
    drawn tokens' mean log-probability sits at minus the mean row entropy (what sampling from
    the rows themselves gives, and what neither argmax nor uniform draws give);
  * top-k: every value is the rounded product of its (row, token) probability and the parent
    probability, values are sorted (ties by index), and the count of strictly larger / larger-or-equal
    products brackets k for every row (checked with torch on the device)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import verify as ov
from subspec_amd import ops, workloads as W

DEV = "cuda:0"
KEYS = ("tokens", "contexts", "counts", "target")


def _verify(logits, tokens, parents, cfg):
    """Verifier outputs with the unused tail of ``tokens`` / ``contexts`` (beyond the emitted count, left
    unwritten by the kernel) set to -1 so that whole tensors can be compared."""
    out = _verify_raw(logits, tokens, parents, cfg)
    live = torch.arange(out["tokens"].shape[1], device=DEV)[None, :] < out["counts"][:, :1]
    out["tokens"] = torch.where(live, out["tokens"], torch.full_like(out["tokens"], -1))
    out["contexts"] = torch.where(live, out["contexts"], torch.full_like(out["contexts"], -1))
    return out


def _verify_raw(logits, tokens, parents, cfg):
    out = ops.tree_verify(logits, torch.tensor(tokens, dtype=torch.int32, device=DEV),
                          torch.tensor(parents, dtype=torch.int32, device=DEV), verify_method="lossy",
                          threshold_method="entropy", threshold=cfg["threshold"], window_size=cfg["window_size"])
    torch.cuda.synchronize()
    return out


def test_verify_full_batch_properties():
    print("full-size verify: 32 x 64 x 152064 bf16", flush=True)
    cfg = W.lossy_config(seed=0, batch=32, device=DEV)
    full = _verify(cfg["logits"], cfg["tokens"], cfg["parents"], cfg)
    again = _verify(cfg["logits"], cfg["tokens"], cfg["parents"], cfg)
    for k in KEYS + ("entropy",):
        assert torch.equal(full[k], again[k]), k                         # deterministic
    counts = full["counts"].cpu()
    assert int(counts[:, 3].abs().sum()) == 0
    for b in range(32):                                                  # planted flavours
        if cfg["flavours"][b] == 0:
            assert counts[b, 1] == 8, (b, counts[b].tolist())
        if cfg["flavours"][b] == 4:
            assert counts[b, 1] == 0, (b, counts[b].tolist())
    assert counts[:, 0].tolist() == (counts[:, 1] + 1).tolist()          # accepted drafts + one bonus token
    for b in (0, 1, 2, 3, 4, 13, 31):                                    # batch independence, and the oracle on a sample
        alone = _verify(cfg["logits"][b:b + 1], cfg["tokens"][b:b + 1], cfg["parents"][b:b + 1], cfg)
        for k in KEYS:
            assert torch.equal(alone[k][0], full[k][b]), (b, k)
        if b < 5:
            exp = ov.verify_logits(cfg["logits"][b].cpu(), cfg["tokens"][b], cfg["parents"][b], verify_method="lossy",
                                   verify_kwargs=dict(threshold=cfg["threshold"], window_size=cfg["window_size"],
                                                      threshold_method="entropy"))
            n = int(counts[b, 0])
            got = (full["tokens"][b, :n].tolist(), full["contexts"][b, :n].tolist(), (int(counts[b, 2]), int(counts[b, 1])))
            assert got == exp, b
    perm = torch.randperm(32, generator=torch.Generator().manual_seed(5)).tolist()
    shuffled = _verify(cfg["logits"][perm], [cfg["tokens"][i] for i in perm], [cfg["parents"][i] for i in perm], cfg)
    for k in KEYS:
        assert torch.equal(shuffled[k], full[k][perm]), k


def test_sampling_verify_full_batch_properties():
    from oracle import sampling as osamp
    print("full-size sampling verify: 32 x 64 x 152064 bf16, T = 0.8", flush=True)
    cfg = W.lossy_config(seed=1, batch=32, device=DEV)
    tok = torch.tensor(cfg["tokens"], dtype=torch.int32, device=DEV)
    par = torch.tensor(cfg["parents"], dtype=torch.int32, device=DEV)
    T = 0.8

    def run(logits, tok, par, seed, offset):
        out = ops.tree_verify(logits, tok, par, verify_method="exact", do_sample=True, temperature=T, seed=seed,
                              offset=offset)
        torch.cuda.synchronize()
        return out

    full = run(cfg["logits"], tok, par, 17, 3)
    again = run(cfg["logits"], tok, par, 17, 3)
    other = run(cfg["logits"], tok, par, 17, 4)
    assert torch.equal(full["target"], again["target"]) and torch.equal(full["counts"], again["counts"])
    assert (full["target"] != other["target"]).float().mean().item() > 0.3
    counts = full["counts"].cpu()
    assert int(counts[:, 3].abs().sum()) == 0
    # every emitted token is the draw of its context node (exact verifier, skip_nodes = 0)
    for b in range(32):
        n = int(counts[b, 0])
        ctx = full["contexts"][b, :n]
        assert torch.equal(full["tokens"][b, :n], full["target"][b][ctx]), b
        assert n == int(counts[b, 1]) + 1
    # tree 0 alone occupies the same global rows 0..63: identical draws and walk
    alone = run(cfg["logits"][:1], tok[:1], par[:1], 17, 3)
    assert torch.equal(alone["target"][0], full["target"][0])
    assert torch.equal(alone["counts"][0], full["counts"][0])
    # the oracle on a sample of rows of trees 0 and 31 (global row = 64 * tree + row)
    for b, rows in ((0, [0, 1, 17, 63]), (31, [0, 5, 62])):
        lg = cfg["logits"][b][rows].cpu()
        for j, r in enumerate(rows):
            want, margin = osamp.draw_tokens(osamp.warp_probs(lg[j:j + 1], T), 17, 3, first_row=64 * b + r)
            assert int(full["target"][b, r]) == want[0] or margin[0] < 2.0 ** -6, (b, r)
    # distribution-level check over all 2048 draws: E[log p(draw)] = -H(row), both estimated in fp32
    lp_sum = ent_sum = 0.0
    for b in range(32):
        logp = torch.log_softmax((cfg["logits"][b].float() / T).to(torch.bfloat16).float(), -1)
        lp_sum += float(torch.gather(logp, 1, full["target"][b].unsqueeze(1)).sum())
        ent_sum += float(-(logp.exp() * logp).sum())
    mean_lp, mean_h = lp_sum / 2048, ent_sum / 2048
    print("mean log p(draw)", mean_lp, "mean entropy", mean_h, flush=True)
    assert abs(mean_lp + mean_h) < 0.05 * max(1.0, mean_h)


def test_topk_full_size_properties():
    print("full-size top-k: 2048 x 152064 bf16, k = 16", flush=True)
    R, V, k = 2048, 152064, 16
    g = torch.Generator(device=DEV).manual_seed(9)
    probs = torch.empty(R, 1, V, dtype=torch.bfloat16, device=DEV)
    for r0 in range(0, R, 64):
        z = torch.randn(64, 1, V, generator=g, device=DEV) * (torch.rand(64, 1, 1, generator=g, device=DEV) * 2.5 + 0.5)
        probs[r0:r0 + 64] = torch.softmax(z.to(torch.bfloat16), -1)
    parent = torch.rand(R, 1, generator=g, device=DEV).to(torch.bfloat16)
    tok, val, par = ops.topk_expand(probs, parent, k)
    tok2, val2, par2 = ops.topk_expand(probs, parent, k)
    torch.cuda.synchronize()
    assert torch.equal(tok, tok2) and torch.equal(val, val2) and torch.equal(par, par2)
    assert int(par.abs().sum()) == 0 and tok.shape == (R, k)
    buf = probs[:, 0] * parent                                            # [R, V], rounded to bf16 like the reference's buf
    assert torch.equal(val, torch.gather(buf, 1, tok))                    # each value is its element's product
    v32, t64 = val.float(), tok.to(torch.int64)
    assert bool((v32[:, :-1] >= v32[:, 1:]).all())                        # sorted by value ...
    tie = v32[:, :-1] == v32[:, 1:]
    assert bool((t64[:, :-1][tie] < t64[:, 1:][tie]).all())               # ... ties by ascending index
    kth = v32[:, -1:]
    b32 = buf.float()
    assert bool(((b32 > kth).sum(1) < k).all()) and bool(((b32 >= kth).sum(1) >= k).all())
    # a tie at the k-th value must have been resolved towards the lowest indices
    for r in torch.nonzero((b32 == kth).sum(1) > (v32 == kth).sum(1)).flatten().tolist()[:64]:
        cand = torch.nonzero(b32[r] == kth[r]).flatten()[: int((v32[r] == kth[r]).sum())]
        assert sorted(t64[r][v32[r] == kth[r, 0]].tolist()) == cand.tolist(), r
    assert torch.equal(val, torch.topk(buf, k, dim=-1).values)            # the library routine's values
