"""GPU: the benchmark workload at its FULL size (32 trees x 64 nodes x 152064 bf16 logits, top-16 of
2048 x 152064 bf16 rows), checked through properties that do not need the CPU oracle at that size:

  * batch independence: a tree verified inside the 32-tree batch gives exactly what it gives alone,
    and a sample of trees equals the oracle;
  * determinism: a second launch is bit-identical;
  * permutation: reordering the trees reorders the outputs;
  * planted flavours: trees built with an all-exact depth-8 path accept all 8 draft tokens, trees
    with nothing planted accept none;
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
