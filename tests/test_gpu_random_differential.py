"""GPU: seeded random differential run of the verifier, the top-k expansion and the linear kernels against the oracle.

Shapes, dtypes, tree forms and parameters are drawn at random (fixed seeds): trees of 1 to 300 nodes, vocabularies
that are and are not multiples of the vector width, peaked / masked / heavily tied rows, an EOS token that may sit
on the accepted path, exact and lossy verification with both gates, and windows of a larger tree (``skip_nodes``,
a root inside the window, fewer scored rows than nodes) as the post-speculating driver verifies them.  Every case
must reproduce the oracle's tokens, contexts and lengths exactly."""
import random

import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import topk as ot
from oracle import verify as ov
from subspec_amd import ops, workloads as W

DEV = "cuda:0"


def _case(seed, long_rows=False):
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    if long_rows:
        # few rows of a long vocabulary: the verifier cuts such rows into slices (and, without the entropy gate,
        # looks for ties of the rounded probabilities in the acceptance kernel instead of a separate pass)
        n = rng.choice([1, 2, 5, 9, 17, 33, 64, 65, 100])
        vocab = rng.choice([16384, 32000, 40000, 50257, 65536, 152064])
    else:
        n = rng.choice([1, 2, 5, 17, 33, 64, 65, 100, 130, 257, 300])
        vocab = rng.choice([7, 64, 100, 1000, 4096, 5000, 8191, 8192, 32000, 50257])
    dtype = rng.choice([torch.bfloat16, torch.float16, torch.float32])
    depth = rng.choice([2, 4, 8, 16])
    ch = min(rng.choice([2, 4, 8]), vocab - 1)
    while sum(ch ** d for d in range(depth + 1)) < n:
        depth += 1
    parents, toks, depths = W.random_tree(g, n=n, max_depth=depth, max_children=ch, vocab=vocab,
                                          chain_depth=rng.choice([0, min(depth, n - 1)]))
    kids = ov.children_from_parents(parents)
    skip, root, rows = 0, 0, n
    if depths[-1] >= 2 and rng.random() < 0.3:
        # a window of the tree, as after post-speculation: the levels up to d1 were verified before (skip_nodes), the
        # root is a node behind them, and the levels beyond d2 were added after the forward and have no scored row
        upto = [sum(1 for d in depths if d <= lv) for lv in range(depths[-1] + 1)]     # level order: nodes of depth <= lv
        d1 = rng.randrange(0, depths[-1])
        skip = upto[d1]
        root = rng.randrange(skip, n)
        # the reference walks from the root without asking whether its children were scored (tree_verify.py:71-75), so a
        # window always reaches at least one level below the root
        d2 = rng.randrange(min(depths[root] + 1, depths[-1]), depths[-1] + 1)
        rows = upto[d2] - skip
    logits = torch.randn(rows, vocab, generator=g) * rng.choice([0.3, 1.0, 3.0])
    mode = rng.choice(["plain", "peaked", "masked", "ties"])
    for r in range(rows):
        node = r + skip
        if mode == "peaked" or (kids[node] and rng.random() < 0.6):
            j = toks[rng.choice(kids[node])] if kids[node] and rng.random() < 0.8 else rng.randrange(vocab)
            logits[r, j] += rng.choice([4.0, 8.0, 15.0])
        if mode == "masked":
            m = torch.rand(vocab, generator=g) < 0.9
            m[rng.randrange(vocab)] = False
            logits[r, m] = float("-inf")
    logits = logits.to(dtype)
    if mode == "ties":
        logits = (logits.float() * 4).round().div(4).to(dtype)          # many exactly equal logits
    method = rng.choice(["exact", "lossy"])
    vk = {}
    if method == "lossy":
        vk = {"threshold_method": rng.choice(["prob", "entropy"]), "threshold": rng.choice([0.0, 0.05, 0.3, 0.7, 1.5]),
              "window_size": rng.choice([0, 1, 2, 6])}
    eos = rng.choice([None, None, toks[rng.randrange(n)]])
    L = rng.choice([1, 2, 6, 8])
    k = min(rng.choice([1, 4, 8, 16, 64]), vocab)
    probs = torch.softmax(torch.randn(1, L, vocab, generator=g) * rng.choice([0.5, 2.0, 6.0]), -1)
    if mode == "ties":
        probs = (probs * 64).round() / 64
    return dict(n=n, vocab=vocab, dtype=dtype, parents=parents, toks=toks, skip=skip, root=root, logits=logits, mode=mode,
                method=method, vk=vk, eos=eos, probs=probs.to(dtype), parent_probs=torch.rand(1, L, generator=g).to(dtype), k=k)


@pytest.mark.parametrize("block", range(5))
def test_random_cases_match_the_oracle(block):
    for i in range(100 if block < 4 else 60):
        seed = 7_000_000 + block * 100 + i
        c = _case(seed, long_rows=block == 4)
        tag = (seed, c["n"], c["vocab"], c["dtype"], c["mode"], c["method"], c["vk"], c["eos"], c["skip"], c["root"],
               tuple(c["logits"].shape))
        if i % 20 == 0:
            print("random case", tag, flush=True)
        vk = c["vk"]
        out = ops.tree_verify(c["logits"].to(DEV), torch.tensor(c["toks"], dtype=torch.int32, device=DEV),
                              torch.tensor(c["parents"], dtype=torch.int32, device=DEV), root=c["root"],
                              skip_nodes=c["skip"], verify_method=c["method"], exact_entropy=True,
                              threshold_method=vk.get("threshold_method", "prob"), threshold=vk.get("threshold", 0.0),
                              window_size=vk.get("window_size", 1), eos_token_id=c["eos"])
        emitted, accept, total, status = out["counts"][0].tolist()
        got = (out["tokens"][0, :emitted].tolist(), out["contexts"][0, :emitted].tolist(), (total, accept))
        want = ov.verify_logits(c["logits"], c["toks"], c["parents"], root=c["root"], eos_token_id=c["eos"],
                                skip_nodes=c["skip"], verify_method=c["method"], verify_kwargs=vk)
        assert status == 0 and got == (want[0], want[1], want[2]), tag
        t, v, p = ops.topk_expand(c["probs"].to(DEV), c["parent_probs"].to(DEV), c["k"])
        et, ev, ep = ot.topk_expand(c["probs"], c["parent_probs"], c["k"])
        assert torch.equal(t.cpu(), et) and torch.equal(v.cpu().float(), ev.float()) and torch.equal(p.cpu(), ep), tag


@pytest.mark.parametrize("block", range(2))
def test_random_attention_and_compaction_cases(block):
    """Tree attention over random head groupings, prefixes, tree sizes (up to 512 slots) and row windows against the
    fp32 oracle (1e-2 relative, as the benchmark definition states), contiguous and paged; KV compaction of random
    ascending contexts bit for bit."""
    from oracle import attention as oa
    from oracle import kv as okv
    for i in range(30):
        seed = 8_000_000 + block * 100 + i
        rng = random.Random(seed)
        g = torch.Generator().manual_seed(seed)
        dtype = rng.choice([torch.bfloat16, torch.float16])
        Hkv = rng.choice([1, 2, 4])
        Hq = Hkv * rng.choice([1, 2, 7, 8])
        B = rng.choice([1, 1, 2])
        n_slots = rng.choice([1, 3, 17, 64, 65, 128, 129, 200, 300, 512])
        P = rng.choice([0, 1, 63, 64, 65, 200, 777])
        S = P + n_slots + rng.choice([0, 5, 100])
        depth = rng.choice([3, 8, 40])
        ch = rng.choice([2, 4, 6])
        while sum(ch ** d for d in range(depth + 1)) < n_slots:
            depth += 1
        parents, _, _ = W.random_tree(g, n=n_slots, max_depth=depth, max_children=ch, vocab=1000,
                                      chain_depth=min(depth, n_slots - 1))
        q = torch.randn(B, Hq, n_slots, 128, generator=g).to(dtype)
        k = torch.randn(B, Hkv, S, 128, generator=g).to(dtype)
        v = torch.randn(B, Hkv, S, 128, generator=g).to(dtype)
        k[:, :, P + n_slots:] = 1e3                                   # stale rows beyond the tree must not be read
        lo = rng.randrange(0, n_slots)
        hi = rng.randrange(lo + 1, n_slots + 1)
        tag = (seed, dtype, B, Hq, Hkv, n_slots, P, S, lo, hi)
        if i % 10 == 0:
            print("random attention", tag, flush=True)
        ref = oa.tree_attention(q, k, v, parents, P)[:, lo:hi]
        anc = ops.ancestor_bits_tensor(parents, device=DEV)
        out = ops.tree_attention(q[:, :, lo:hi].contiguous().to(DEV), k.to(DEV), v.to(DEV), anc[lo:hi].contiguous(), P,
                                 n_tree_slots=n_slots).float().cpu()
        assert (out - ref).abs().amax().item() <= 1e-2 * ref.abs().amax().item(), tag
        assert torch.allclose(out, ref, rtol=1e-2, atol=2e-2), tag
        # compaction: ascending contexts of random length behind a random offset
        L, H2, seq = rng.choice([1, 3]), rng.choice([1, 2]), rng.choice([70, 300, 700])
        cache = torch.randn(L, 2, 1, H2, seq, 128, generator=g).to(dtype)
        offset = rng.randrange(0, seq - 1)
        count = rng.randrange(1, min(512, seq - offset) + 1)
        ctx = sorted(torch.randperm(seq - offset, generator=g)[:count].tolist())
        dev = cache.to(DEV)
        ops.kv_compact_(dev, torch.tensor(ctx, dtype=torch.int64, device=DEV), offset)
        assert torch.equal(dev.cpu(), okv.compact_static(cache, ctx, offset)), (tag, offset, count)


@pytest.mark.parametrize("block", range(2))
def test_random_linear_shapes_match_the_oracle(block):
    """int4 g64 and dense projections (and the gate|up pair kernels with the SwiGLU stage) at random N, K, M: K from
    one to 40 groups of 64 (every count of pipeline steps per wavefront, odd and even, shorter than the prefetch
    distance and longer than one unrolled trip), 1 to 200 rows (one tile to several passes of 64)."""
    from oracle import int4 as oi
    from subspec_amd import quant
    for case in range(20):
        seed = 881000 + 100 * block + case
        rng = random.Random(seed)
        g = torch.Generator().manual_seed(seed)
        dtype = rng.choice([torch.bfloat16, torch.float16])
        N = 32 * rng.randrange(1, 48)
        K = 64 * rng.randrange(1, 41)
        M = rng.choice([1, 2, 7, 8, 16, 17, 32, 33, 64, 65, 200])
        w = torch.randn(N, K, generator=g) * 0.02
        x = torch.randn(M, K, generator=g).to(dtype)
        b = (torch.randn(N, generator=g) * 0.1).to(dtype) if rng.random() < 0.5 else None
        bd = None if b is None else b.to(DEV)
        codes, scale, zero = quant.quantize_int4_g64(w)
        wq, sz = quant.pack_tiled(codes, scale, zero)
        tag = (seed, dtype, N, K, M, b is not None)

        def silu_pairs(proj):                                    # float reference of the pair kernels' output
            gate, up = proj[:, :N // 2].double(), proj[:, N // 2:].double()
            return (gate / (1 + torch.exp(-gate)) * up).float()

        def close(got, want):                                    # the fixed-shape tests hold the last-place checks
            return (got - want).abs().amax().item() <= 1e-2 * max(want.abs().amax().item(), 1e-6)

        want = oi.linear(x, codes, scale, zero, b)
        assert close(ops.int4_linear(x.to(DEV), wq.to(DEV), sz.to(DEV), N, bd).float().cpu(), want), tag
        if M <= 64:
            assert close(ops.int4_gate_up_silu(x.to(DEV), wq.to(DEV), sz.to(DEV), N // 2, bd).float().cpu(), silu_pairs(want)), tag
            wd = w.to(dtype)
            want = x.float() @ wd.float().T + (0 if b is None else b.float())
            assert close(ops.dense_linear(x.to(DEV), wd.to(DEV), bd).float().cpu(), want), tag
            assert close(ops.dense_gate_up_silu(x.to(DEV), wd.to(DEV), bd).float().cpu(), silu_pairs(want)), tag
