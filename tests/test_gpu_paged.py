"""GPU: tree attention and KV compaction over the paged pool (through the C ABI).

Attention over pages runs the same arithmetic in the same order as over the contiguous cache, so the
two must agree bit for bit whatever the page size and page order; compaction is data movement and is
compared bit for bit with the oracle."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import attention as oa
from oracle import kv as okv
from subspec_amd import ops, workloads as W
from subspec_amd.paged_cache import KvCachePool, RequestKvCache

DEV = "cuda:0"


def _scatter(k, v, page_len, max_pages, perm):
    """Contiguous k, v [1, H, S, D] -> pool layer [max_pages, 2, page_len, H, D] with logical page i at perm[i]."""
    _, H, S, D = k.shape
    n_pages = (S + page_len - 1) // page_len
    layer = torch.randn(max_pages, 2, page_len, H, D, generator=torch.Generator().manual_seed(1)).to(k.dtype)   # junk elsewhere
    pad = n_pages * page_len - S
    kk = torch.cat([k[0].transpose(0, 1), torch.zeros(pad, H, D, dtype=k.dtype)]).view(n_pages, page_len, H, D)
    vv = torch.cat([v[0].transpose(0, 1), torch.zeros(pad, H, D, dtype=k.dtype)]).view(n_pages, page_len, H, D)
    pages = torch.tensor(perm[:n_pages])
    layer[pages, 0] = kk
    layer[pages, 1] = vv
    return layer, pages.to(torch.int32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("page_len,prefix,n", [(16, 100, 20), (8, 1000, 64), (64, 37, 9), (1, 70, 5), (16, 4096, 64), (256, 300, 33)])
def test_paged_attention_equals_contiguous(dtype, page_len, prefix, n):
    print("paged attention", dtype, page_len, prefix, n, flush=True)
    g = torch.Generator().manual_seed(page_len + prefix)
    Hq, Hkv, D = 8, 2, 128
    S = prefix + n
    q = torch.randn(1, Hq, n, D, generator=g).to(dtype)
    k = torch.randn(1, Hkv, S, D, generator=g).to(dtype)
    v = torch.randn(1, Hkv, S, D, generator=g).to(dtype)
    parents, _, _ = W.random_tree(g, n=n, max_depth=6, max_children=3, vocab=100, chain_depth=3)
    anc = ops.ancestor_bits_tensor(parents, device=DEV)
    n_pages = (S + page_len - 1) // page_len
    max_pages = n_pages + 7
    perm = torch.randperm(max_pages, generator=g).tolist()
    layer, pages = _scatter(k, v, page_len, max_pages, perm)
    want = ops.tree_attention(q.to(DEV), k.to(DEV), v.to(DEV), anc, prefix)
    got = ops.tree_attention_paged(q.to(DEV), layer.to(DEV), pages.to(DEV), anc, prefix)
    assert torch.equal(got, want)
    # gathering the pages back gives the contiguous tensors (pins the layout helper used above)
    kk, vv = okv.gather_paged(layer, pages, S)
    assert torch.equal(kk, k) and torch.equal(vv, v)
    if prefix <= 300:                                         # and the attention oracle on the small cases
        ref = oa.tree_attention(q.float(), k.float(), v.float(), parents, prefix)
        assert (got.float().cpu() - ref).abs().amax().item() <= 1e-2 * ref.abs().amax().item() + 1e-2


def test_paged_attention_argument_errors():
    q = torch.zeros(1, 4, 8, 128, dtype=torch.bfloat16, device=DEV)
    layer = torch.zeros(6, 2, 16, 2, 128, dtype=torch.bfloat16, device=DEV)
    anc = torch.ones(8, dtype=torch.int64, device=DEV)
    pages = torch.arange(3, dtype=torch.int32, device=DEV)
    ops.tree_attention_paged(q, layer, pages, anc, 30)                         # 38 rows fit 3 pages of 16
    with pytest.raises(ValueError):
        ops.tree_attention_paged(q, layer, pages, anc, 45)                     # 53 rows do not
    with pytest.raises(ValueError):
        ops.tree_attention_paged(q, layer, pages.long(), anc, 30)              # table must be int32
    with pytest.raises(ValueError):
        ops.tree_attention_paged(q, torch.zeros(6, 2, 12, 2, 128, dtype=torch.bfloat16, device=DEV), pages, anc, 10)   # page_len 12
    # a corrupt table is clamped into the pool instead of faulting
    bad = torch.tensor([0, 999999, -5], dtype=torch.int32, device=DEV)
    out = ops.tree_attention_paged(q, layer, bad, anc, 30)
    torch.cuda.synchronize()
    assert out.shape == (1, 8, 4 * 128)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("page_len", [4, 16, 64])
def test_paged_compaction_bit_exact(dtype, page_len):
    g = torch.Generator().manual_seed(page_len)
    L, H, D = 3, 4, 128
    for trial in range(4):
        offset = int(torch.randint(0, 200, (1,), generator=g))
        n = int(torch.randint(1, 65, (1,), generator=g))
        ctx = torch.sort(torch.randperm(64, generator=g)[:min(n, 64)]).values
        n_pages = (offset + 64 + page_len - 1) // page_len
        max_pages = n_pages + 5
        pool = torch.randn(L, max_pages, 2, page_len, H, D, generator=g).to(dtype)
        perm = torch.randperm(max_pages, generator=g)[:n_pages].to(torch.int32)
        print("paged compaction", dtype, page_len, offset, ctx.numel(), flush=True)
        want = okv.compact_paged(pool, perm, ctx.tolist(), offset)
        got = ops.kv_compact_paged_(pool.clone().to(DEV), perm.to(DEV), ctx.to(DEV), offset)
        assert torch.equal(got.cpu(), want)
        # the count may come from device memory: only the first `count` rows move
        cnt = max(1, ctx.numel() // 2)
        want = okv.compact_paged(pool, perm, ctx[:cnt].tolist(), offset)
        got = ops.kv_compact_paged_(pool.clone().to(DEV), perm.to(DEV), ctx.to(DEV), offset,
                                    count_dev=torch.tensor([cnt], dtype=torch.int32, device=DEV))
        assert torch.equal(got.cpu(), want)


def test_request_cache_cycle_matches_static_cache():
    """append -> tree attention -> reorder on a RequestKvCache equals the same steps on contiguous tensors."""
    g = torch.Generator().manual_seed(3)
    Hq, Hkv, D, page_len, prefix, n = 8, 2, 128, 16, 45, 12
    pool = KvCachePool(max_pages=16, num_layers=2, num_heads=Hkv, head_dim=D, page_len=page_len, dtype=torch.bfloat16, device=DEV)
    pool.allocate(3)                                          # the request does not start at page 0
    req = RequestKvCache(pool, page_len, seq_init_len=prefix)
    k = torch.randn(prefix + n, Hkv, D, generator=g).to(torch.bfloat16)
    v = torch.randn(prefix + n, Hkv, D, generator=g).to(torch.bfloat16)
    for layer in range(2):
        req.append(layer, k[:prefix].to(DEV), v[:prefix].to(DEV), first_row=0)
    parents, _, _ = W.random_tree(g, n=n, max_depth=5, max_children=3, vocab=50, chain_depth=3)
    anc = ops.ancestor_bits_tensor(parents, device=DEV)
    q = torch.randn(1, Hq, n, D, generator=g).to(torch.bfloat16).to(DEV)
    table = None
    for layer in range(2):
        table = req.append(layer, k[prefix:].to(DEV), v[prefix:].to(DEV))       # tree rows behind the prefix
    got = req.attention(1, q, anc, prefix, table=table)
    kc = k.transpose(0, 1).unsqueeze(0).contiguous().to(DEV)
    vc = v.transpose(0, 1).unsqueeze(0).contiguous().to(DEV)
    assert torch.equal(got, ops.tree_attention(q, kc, vc, anc, prefix))
    # accept a path: the reference's callers pass offset = sequence length including the tree root's token
    accepted = torch.tensor([0, 2, 5, 7])
    req.reorder_cache_with_offset(accepted, offset=prefix + 1, num_new_tokens=n)
    assert req.get_seq_length() == prefix + 4
    kk, vv = okv.gather_paged(pool.cache_data[0].cpu(), req.kv_page_indices, prefix + 4)
    want_k = okv.compact_static(kc.cpu(), accepted.tolist(), prefix)[:, :, :prefix + 4]
    want_v = okv.compact_static(vc.cpu(), accepted.tolist(), prefix)[:, :, :prefix + 4]
    assert torch.equal(kk, want_k) and torch.equal(vv, want_v)
    assert len(req.kv_page_indices) == (prefix + 4 + page_len - 1) // page_len


@pytest.mark.parametrize("depth,topk", [(5, 4), (20, 6)])          # 21-node trees; 121-node trees (two mask words, row windows)
@pytest.mark.parametrize("driver", ["v1", "v2"])
@pytest.mark.parametrize("native", [False, True])
def test_speculative_cycle_over_the_paged_cache_equals_the_static_cache(driver, depth, topk, native):
    """The whole cycle (prefill, draft levels, target window, verification, compaction) over a page pool whose pages
    were handed out in scrambled order, against the same models over the contiguous cache.  Both runs go the same way
    -- module by module, or through the one-call decoder layers, which write the rotated rows and read the keys
    through the page table --, so the cache layout is the only difference and tokens and cached K / V must agree bit
    for bit."""
    from subspec_amd.cache import create_kv_cache
    from subspec_amd.draft import SubSpecSDDraftModel
    from subspec_amd.generator import SubSpecSDGenerator
    from subspec_amd.generator_v2 import SubSpecSDGeneratorV2
    from subspec_amd.model import DecoderConfig, build_models, init_weights
    from subspec_amd.utils import DraftParams
    cfg = DecoderConfig(num_hidden_layers=3, hidden_size=256, num_attention_heads=2, num_key_value_heads=1,
                        head_dim=128, intermediate_size=512, vocab_size=2048)
    w = init_weights(cfg, 3, DEV)
    prompt = torch.randint(0, cfg.vocab_size, (1, 37), generator=torch.Generator().manual_seed(8)).to(DEV)
    runs = {}
    for impl in ("static", "paged"):
        kv = create_kv_cache(impl, max_cache_len=1024, config=cfg, device=DEV, dtype=torch.bfloat16)
        if impl == "paged":
            pool = kv.cache.pool
            held = pool.allocate(9)                               # scramble the order of the request's pages:
            pool.deallocate(held[::2])                            # gaps in what the pool hands out later, and the
            kv.cache.request.kv_page_indices.extend(reversed(pool.allocate(3)))   # first three logical pages backwards
        target, draft, _ = build_models(cfg, kv, device=DEV, weights=w)
        target.use_native_layers = draft.use_native_layers = native
        assert target.native_layers and draft.native_layers       # both layouts qualify for the one-call layers
        cls, extra = (SubSpecSDGenerator, {}) if driver == "v1" else (SubSpecSDGeneratorV2, dict(postspec_steps=2))
        gen = cls(target, None, SubSpecSDDraftModel(draft), DraftParams(temperature=0.2, max_depth=depth, topk_len=topk),
                  cache_implementation=impl, generator_kwargs=dict(verify_method="exact", **extra))
        out = gen.generate(prompt, max_new_tokens=40, do_sample=False, past_key_values=kv)[0].cpu()
        L = kv.get_seq_length()
        k, v = kv.cache.prefix_kv(1, L)
        runs[impl] = (out, L, k.cpu().clone(), v.cpu().clone(), kv)
    (a, La, ka, va, _), (b, Lb, kb, vb, kvp) = runs["static"], runs["paged"]
    assert a.numel() == 77 and torch.equal(a, b) and La == Lb == 76
    assert torch.equal(ka, kb) and torch.equal(va, vb)
    table = kvp.cache.table().tolist()
    assert table != sorted(table)                                   # the pages really were out of order
    # rows leave the cache: whole pages go back to the pool
    free = int(kvp.cache.pool.num_free_pages())
    kvp.cache.crop(20)
    assert int(kvp.cache.pool.num_free_pages()) == free + (len(table) - 2) and kvp.cache.table().tolist() == table[:2]
    with pytest.raises(ValueError):
        kvp.cache.ensure(100000)
