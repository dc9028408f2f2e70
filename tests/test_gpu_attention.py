"""GPU parity: tree-masked GQA attention through the C ABI against the fp32 oracle on the same
bf16 / fp16 inputs.  Tolerance (stated by the benchmark definition): 1e-2 relative; checked as
max |diff| <= 1e-2 * max |ref| per batch element plus an element-wise allclose."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import attention as oa
from subspec_amd import ops, workloads as W

DEV = "cuda:0"


def _case(seed, B, Hq, Hkv, n, P, S, dtype, depth=8):
    g = torch.Generator().manual_seed(seed)
    parents, _, _ = W.random_tree(g, n=n, max_depth=depth, max_children=4, vocab=1000, chain_depth=min(depth, n - 1))
    q = torch.randn(B, Hq, n, 128, generator=g).to(dtype)
    k = torch.randn(B, Hkv, S, 128, generator=g).to(dtype)
    v = torch.randn(B, Hkv, S, 128, generator=g).to(dtype)
    return parents, q, k, v


def _check(parents, q, k, v, P, tag):
    print("attention", tag, tuple(q.shape), tuple(k.shape), P, flush=True)
    anc = ops.ancestor_bits_tensor(parents, device=DEV)
    out = ops.tree_attention(q.to(DEV), k.to(DEV), v.to(DEV), anc, P)
    torch.cuda.synchronize()
    ref = oa.tree_attention(q, k, v, parents, P)
    got = out.float().cpu()
    assert got.shape == ref.shape
    err = (got - ref).abs().amax().item()
    assert err <= 1e-2 * ref.abs().amax().item(), (tag, err, ref.abs().amax().item())
    assert torch.allclose(got, ref, rtol=1e-2, atol=2e-2), tag


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_small_shapes(dtype):
    for seed, (B, Hq, Hkv, n, P, S) in enumerate([(1, 4, 2, 9, 0, 16), (2, 7, 1, 17, 5, 64), (1, 28, 4, 64, 100, 200),
                                                  (3, 8, 8, 33, 63, 128), (1, 14, 2, 1, 300, 301), (2, 4, 4, 64, 64, 128),
                                                  # more heads per KV head than one workgroup takes, few rows
                                                  (1, 16, 1, 8, 40, 64), (1, 12, 1, 24, 10, 64), (2, 20, 2, 16, 130, 160)]):
        parents, q, k, v = _case(seed, B, Hq, Hkv, n, P, S, dtype, depth=6)
        _check(parents, q, k, v, P, f"small{seed}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_many_sequence_head_pairs(dtype):
    """Windows of 17 to 64 rows with at least 128 (sequence, head) pairs take the kernel whose wavefronts alternate between
    matrix and softmax phases and whose K / V blocks are copied straight into LDS: one, two, three and many 64-key blocks
    per workgroup, one and several key chunks, prefixes that are no multiple of 64 (or empty), ragged last row tiles,
    GQA groups of 1, 4, 7, 8 and 32 heads (workgroups with idle head slots), 17 to 32 rows (a wavefront is a whole head)."""
    shapes = [(8, 16, 2, 64, 100, 200), (5, 28, 4, 40, 1000, 1100), (16, 8, 8, 33, 63, 128), (4, 32, 4, 20, 500, 600),
              (3, 64, 8, 64, 0, 64), (2, 64, 2, 64, 4000, 4200), (32, 4, 1, 17, 7, 40), (6, 28, 4, 64, 1, 70),
              (19, 7, 1, 48, 130, 200), (2, 64, 4, 32, 2500, 2560)]
    for seed, (B, Hq, Hkv, n, P, S) in enumerate(shapes):
        parents, q, k, v = _case(300 + seed, B, Hq, Hkv, n, P, S, dtype, depth=7)
        k[:, :, P + n:] = 1e3                                          # stale rows beyond the tree must not be read
        v[:, :, P + n:] = -1e3
        _check(parents, q, k, v, P, f"pairs{seed}")


def test_many_pairs_peaked_rows():
    """Rows whose maximum moves late and far (a key far above everything before it, in the last chunk): the reference exponent
    of such a row is raised after many blocks, and everything accumulated until then is rescaled."""
    g = torch.Generator().manual_seed(77)
    B, Hq, Hkv, n, P, S = 8, 16, 2, 64, 2048, 2112
    parents, q, k, v = _case(77, B, Hq, Hkv, n, P, S, torch.bfloat16)
    k[:, :, 1900] = 6 * q[:, ::8, 5]                                   # row 5 of every eighth head finds a near-copy of itself
    k[:, :, 3] = -4 * q[:, ::8, 9]
    q[:, :, 11] *= 30                                                  # scores of a few hundred for one row
    q[:, :, 12] *= 0.0                                                 # and a row that is all ties
    _check(parents, q, k, v, P, "peaked")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_many_pairs_large_trees(dtype):
    """Trees beyond 64 slots (two and more mask words per row) with many (sequence, head) pairs: every window of 64 rows."""
    for seed, (B, n_slots, P, S, depth) in enumerate([(16, 128, 70, 256, 16), (16, 289, 200, 512, 48), (20, 100, 0, 128, 12)]):
        g = torch.Generator().manual_seed(500 + seed)
        parents, _, _ = W.random_tree(g, n=n_slots, max_depth=depth, max_children=6, vocab=1000, chain_depth=depth)
        q = torch.randn(B, 8, n_slots, 128, generator=g).to(dtype)
        k = torch.randn(B, 2, S, 128, generator=g).to(dtype)
        v = torch.randn(B, 2, S, 128, generator=g).to(dtype)
        k[:, :, P + n_slots:] = 1e3
        print("attention many pairs, large tree", dtype, B, n_slots, P, flush=True)
        ref = oa.tree_attention(q, k, v, parents, P)
        anc = ops.ancestor_bits_tensor(parents, device=DEV)
        out = ops.tree_attention(q.to(DEV), k.to(DEV), v.to(DEV), anc, P).float().cpu()
        assert (out - ref).abs().amax().item() <= 1e-2 * ref.abs().amax().item()
        assert torch.allclose(out, ref, rtol=1e-2, atol=2e-2)


@pytest.mark.parametrize("B", [1, 8])
def test_config3_qwen_geometry(B):
    parents, q, k, v = _case(100 + B, B, 28, 4, 64, 4096, 4160, torch.bfloat16)
    _check(parents, q, k, v, 4096, f"cfg3-B{B}")


def test_stale_cache_tail_and_per_batch_trees():
    # the static cache is longer than prefix + n and holds garbage beyond: it must not be read into the result
    parents, q, k, v = _case(7, 2, 28, 4, 40, 1000, 2113, torch.bfloat16)
    k[:, :, 1040:] = 1e3
    v[:, :, 1040:] = -1e3
    _check(parents, q, k, v, 1000, "stale-tail")
    # different tree per batch element
    g = torch.Generator().manual_seed(5)
    p2, _, _ = W.random_tree(g, n=40, max_depth=5, max_children=4, vocab=1000)
    anc = torch.stack([ops.ancestor_bits_tensor(parents), ops.ancestor_bits_tensor(p2)]).to(DEV)
    out = ops.tree_attention(q.to(DEV), k.to(DEV), v.to(DEV), anc, 1000).float().cpu()
    ref = torch.cat([oa.tree_attention(q[:1], k[:1], v[:1], parents, 1000), oa.tree_attention(q[1:], k[1:], v[1:], p2, 1000)])
    assert torch.allclose(out, ref, rtol=1e-2, atol=2e-2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_extended_tree_up_to_128_slots(dtype):
    """A tree grown during the target forward occupies up to 128 slots (two mask words per row); the
    query rows are a window of at most 64 of its nodes."""
    for seed, (B, n_slots, P, S) in enumerate([(1, 128, 70, 256), (2, 100, 1000, 1200), (1, 65, 0, 80)]):
        g = torch.Generator().manual_seed(40 + seed)
        parents, _, _ = W.random_tree(g, n=n_slots, max_depth=16, max_children=4, vocab=1000, chain_depth=16)
        q = torch.randn(B, 8, n_slots, 128, generator=g).to(dtype)
        k = torch.randn(B, 2, S, 128, generator=g).to(dtype)
        v = torch.randn(B, 2, S, 128, generator=g).to(dtype)
        k[:, :, P + n_slots:] = 1e3                                   # stale rows beyond the tree
        ref = oa.tree_attention(q, k, v, parents, P)                   # all n_slots rows
        anc = ops.ancestor_bits_tensor(parents, device=DEV)
        assert anc.shape == (n_slots, 2)
        for lo, hi in ((0, 64), (n_slots - 40, n_slots), (60, 70)):
            print("attention 128-slot", dtype, B, n_slots, P, lo, hi, flush=True)
            out = ops.tree_attention(q[:, :, lo:hi].contiguous().to(DEV), k.to(DEV), v.to(DEV), anc[lo:hi].contiguous(), P,
                                     n_tree_slots=n_slots).float().cpu()
            want = ref[:, lo:hi]
            assert (out - want).abs().amax().item() <= 1e-2 * want.abs().amax().item()
            assert torch.allclose(out, want, rtol=1e-2, atol=2e-2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_large_trees_up_to_512_slots(dtype):
    """Trees of the reference's offloading configurations (1 + 48 * 6 = 289 nodes) and the largest the masks describe
    (512 slots, eight words per row): all rows in one call (windows of 64 rows inside), and windows of few rows
    as a draft step or a post-speculation window queries them.  Prefixes that are and are not multiples of 64, so
    that a 64-key block straddles two mask words."""
    for seed, (B, n_slots, P, S, depth) in enumerate([(1, 289, 70, 400, 48), (2, 512, 1000, 1600, 60), (1, 200, 0, 256, 30),
                                                      (1, 130, 64, 320, 20)]):
        g = torch.Generator().manual_seed(90 + seed)
        parents, _, _ = W.random_tree(g, n=n_slots, max_depth=depth, max_children=6, vocab=1000, chain_depth=depth)
        q = torch.randn(B, 8, n_slots, 128, generator=g).to(dtype)
        k = torch.randn(B, 2, S, 128, generator=g).to(dtype)
        v = torch.randn(B, 2, S, 128, generator=g).to(dtype)
        k[:, :, P + n_slots:] = 1e3                                   # stale rows beyond the tree
        ref = oa.tree_attention(q, k, v, parents, P)
        anc = ops.ancestor_bits_tensor(parents, device=DEV)
        assert anc.shape == (n_slots, (n_slots + 63) // 64)
        print("attention large tree", dtype, B, n_slots, P, "all rows", flush=True)
        out = ops.tree_attention(q.to(DEV), k.to(DEV), v.to(DEV), anc, P).float().cpu()
        assert (out - ref).abs().amax().item() <= 1e-2 * ref.abs().amax().item()
        assert torch.allclose(out, ref, rtol=1e-2, atol=2e-2)
        for lo, hi in ((n_slots - 6, n_slots), (100, 164), (n_slots - 70, n_slots - 3)):
            print("attention large tree", dtype, B, n_slots, P, lo, hi, flush=True)
            out = ops.tree_attention(q[:, :, lo:hi].contiguous().to(DEV), k.to(DEV), v.to(DEV), anc[lo:hi].contiguous(), P,
                                     n_tree_slots=n_slots).float().cpu()
            want = ref[:, lo:hi]
            assert (out - want).abs().amax().item() <= 1e-2 * want.abs().amax().item()
            assert torch.allclose(out, want, rtol=1e-2, atol=2e-2)
    with pytest.raises(ValueError):
        ops.ancestor_bits_tensor([-1] + list(range(512)))              # 513 nodes


def test_argument_errors():
    q = torch.zeros(1, 4, 8, 128, dtype=torch.bfloat16, device=DEV)
    k = torch.zeros(1, 2, 64, 128, dtype=torch.bfloat16, device=DEV)
    anc = torch.zeros(8, dtype=torch.int64, device=DEV)
    with pytest.raises(ValueError):
        ops.tree_attention(q, k, k, anc, 60)                       # prefix + n beyond the cache
    with pytest.raises(ValueError):
        ops.tree_attention(q.float(), k.float(), k.float(), anc, 8)   # fp32 not supported
    with pytest.raises(ValueError):
        ops.tree_attention(torch.zeros(1, 4, 65, 128, dtype=torch.bfloat16, device=DEV), k, k,
                           torch.zeros(65, dtype=torch.int64, device=DEV), 0)
    with pytest.raises(ValueError):
        ops.tree_attention(q[..., :64].contiguous(), k[..., :64].contiguous(), k[..., :64].contiguous(), anc, 8)
