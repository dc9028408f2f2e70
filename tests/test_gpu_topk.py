"""GPU parity: top-k draft-tree expansion through the C ABI against the oracle.
Bar: values, token ids and parent indices bit-exact under the canonical tie rule
(value descending, flat index ascending)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import topk as ot
from subspec_amd import ops

DEV = "cuda:0"


def _check(probs, parent, k):
    tok, val, par = ops.topk_expand(probs.to(DEV), parent.to(DEV), k)
    torch.cuda.synchronize()
    e_tok, e_val, e_par = ot.topk_expand(probs, parent, k)
    assert torch.equal(val.cpu(), e_val), (val.cpu(), e_val)
    assert torch.equal(tok.cpu(), e_tok)
    assert torch.equal(par.cpu(), e_par)
    return tok.cpu(), val.cpu(), par.cpu()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_small_shapes_ragged_vocab(dtype):
    g = torch.Generator().manual_seed(1)
    for B, L, V, k in ((1, 1, 9, 9), (2, 3, 17, 5), (3, 4, 1001, 16), (1, 8, 5000, 8), (2, 10, 32000, 10),
                       (4, 1, 40960, 64), (1, 6, 777, 6)):
        print("topk", dtype, B, L, V, k, flush=True)
        probs = torch.softmax(torch.randn(B, L, V, generator=g) * 3, -1).to(dtype)
        parent = torch.rand(B, L, generator=g).to(dtype)
        _check(probs, parent, k)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_heavy_ties_and_adversarial_order(dtype):
    V = 40000
    # fewer non-zero entries than k: the rest must be the lowest flat indices holding zero
    probs = torch.zeros(1, 3, V, dtype=dtype)
    probs[0, 1, 77] = 0.5
    probs[0, 2, 5] = 0.25
    parent = torch.tensor([[1.0, 0.5, 1.0]], dtype=dtype)
    tok, val, par = _check(probs, parent, 8)
    assert par.tolist()[0][:2] == [1, 2] or val.tolist()[0][0] == 0.25
    # constant rows: every element ties
    _check(torch.full((2, 2, V), 0.001, dtype=dtype), torch.ones(2, 2, dtype=dtype), 16)
    # ascending order: every new element beats the running threshold
    asc = (torch.arange(V, dtype=torch.float32) / V).to(dtype).view(1, 1, V)
    _check(asc, torch.ones(1, 1, dtype=dtype), 16)
    # descending order
    _check(asc.flip(-1).contiguous(), torch.ones(1, 1, dtype=dtype), 16)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("batch", [1, 24])
def test_rows_that_are_mostly_one_value(dtype, batch):
    """Rows in which most elements share one value, so the bound the kernel takes from its sample is that value and
    thousands of elements tie with it: the k best are whatever lies above, then the ties of lowest index."""
    g = torch.Generator().manual_seed(11)
    V, k = 152064, 16
    print("ties", dtype, batch, flush=True)
    base = torch.full((batch, 1, V), 1.0 / V)
    rows = []
    for b in range(batch):
        r = base[b, 0].clone()
        kind = b % 6
        if kind == 1:                                   # a handful above the plateau, fewer than k
            r[torch.randint(0, V, (5,), generator=g)] = 0.01
        elif kind == 2:                                 # more than k above it, late in the row
            r[V - 4000 + torch.randperm(3000, generator=g)[:40]] = torch.rand(40, generator=g) * 0.01 + 1e-4
        elif kind == 3:                                 # one-hot: the plateau is zero
            r.zero_()
            r[int(torch.randint(0, V, (1,), generator=g))] = 1.0
        elif kind == 4:                                 # plateau only in the first part, smaller values after it
            r[20000:] = 1e-7
        elif kind == 5:                                 # every thread's sample holds one larger value among ties
            r[::64] = 2.0 / V
        rows.append(r)
    probs = torch.stack(rows).view(batch, 1, V).to(dtype)
    parent = (torch.rand(batch, 1, generator=g) * 0.9 + 0.1).to(dtype)
    _check(probs, parent, k)
    # several leaves per tree: the flat index order across leaves decides among ties
    _check(probs[:1].expand(1, 4, V).contiguous(), torch.full((1, 4), 0.5, dtype=dtype), k)


def test_config2_rows_bf16_full_vocab():
    g = torch.Generator().manual_seed(2)
    V = 152064
    logits = (torch.randn(48, 1, V, generator=g) * (torch.rand(48, 1, 1, generator=g) * 2.5 + 0.5)).to(torch.bfloat16)
    probs = torch.softmax(logits, -1)
    parent = torch.rand(48, 1, generator=g).to(torch.bfloat16)
    tok, val, par = _check(probs, parent, 16)
    # same values as the reference's literal torch.topk call (its index order within ties is unspecified)
    t_tok, t_val, t_par = ot.topk_expand_torch(probs, parent, 16)
    assert torch.equal(val, t_val)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_draft_step_shape_full_vocab(dtype):
    # one draft step of the real pipeline: batch 1, k leaves, temperature-sharpened distribution
    g = torch.Generator().manual_seed(3)
    V = 152064
    probs = torch.softmax((torch.randn(1, 8, V, generator=g) * 2).to(dtype) / 0.2, -1)
    parent = torch.rand(1, 8, generator=g).to(dtype)
    _check(probs, parent, 8)
    root = torch.softmax((torch.randn(1, 1, V, generator=g) * 2).to(dtype) / 0.2, -1)
    _check(root, torch.ones(1, 1, dtype=dtype), 8)


def test_argument_errors():
    p = torch.rand(1, 1, 128, device=DEV)
    with pytest.raises(ValueError):
        ops.topk_expand(p, torch.ones(1, 2, device=DEV), 4)
    with pytest.raises(ValueError):
        ops.topk_expand(p, torch.ones(1, 1, device=DEV, dtype=torch.bfloat16), 4)
    with pytest.raises(ValueError):
        ops.topk_expand(p, torch.ones(1, 1, device=DEV), 100)       # k beyond the kernel's limit
    tok, val, par = ops.topk_expand(torch.rand(1, 1, 5, device=DEV), torch.ones(1, 1, device=DEV), 50)
    assert tok.shape == (1, 5)                                     # k clamps to the vocabulary


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_draft_probabilities_softmax_with_temperature(dtype):
    """softmax(logits / T) of a draft step against torch on the CPU.  Floating point: the two differ in
    the last place of exp and of the row sum, so values agree to one unit in the last place of the
    dtype (tolerance 2^-7 relative for bf16, 2^-10 for fp16, 1e-5 for fp32) and nearly all are equal."""
    g = torch.Generator().manual_seed(11)
    # few rows x several slices (two launches), one slice, and many rows (one workgroup per row)
    for rows, V, T in ((8, 152064, 0.2), (1, 152064, 1.0), (5, 1000, 0.7), (3, 77, 0.2), (3, 9001, 0.5), (300, 5000, 0.3)):
        print("softmax_temperature", dtype, rows, V, T, flush=True)
        logits = (torch.randn(rows, V, generator=g) * 3).to(dtype)
        logits[0, 3] = float("-inf")                                  # masked entry
        ref = ot.draft_probs(logits, T)
        got = ops.softmax_temperature(logits.to(DEV), T).cpu()
        assert got.dtype == dtype and got.shape == ref.shape
        rtol = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10, torch.float32: 1e-5}[dtype]
        atol = {torch.bfloat16: 2.0 ** -133, torch.float16: 2.0 ** -24, torch.float32: 1e-38}[dtype]   # one subnormal step
        assert torch.allclose(got.float(), ref.float(), rtol=rtol, atol=atol)
        assert (got == ref).float().mean().item() >= (0.98 if dtype != torch.float32 else 0.0)
        assert got[0, 3] == 0
        assert torch.allclose(got.float().sum(-1), torch.ones(rows), atol=2e-2)
        # the expansion on top of the device probabilities equals the oracle's on the same rows
        parent = torch.rand(1, rows, generator=g).to(dtype)
        tok, val, par = ops.topk_expand(got.reshape(1, rows, V).to(DEV), parent.to(DEV), 8)
        e_tok, e_val, e_par = ot.topk_expand(got.reshape(1, rows, V), parent, 8)
        assert torch.equal(tok.cpu(), e_tok) and torch.equal(val.cpu(), e_val) and torch.equal(par.cpu(), e_par)
    with pytest.raises(ValueError):
        ops.softmax_temperature(torch.zeros(2, 8, device=DEV), 0.0)
