"""The allocation-free entry point subspec_tree_verify_static (scratch array built into the library) against
subspec_tree_verify (caller's workspace), through the C ABI: same inputs, bit-identical outputs, on two calls in a
row, the second with a smaller input, so that what the first call left in the shared array is shown not to matter.
Collected last (the file name sorts behind every other test file)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from subspec_amd import _lib as L
from subspec_amd import ops, workloads as W

DEV = "cuda:0"
KEYS = ("tokens", "contexts", "counts", "target", "entropy", "child_prob")


def _pair(cfg, **kw):
    logits = cfg["logits"].to(DEV)
    if logits.dim() == 2:
        logits = logits.unsqueeze(0)
    tokens = torch.tensor(cfg["tokens"], dtype=torch.int32, device=DEV).reshape(logits.shape[0], -1)
    parents = torch.tensor(cfg["parents"], dtype=torch.int32, device=DEV).reshape(logits.shape[0], -1)
    ref = ops.tree_verify(logits, tokens, parents, **kw)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(DEV)
    out = {k: torch.empty_like(v) for k, v in ref.items()}
    held = torch.cuda.memory_allocated(DEV)
    if not _pair.warm:                                               # the first call on the device looks up the array's address
        ops.tree_verify(logits, tokens, parents, static_scratch=True, out=out, **kw)
        torch.cuda.synchronize()
        _pair.warm = True
    free_before = torch.cuda.mem_get_info(DEV)[0]                    # the driver's view: sees a hipMalloc made inside the library
    got = ops.tree_verify(logits, tokens, parents, static_scratch=True, out=out, **kw)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(DEV) == held >= before       # torch allocated nothing during the call
    assert torch.cuda.mem_get_info(DEV)[0] == free_before            # and neither did the library
    return ref, got


_pair.warm = False


def _same(ref, got, tag):
    for b in range(ref["counts"].shape[0]):
        emitted = int(ref["counts"][b, 0])
        assert ref["counts"][b].tolist() == got["counts"][b].tolist(), (tag, b)
        assert int(ref["counts"][b, 3]) == 0
        for k in ("tokens", "contexts"):
            assert torch.equal(ref[k][b, :emitted], got[k][b, :emitted]), (tag, k, b)
    for k in ("target", "entropy", "child_prob"):
        # same kernels on the same inputs: bit-identical, not merely close (compare the bit patterns so that a NaN
        # would not hide a difference)
        a, g = ref[k].contiguous(), got[k].contiguous()
        assert torch.equal(a.view(torch.int32) if a.dtype == torch.float32 else a,
                           g.view(torch.int32) if g.dtype == torch.float32 else g), (tag, k)


def test_static_scratch_equals_workspace_on_two_calls_in_a_row():
    lossy = dict(verify_method="lossy", threshold_method="entropy", threshold=0.3, window_size=6)
    big = W.lossy_config(seed=3, batch=6, n=64, vocab=32768)
    print("no-alloc verify: 6 x 64 x 32768 bf16 lossy", flush=True)
    _same(*_pair(big, **lossy), "big")
    small = W.lossy_config(seed=4, batch=2, n=24, vocab=4096 + 24)
    print("no-alloc verify: 2 x 24 x 4120 bf16 lossy (smaller, ragged vocabulary)", flush=True)
    _same(*_pair(small, **lossy), "small")
    greedy = W.greedy_config(seed=5, n=33, vocab=50257)
    print("no-alloc verify: 33 x 50257 fp32 exact", flush=True)
    _same(*_pair(greedy, verify_method="exact"), "greedy")
    # few rows of a long vocabulary with the entropy gate: the rows are cut into slices and the exact pass (a launch of
    # its own, with its own records in the built-in array) runs on the rows near the threshold
    sliced = W.lossy_config(seed=6, batch=1, n=24, vocab=65536)
    print("no-alloc verify: 1 x 24 x 65536 bf16 lossy, sliced rows, every entropy exact", flush=True)
    _same(*_pair(sliced, exact_entropy=True, **lossy), "sliced")


def test_static_scratch_rejects_more_rows_than_it_holds():
    rows = L.TREE_VERIFY_STATIC_MAX_ROWS // 8 + 1
    logits = torch.zeros((8, rows, 8), dtype=torch.bfloat16, device=DEV)
    tree = torch.zeros((8, rows), dtype=torch.int32, device=DEV)
    with pytest.raises(ValueError, match="scratch"):
        ops.tree_verify(logits, tree, tree, static_scratch=True)
