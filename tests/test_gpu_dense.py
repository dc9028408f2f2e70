"""GPU: the dense 16-bit linear for the rows of a tree (1 to 384) and the target's one-call decoder layer (through the C ABI).

Bar (floating point): fp32 accumulation in a different order than the reference product, one rounding
to the activation dtype: |y - ref| <= 2^-7 |ref| + 1e-2 of the output scale for bf16 (2^-10 for
fp16) against a float64 product of the same 16-bit operands, and nearly all values equal to the
correctly rounded result."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import decoder as od
from subspec_amd import ops, workloads as W
from subspec_amd.cache import create_kv_cache
from subspec_amd.model import DecoderConfig, build_models

DEV = "cuda:0"
CFG = DecoderConfig(num_hidden_layers=3, hidden_size=256, num_attention_heads=2, num_key_value_heads=1,
                    head_dim=128, intermediate_size=512, vocab_size=2048)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("N,K", [(16, 64), (256, 256), (4608, 3584), (3584, 18944), (37888, 3584), (1040, 448),
                                 (32, 64), (96, 128), (1056, 448)])
def test_dense_linear_matches_float64_product(dtype, N, K):
    g = torch.Generator().manual_seed(N + K)
    w = (torch.randn(N, K, generator=g) * 0.05).to(dtype)
    bias = (torch.randn(N, generator=g) * 0.1).to(dtype)
    wd = w.to(DEV)
    for M in (1, 5, 16, 17, 33, 64, 65, 130, 289, 384):
        if M > 64 and N % 32:                        # more than 64 rows: weight tiles of 32 rows
            continue
        print("dense_linear", dtype, N, K, M, flush=True)
        x = torch.randn(M, K, generator=g).to(dtype)
        for b in (None, bias):
            got = ops.dense_linear(x.to(DEV), wd, None if b is None else b.to(DEV)).cpu()
            ref = x.double() @ w.double().T + (0 if b is None else b.double())
            scale = ref.abs().amax().item()
            rel = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
            assert got.shape == (M, N) and got.dtype == dtype
            assert ((got.double() - ref).abs() <= rel * ref.abs() + 1e-3 * scale).all()
            assert (got == ref.to(dtype)).float().mean().item() >= 0.97
    # determinism: the reduction order is fixed
    x = torch.randn(64, K, generator=g).to(dtype).to(DEV)
    assert torch.equal(ops.dense_linear(x, wd, None), ops.dense_linear(x, wd, None))


def test_dense_linear_ragged_shapes_above_32_rows():
    """Row counts that leave row tiles partly empty, weight-tile counts that do not divide by the tiles of a workgroup,
    K of one to many chunks, with and without K ranges; bias and the SwiGLU pair kernel on the same shapes."""
    g = torch.Generator().manual_seed(77)
    for case in range(24):
        M = int(torch.randint(33, 385, (1,), generator=g))
        N = 32 * int(torch.randint(1, 80, (1,), generator=g))
        K = 64 * int(torch.randint(1, 40, (1,), generator=g))
        dtype = torch.bfloat16 if case % 3 else torch.float16
        print("dense_linear ragged", dtype, M, N, K, flush=True)
        w = (torch.randn(N, K, generator=g) * (1.0 / K ** 0.5)).to(dtype)
        x = torch.randn(M, K, generator=g).to(dtype)
        b = (torch.randn(N, generator=g) * 0.1).to(dtype)
        got = ops.dense_linear(x.to(DEV), w.to(DEV), b.to(DEV)).cpu()
        ref = x.double() @ w.double().T + b.double()
        rel = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
        assert ((got.double() - ref).abs() <= rel * ref.abs() + 1e-3 * ref.abs().amax().item()).all(), (M, N, K)
        assert (got == ref.to(dtype)).float().mean().item() >= 0.97, (M, N, K)
        if N % 64 == 0:
            F_ = N // 2
            act = ops.dense_gate_up_silu(x.to(DEV), w.to(DEV), b.to(DEV)).cpu()
            gate, up = got[:, :F_].float(), got[:, F_:].float()
            want = ((gate / (1 + torch.exp(-gate))).to(dtype).float() * up).to(dtype)
            # (the plain projection may have split K where the pair kernel does not: gate and up then differ in their
            # last place here and there)
            assert int((act != want).sum()) <= max(1, act.numel() // 100), (M, N, K)
            ulp = 2.0 ** (-7 if dtype == torch.bfloat16 else -10)
            assert ((act.float() - want.float()).abs() <= 4 * ulp * want.float().abs() + 1e-3 * want.float().abs().amax()).all(), (M, N, K)


def test_dense_linear_at_the_size_of_the_vocabulary_head():
    """152064 x 3584 (the draft's lm_head): 9504 tiles, two per workgroup; fp32 reference (its error is far below the
    bf16 rounding of the outputs)."""
    g = torch.Generator().manual_seed(152064)
    N, K = 152064, 3584
    w = (torch.randn(N, K, generator=g) * 0.03).to(torch.bfloat16)
    wd, wf = w.to(DEV), w.float()
    for M in (1, 8, 16):
        print("dense_linear head", M, flush=True)
        x = torch.randn(M, K, generator=g).to(torch.bfloat16)
        got = ops.dense_linear(x.to(DEV), wd, None).cpu()
        ref = x.float() @ wf.T
        scale = ref.abs().amax().item()
        assert got.shape == (M, N)
        assert ((got.float() - ref).abs() <= 2.0 ** -7 * ref.abs() + 1e-3 * scale).all()
        assert (got == ref.to(torch.bfloat16)).float().mean().item() >= 0.97


def test_dense_linear_special_cases():
    # integer-valued operands: every product and partial sum is exact, so the result is exact whatever the order
    g = torch.Generator().manual_seed(2)
    x = torch.randint(-4, 5, (37, 512), generator=g).to(torch.bfloat16)
    w = torch.randint(-3, 4, (96, 512), generator=g).to(torch.bfloat16)
    got = ops.dense_linear(x.to(DEV), w.to(DEV)).cpu()
    want = (x.double() @ w.double().T)
    assert torch.equal(got.double(), want.to(torch.bfloat16).double())
    # identity weight returns the activations
    eye = torch.eye(256, dtype=torch.bfloat16)
    x = torch.randn(9, 256, generator=g).to(torch.bfloat16)
    assert torch.equal(ops.dense_linear(x.to(DEV), eye.to(DEV)).cpu(), x)
    # leading dimensions are kept
    y = ops.dense_linear(torch.zeros(2, 3, 256, dtype=torch.bfloat16, device=DEV), eye.to(DEV))
    assert y.shape == (2, 3, 256)
    for bad in (dict(M=385, N=256, K=256), dict(M=4, N=250, K=256), dict(M=4, N=256, K=200), dict(M=65, N=48, K=256)):
        with pytest.raises(ValueError):
            ops.dense_linear(torch.zeros(bad["M"], bad["K"], dtype=torch.bfloat16, device=DEV),
                             torch.zeros(bad["N"], bad["K"], dtype=torch.bfloat16, device=DEV))
    with pytest.raises(ValueError):
        ops.dense_linear(torch.zeros(4, 256, device=DEV), torch.zeros(16, 256, device=DEV))          # fp32


def _setup(seed, prefix, n, first_streamed=None):
    kv = create_kv_cache("static", max_cache_len=max(256, prefix + n + 8), config=CFG, device=DEV, dtype=torch.bfloat16)
    target, draft, w = build_models(CFG, kv, seed=seed, device=DEV, first_streamed=first_streamed)
    g = torch.Generator().manual_seed(seed)
    prompt = torch.randint(0, CFG.vocab_size, (prefix,), generator=g).to(DEV)
    target.prefill(prompt, 0)
    parents, _, depths = W.random_tree(g, n=n, max_depth=5, max_children=3 if n <= 200 else 4, vocab=CFG.vocab_size, chain_depth=3)
    toks = torch.randint(0, CFG.vocab_size, (n,), generator=g).to(DEV)
    anc = ops.ancestor_bits_tensor(parents, device=DEV)
    return kv, target, toks, torch.tensor(depths, device=DEV), anc


@pytest.mark.parametrize("n,prefix,first_streamed", [(1, 17, None), (9, 40, None), (33, 100, 1), (64, 130, None),
                                                     (65, 70, None), (200, 300, 1), (289, 130, None), (384, 64, None)])
def test_target_native_layers_match_module_path(n, prefix, first_streamed):
    print("dense decoder layer stack", n, prefix, first_streamed, flush=True)
    kv, target, toks, depths, anc = _setup(21 + n, prefix, n, first_streamed)
    assert target.native_layers
    saved = kv.cache.data.clone()
    target.use_native_layers = False
    ref = target.tree_forward(toks, depths, anc, prefix)
    ref_cache = kv.cache.data.clone()
    kv.cache.data.copy_(saved)
    target.use_native_layers = True
    got = target.tree_forward(toks, depths, anc, prefix)
    scale = ref.float().abs().amax().item()
    assert (got.float() - ref.float()).abs().amax().item() <= 2e-2 * scale
    dc = (kv.cache.data.float() - ref_cache.float()).abs()
    assert dc[..., :prefix, :].amax().item() == 0 and dc[..., prefix + n:, :].amax().item() == 0
    assert dc.amax().item() <= 2e-2 * ref_cache.float().abs().amax().item()
    assert (got.argmax(-1) == ref.argmax(-1)).float().mean().item() >= 0.9
    # a second forward (slab ring keeps turning for the streamed layers) gives the same bits
    kv.cache.data.copy_(saved)
    assert torch.equal(target.tree_forward(toks, depths, anc, prefix), got)


def test_single_dense_layer_against_float32_oracle():
    n, prefix = 12, 29
    kv, target, toks, depths, anc = _setup(5, prefix, n)
    cfg = CFG
    wl = target.layers[0]
    x0 = target.embed[toks].clone()
    positions = (depths + prefix).to(torch.int32)
    rows = torch.arange(prefix, prefix + n, device=DEV, dtype=torch.int32)
    dims = ops.decoder_layer_dims(torch.bfloat16, n, cfg.hidden_size, cfg.intermediate_size, cfg.num_attention_heads,
                                  cfg.num_key_value_heads, cfg.head_dim, 256, prefix, n, cfg.rms_norm_eps, cfg.rope_theta)
    ws = torch.empty(ops.decoder_layer_workspace(dims), dtype=torch.uint8, device=DEV)
    kc, vc = kv.cache.k(0)[0].float().cpu().clone(), kv.cache.v(0)[0].float().cpu().clone()
    x = x0.clone()
    ops.decoder_layer_(x, dims, ops.dense_layer_weights(wl), positions, rows, anc, kv.cache.k(0), kv.cache.v(0), ws)
    wd = {"input_norm": wl["input_layernorm.weight"].float().cpu(), "post_norm": wl["post_attention_layernorm.weight"].float().cpu(),
          "qkv": wl["qkv_proj.weight"].float().cpu(), "qkv_bias": wl["qkv_proj.bias"].float().cpu() if "qkv_proj.bias" in wl else None,
          "o": wl["o_proj.weight"].float().cpu(), "gate_up": wl["gate_up_proj.weight"].float().cpu(),
          "down": wl["down_proj.weight"].float().cpu()}
    bits = [int(b) & ((1 << 64) - 1) for b in anc.cpu().tolist()]
    want = od.decoder_layer(x0.float().cpu(), wd, kc, vc, positions.cpu().long(), rows.cpu().long(), bits, prefix,
                            cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim, cfg.rms_norm_eps, cfg.rope_theta)
    err = (x.float().cpu() - want).abs().amax().item()
    assert err <= 2e-2 * want.abs().amax().item(), (err, want.abs().amax().item())
    assert (kv.cache.k(0)[0].float().cpu() - kc).abs().amax().item() <= 2e-2 * kc.abs().amax().item()
    assert (kv.cache.v(0)[0].float().cpu() - vc).abs().amax().item() <= 2e-2 * vc.abs().amax().item()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_dense_gate_up_projection_with_the_activation_in_its_output_stage(dtype):
    """As for the int4 twin: the fused launch against the plain projection followed by the activation on the values
    it stored; only the exponential may differ in its last place."""
    for seed, (F, K, M, bias) in enumerate([(16, 64, 1, False), (48, 192, 5, True), (1184, 128, 17, True), (18944, 3584, 8, False),
                                            (18944, 3584, 64, False), (2048, 512, 33, True), (40000, 64, 3, False),
                                            (2048, 512, 65, True), (18944, 3584, 289, False), (1184, 128, 384, True)]):
        print("dense gate|up + silu", dtype, F, K, M, bias, flush=True)
        g = torch.Generator().manual_seed(800 + seed)
        W = (torch.randn(2 * F, K, generator=g) * (2.0 / K ** 0.5)).to(dtype).to(DEV)
        x = torch.randn(M, K, generator=g).to(dtype).to(DEV)
        b = (torch.randn(2 * F, generator=g) * 0.1).to(dtype).to(DEV) if bias else None
        got = ops.dense_gate_up_silu(x, W, b)
        gu = ops.dense_linear(x, W, b)
        gate, up = gu[:, :F].float(), gu[:, F:].float()
        want = ((gate / (1 + torch.exp(-gate))).to(dtype).float() * up).to(dtype)
        assert got.shape == (M, F) and got.dtype == dtype
        differing = int((got != want).sum())
        assert differing <= max(1, got.numel() // 1000), (F, K, M, differing)
        ulp = 2.0 ** (-7 if dtype == torch.bfloat16 else -10)
        assert ((got.float() - want.float()).abs() <= 2 * ulp * want.float().abs() + 1e-6).all()
