"""GPU: the one-call int4 decoder layer against (a) the module-by-module path built from the same
library kernels plus eager torch glue and (b) the float32 oracle on dequantized weights."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import decoder as od
from oracle import int4 as oi
from subspec_amd import ops, quant, workloads as W
from subspec_amd.cache import create_kv_cache
from subspec_amd.model import DecoderConfig, build_models

DEV = "cuda:0"
CFG = DecoderConfig(num_hidden_layers=3, hidden_size=256, num_attention_heads=2, num_key_value_heads=1,
                    head_dim=128, intermediate_size=512, vocab_size=2048)


def _setup(seed, prefix, n):
    kv = create_kv_cache("static", max_cache_len=256, config=CFG, device=DEV, dtype=torch.bfloat16)
    target, draft, w = build_models(CFG, kv, seed=seed, device=DEV)
    g = torch.Generator().manual_seed(seed)
    prompt = torch.randint(0, CFG.vocab_size, (prefix,), generator=g).to(DEV)
    target.prefill(prompt, 0)
    parents, _, depths = W.random_tree(g, n=n, max_depth=5, max_children=3, vocab=CFG.vocab_size, chain_depth=3)
    toks = torch.randint(0, CFG.vocab_size, (n,), generator=g).to(DEV)
    anc = ops.ancestor_bits_tensor(parents, device=DEV)
    return kv, draft, toks, torch.tensor(depths, device=DEV), anc


@pytest.mark.parametrize("n,prefix", [(1, 17), (9, 40), (33, 100), (64, 130)])
def test_native_layer_stack_matches_module_path(n, prefix):
    print("decoder layer stack", n, prefix, flush=True)
    kv, draft, toks, depths, anc = _setup(11 + n, prefix, n)
    assert draft.native_layers
    saved = kv.cache.data.clone()
    draft.use_native_layers = False
    ref = draft.tree_forward(toks, depths, anc, prefix)
    ref_cache = kv.cache.data.clone()
    kv.cache.data.copy_(saved)
    draft.use_native_layers = True
    got = draft.tree_forward(toks, depths, anc, prefix)
    scale = ref.float().abs().amax().item()
    assert (got.float() - ref.float()).abs().amax().item() <= 2e-2 * scale          # bf16 glue, rounded per op in both
    # K / V rows written by the native rotary kernel against the eager ones; rows outside the tree untouched
    dc = (kv.cache.data.float() - ref_cache.float()).abs()
    assert dc[..., :prefix, :].amax().item() == 0 and dc[..., prefix + n:, :].amax().item() == 0
    assert dc.amax().item() <= 2e-2 * ref_cache.float().abs().amax().item()
    assert (got.argmax(-1) == ref.argmax(-1)).float().mean().item() >= 0.9


@pytest.mark.parametrize("n_slots,lo,hi", [(289, 283, 289), (289, 225, 289), (400, 130, 190), (512, 448, 512)])
def test_windows_of_large_trees(n_slots, lo, hi):
    """A window of rows of a tree with up to 512 occupied slots (a draft level of a depth-48 tree, a
    post-speculation window): the one-call layers against the whole tree decoded module by module."""
    print("decoder layer large tree", n_slots, lo, hi, flush=True)
    prefix = 70
    kv = create_kv_cache("static", max_cache_len=640, config=CFG, device=DEV, dtype=torch.bfloat16)
    target, draft, w = build_models(CFG, kv, seed=n_slots, device=DEV)
    g = torch.Generator().manual_seed(n_slots)
    target.prefill(torch.randint(0, CFG.vocab_size, (prefix,), generator=g).to(DEV), 0)
    parents, _, depths = W.random_tree(g, n=n_slots, max_depth=48, max_children=6, vocab=CFG.vocab_size, chain_depth=40)
    toks = torch.randint(0, CFG.vocab_size, (n_slots,), generator=g).to(DEV)
    anc = ops.ancestor_bits_tensor(parents, device=DEV)
    dep = torch.tensor(depths, device=DEV)
    # the whole tree, module by module (rows beyond one 64-row launch): fills the cache rows of every node
    ref = draft.tree_forward(toks, dep, anc, prefix)
    ref_cache = kv.cache.data.clone()
    # the window again through the one-call layers, over the cache the first pass left
    got = draft.tree_forward(toks[lo:hi], dep[lo:hi], anc[lo:hi].contiguous(), prefix, first_slot=lo, n_tree_slots=n_slots)
    scale = ref.float().abs().amax().item()
    assert (got.float() - ref[lo:hi].float()).abs().amax().item() <= 2e-2 * scale
    assert (got.argmax(-1) == ref[lo:hi].argmax(-1)).float().mean().item() >= 0.9
    dc = (kv.cache.data.float() - ref_cache.float()).abs()
    assert dc[..., :prefix + lo, :].amax().item() == 0 and dc[..., prefix + hi:, :].amax().item() == 0
    assert dc.amax().item() <= 2e-2 * ref_cache.float().abs().amax().item()


def test_single_layer_against_float32_oracle():
    n, prefix = 12, 29
    kv, draft, toks, depths, anc = _setup(5, prefix, n)
    cfg = CFG
    wl = draft.layers[0]
    x0 = draft.embed[toks].clone()
    positions = (depths + prefix).to(torch.int32)
    rows = torch.arange(prefix, prefix + n, device=DEV, dtype=torch.int32)
    dims = ops.decoder_layer_dims(torch.bfloat16, n, cfg.hidden_size, cfg.intermediate_size, cfg.num_attention_heads,
                                  cfg.num_key_value_heads, cfg.head_dim, 256, prefix, n, cfg.rms_norm_eps, cfg.rope_theta)
    ws = torch.empty(ops.decoder_layer_workspace(dims), dtype=torch.uint8, device=DEV)
    kc, vc = kv.cache.k(0)[0].float().cpu().clone(), kv.cache.v(0)[0].float().cpu().clone()
    x = x0.clone()
    ops.int4_decoder_layer_(x, dims, ops.decoder_layer_weights(wl), positions, rows, anc, kv.cache.k(0), kv.cache.v(0), ws)

    def dense(name, N, K):
        wq, sz = wl[name + ".wq"].cpu(), wl[name + ".sz"].cpu()
        return oi.dequant(*oi.unpack_tiled(wq, sz, N, K))
    Q, KV, H, F = cfg.q_size, cfg.kv_size, cfg.hidden_size, cfg.intermediate_size
    wd = {"input_norm": wl["input_layernorm.weight"].float().cpu(), "post_norm": wl["post_attention_layernorm.weight"].float().cpu(),
          "qkv": dense("qkv_proj", Q + 2 * KV, H), "qkv_bias": wl["qkv_proj.bias"].float().cpu() if "qkv_proj.bias" in wl else None,
          "o": dense("o_proj", H, Q), "gate_up": dense("gate_up_proj", 2 * F, H), "down": dense("down_proj", H, F)}
    bits = [int(b) & ((1 << 64) - 1) for b in anc.cpu().tolist()]
    want = od.decoder_layer(x0.float().cpu(), wd, kc, vc, positions.cpu().long(), rows.cpu().long(), bits, prefix,
                            cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim, cfg.rms_norm_eps, cfg.rope_theta)
    err = (x.float().cpu() - want).abs().amax().item()
    assert err <= 2e-2 * want.abs().amax().item(), (err, want.abs().amax().item())
    assert (kv.cache.k(0)[0].float().cpu() - kc).abs().amax().item() <= 2e-2 * kc.abs().amax().item()
    assert (kv.cache.v(0)[0].float().cpu() - vc).abs().amax().item() <= 2e-2 * vc.abs().amax().item()


def test_rejects_bad_arguments():
    dims = ops.decoder_layer_dims(torch.bfloat16, 385, 256, 512, 2, 1, 128, 1024, 10, 8, 1e-6, 1e6)
    with pytest.raises(ValueError):
        ops.decoder_layer_workspace(dims)
    # the int4 stack takes windows of at most 64 rows (the dense stack up to 384)
    kv, draft, _, _, _ = _setup(3, 20, 8)
    dims = ops.decoder_layer_dims(torch.bfloat16, 65, CFG.hidden_size, CFG.intermediate_size, CFG.num_attention_heads,
                                  CFG.num_key_value_heads, CFG.head_dim, 256, 10, 65, CFG.rms_norm_eps, CFG.rope_theta)
    ws = torch.empty(ops.decoder_layer_workspace(dims), dtype=torch.uint8, device=DEV)
    with pytest.raises(ValueError):
        ops.int4_decoder_layer_(torch.zeros(65, CFG.hidden_size, dtype=torch.bfloat16, device=DEV), dims,
                                ops.decoder_layer_weights(draft.layers[0]), torch.zeros(65, dtype=torch.int32, device=DEV),
                                torch.zeros(65, dtype=torch.int32, device=DEV), torch.zeros(65, 2, dtype=torch.int64, device=DEV),
                                kv.cache.k(0), kv.cache.v(0), ws)
    with pytest.raises(ValueError):
        ops.decoder_layer_dims(torch.float32, 8, 256, 512, 2, 1, 128, 256, 10, 8, 1e-6, 1e6)
    dims = ops.decoder_layer_dims(torch.bfloat16, 8, 256, 512, 2, 1, 64, 256, 10, 8, 1e-6, 1e6)    # head_dim 64
    with pytest.raises(ValueError):
        ops.decoder_layer_workspace(dims)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_rms_norm_matches_the_eager_formula(dtype):
    """The standalone RMSNorm against HuggingFace's formula (fp32 normalization, rounded, then the gain) evaluated
    by torch on the same inputs: the only freedom is the order of the fp32 sum of squares, so values agree to a
    couple of units in the last place of the 16-bit type and almost all agree exactly."""
    g = torch.Generator().manual_seed(1)
    for rows, hidden in ((1, 8), (7, 256), (64, 3584), (300, 5120), (3, 16384)):
        x = (torch.randn(rows, hidden, generator=g) * 3).to(dtype)
        w = (1 + 0.1 * torch.randn(hidden, generator=g)).to(dtype)
        got = ops.rms_norm(x.to(DEV), w.to(DEV), 1e-6).cpu()
        xf = x.float()
        ref = w * (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6)).to(dtype)
        assert got.shape == ref.shape and got.dtype == dtype
        same = (got == ref).float().mean().item()
        assert same >= 0.99, (rows, hidden, same)
        ulp = 2.0 ** (-7 if dtype == torch.bfloat16 else -10)
        assert ((got.float() - ref.float()).abs() <= 2.5 * ulp * ref.float().abs() + 1e-6).all()     # a flipped rounding of the normalized value, times the gain, rounded again
    # leading dimensions are kept, a zero row stays zero
    x = torch.zeros(2, 3, 64, dtype=dtype, device=DEV)
    assert ops.rms_norm(x, torch.ones(64, dtype=dtype, device=DEV), 1e-6).abs().max().item() == 0
    with pytest.raises(ValueError):
        ops.rms_norm(torch.zeros(2, 12, dtype=dtype, device=DEV), torch.ones(12, dtype=dtype, device=DEV), 1e-6)
    with pytest.raises(ValueError):
        ops.rms_norm(torch.zeros(2, 64, device=DEV), torch.ones(64, device=DEV), 1e-6)          # fp32
