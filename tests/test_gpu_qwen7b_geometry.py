"""GPU: the decoder-layer path at the Qwen2.5-7B geometry of BASELINE config 5 -- hidden 3584, 28 query heads over
4 KV heads (7:1 GQA), head_dim 128, FFN 18944, prefix 2048 -- instead of the small decoder the other cycle tests use.

* one `subspec_int4_decoder_layer` (8 and 64 tree rows) and one `subspec_dense_decoder_layer` call (8 to 289 rows) against the
  float32 oracle layer (`oracle/decoder.py`) on the same (for the draft: dequantized) weights: residual stream and
  the K / V rows written, tolerance 2e-2 of the largest magnitude (bf16 intermediates, as for the small geometry);
* rotary positions near 32k (the reference's `max_position_embeddings`) through the same entry point;
* a target whose last two layers stream through the 466 MB device slab ring equals the all-resident target bit for
  bit, over several forwards (the ring keeps turning across forwards).
"""
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import decoder as od
from oracle import int4 as oi
from subspec_amd import ops, workloads as W
from subspec_amd.cache import create_kv_cache
from subspec_amd.model import DecoderConfig, build_models, init_weights, layer_shapes, quantize_layers

DEV = "cuda:0"
PREFIX = 2048


def _cfg(layers=1, vocab=4096):
    return DecoderConfig(num_hidden_layers=layers, vocab_size=vocab)        # every other field defaults to Qwen2.5-7B


def _layer_case(seed, n, prefix, max_len, depth_base=0):
    cfg = _cfg()
    g = torch.Generator().manual_seed(seed)
    w = init_weights(cfg, seed, DEV)["layers"][0]
    # norm gains away from 1 so that a dropped gain would show
    for name in ("input_layernorm.weight", "post_attention_layernorm.weight"):
        w[name] = (1 + 0.2 * torch.randn(cfg.hidden_size, generator=g)).to(torch.bfloat16).to(DEV)
    parents, _, depths = W.random_tree(g, n=n, max_depth=8, max_children=4, vocab=cfg.vocab_size, chain_depth=6)
    anc = ops.ancestor_bits_tensor(parents, device=DEV)
    x0 = torch.randn(n, cfg.hidden_size, generator=g).to(torch.bfloat16).to(DEV)
    kc = torch.randn(cfg.num_key_value_heads, max_len, cfg.head_dim, generator=g).to(torch.bfloat16)
    vc = torch.randn(cfg.num_key_value_heads, max_len, cfg.head_dim, generator=g).to(torch.bfloat16)
    positions = (torch.tensor(depths) + prefix + depth_base).to(torch.int32).to(DEV)
    rows = torch.arange(prefix, prefix + n, dtype=torch.int32, device=DEV)
    return cfg, w, anc, x0, kc, vc, positions, rows


def _oracle(cfg, wd, x0, kc, vc, positions, rows, anc, prefix):
    mask = (1 << 64) - 1
    if anc.dim() == 1:
        bits = [int(b) & mask for b in anc.cpu().tolist()]
    else:                                            # more than 64 tree slots: several 64-bit words per row
        bits = [sum((int(wd_) & mask) << (64 * i) for i, wd_ in enumerate(row)) for row in anc.cpu().tolist()]
    k, v = kc.float().clone(), vc.float().clone()
    want = od.decoder_layer(x0.float().cpu(), wd, k, v, positions.cpu().long(), rows.cpu().long(), bits, prefix,
                            cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim, cfg.rms_norm_eps, cfg.rope_theta)
    return want, k, v


def _check(x, kd, vd, want, k, v, prefix, n, tag):
    err = (x.float().cpu() - want).abs().amax().item()
    assert err <= 2e-2 * want.abs().amax().item(), (tag, err, want.abs().amax().item())
    for got, ref, name in ((kd, k, "K"), (vd, v, "V")):
        got = got.float().cpu()
        # rows outside the tree are untouched, the tree rows hold the rotated keys / the values
        assert torch.equal(got[:, :prefix], ref[:, :prefix]) and torch.equal(got[:, prefix + n:], ref[:, prefix + n:]), (tag, name)
        d = (got[:, prefix:prefix + n] - ref[:, prefix:prefix + n]).abs().amax().item()
        assert d <= 2e-2 * ref[:, prefix:prefix + n].abs().amax().item(), (tag, name, d)


def _dims(cfg, n, max_len, prefix):
    return ops.decoder_layer_dims(torch.bfloat16, n, cfg.hidden_size, cfg.intermediate_size, cfg.num_attention_heads,
                                  cfg.num_key_value_heads, cfg.head_dim, max_len, prefix, n, cfg.rms_norm_eps, cfg.rope_theta)


@pytest.mark.parametrize("n", [8, 64, 65, 289])
def test_dense_target_layer_at_7b_geometry(n):
    """65 and 289 rows (a whole depth-48, k-6 tree of the reference's offloading configuration, 1 + 48 * 6 nodes) take the
    32 x 32 x 16 projections and several 64-row attention windows inside the same call."""
    print("7B geometry, dense layer, rows", n, flush=True)
    max_len = PREFIX + max(64, n)
    cfg, w, anc, x0, kc, vc, positions, rows = _layer_case(100 + n, n, PREFIX, max_len)
    dims = _dims(cfg, n, max_len, PREFIX)
    ws = torch.empty(ops.decoder_layer_workspace(dims), dtype=torch.uint8, device=DEV)
    kd, vd = kc.to(DEV).unsqueeze(0), vc.to(DEV).unsqueeze(0)
    x = x0.clone()
    ops.decoder_layer_(x, dims, ops.dense_layer_weights(w), positions, rows, anc, kd, vd, ws)
    torch.cuda.synchronize()
    wd = {"input_norm": w["input_layernorm.weight"].float().cpu(), "post_norm": w["post_attention_layernorm.weight"].float().cpu(),
          "qkv": w["qkv_proj.weight"].float().cpu(), "qkv_bias": w["qkv_proj.bias"].float().cpu(),
          "o": w["o_proj.weight"].float().cpu(), "gate_up": w["gate_up_proj.weight"].float().cpu(),
          "down": w["down_proj.weight"].float().cpu()}
    want, k, v = _oracle(cfg, wd, x0, kc, vc, positions, rows, anc, PREFIX)
    _check(x, kd[0], vd[0], want, k, v, PREFIX, n, ("dense", n))


@pytest.mark.parametrize("n,prefix,depth_base", [(8, PREFIX, 0), (64, PREFIX, 0), (8, 40, 32000), (13, PREFIX, 0), (16, 300, 0)])
def test_int4_draft_layer_at_7b_geometry(n, prefix, depth_base):
    """depth_base = 32000: rotary positions near 32k through the same kernels (the angle is formed in fp32 from the
    position and the inverse frequency; the oracle's table is the eager formula)."""
    print("7B geometry, int4 layer, rows", n, "prefix", prefix, "positions from", prefix + depth_base, flush=True)
    max_len = prefix + 64
    cfg, w, anc, x0, kc, vc, positions, rows = _layer_case(200 + n, n, prefix, max_len, depth_base)
    wl = quantize_layers([w])[0]
    dims = _dims(cfg, n, max_len, prefix)
    ws = torch.empty(ops.decoder_layer_workspace(dims), dtype=torch.uint8, device=DEV)
    kd, vd = kc.to(DEV).unsqueeze(0), vc.to(DEV).unsqueeze(0)
    x = x0.clone()
    ops.decoder_layer_(x, dims, ops.decoder_layer_weights(wl), positions, rows, anc, kd, vd, ws)
    torch.cuda.synchronize()

    def dense(name, N, K):
        return oi.dequant(*oi.unpack_tiled(wl[name + ".wq"].cpu(), wl[name + ".sz"].cpu(), N, K))
    Q, KV, H, F = cfg.q_size, cfg.kv_size, cfg.hidden_size, cfg.intermediate_size
    wd = {"input_norm": w["input_layernorm.weight"].float().cpu(), "post_norm": w["post_attention_layernorm.weight"].float().cpu(),
          "qkv": dense("qkv_proj", Q + 2 * KV, H), "qkv_bias": w["qkv_proj.bias"].float().cpu(),
          "o": dense("o_proj", H, Q), "gate_up": dense("gate_up_proj", 2 * F, H), "down": dense("down_proj", H, F)}
    want, k, v = _oracle(cfg, wd, x0, kc, vc, positions, rows, anc, prefix)
    _check(x, kd[0], vd[0], want, k, v, prefix, n, ("int4", n, prefix))


def test_slab_ring_at_7b_layer_size_is_bit_identical_to_resident():
    """Three 7B-shaped layers, the last two streamed from pinned host memory through the device slab ring (466 MB per
    slab) against the same weights all resident: logits and cache bit-identical over a prefill and three tree
    forwards (the ring prefetches the next forward's first layers while the current one ends)."""
    cfg = _cfg(layers=3, vocab=2048)
    print("7B geometry, slab ring: 3 layers, 2 streamed,", sum(int(torch.tensor(s).prod()) for s in layer_shapes(cfg).values()) * 2,
          "bytes per layer", flush=True)
    w = init_weights(cfg, 7, DEV)
    kv_a = create_kv_cache("static", max_cache_len=256, config=cfg, device=DEV, dtype=torch.bfloat16)
    kv_b = create_kv_cache("static", max_cache_len=256, config=cfg, device=DEV, dtype=torch.bfloat16)
    tgt_a, _, _ = build_models(cfg, kv_a, device=DEV, weights=w)
    tgt_b, _, _ = build_models(cfg, kv_b, device=DEV, weights=w, first_streamed=1)
    assert tgt_b.streamer is not None and tgt_b.streamer.n == 2 and tgt_b.streamer.layout.nbytes > 460_000_000
    g = torch.Generator().manual_seed(9)
    prompt = torch.randint(0, cfg.vocab_size, (48,), generator=g).to(DEV)
    assert torch.equal(tgt_a.prefill(prompt, 0), tgt_b.prefill(prompt, 0))
    for n in (64, 8, 33):
        parents, _, depths = W.random_tree(g, n=n, max_depth=8, max_children=4, vocab=cfg.vocab_size, chain_depth=4)
        toks = torch.randint(0, cfg.vocab_size, (n,), generator=g).to(DEV)
        anc = ops.ancestor_bits_tensor(parents, device=DEV)
        dep = torch.tensor(depths, device=DEV)
        la = tgt_a.tree_forward(toks, dep, anc, 48)
        lb = tgt_b.tree_forward(toks, dep, anc, 48)
        assert torch.equal(la, lb), n
        assert torch.equal(kv_a.cache.data, kv_b.cache.data), n
    st = tgt_b.streamer
    assert 4 * 2 * st.layout.nbytes <= st.bytes_streamed <= (4 * 2 + st.n_slabs - 1) * st.layout.nbytes
