"""GPU: the post-speculation cycle driver.  What the reference fixes here is an invariant, not a vector (the number
of post-speculation steps that fit into a target forward depends on timing there): whatever the draft adds to the
tree while the target runs, the emitted tokens are the target's own continuation, and the KV cache ends up holding
exactly the accepted rows.  So the v2 driver is compared with the v1 driver on the same models, with the number of
post-speculation steps forced to 0, 1, 4 and polled, for a draft that agrees with the target (long accepted
paths, the post-verify branch taken every other cycle) and one that does not (random weights)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from subspec_amd import quant
from subspec_amd.cache import create_kv_cache
from subspec_amd.draft import SubSpecSDDraftModel
from subspec_amd.generator import SubSpecSDGenerator
from subspec_amd.generator_v2 import SubSpecSDGeneratorV2
from subspec_amd.model import QUANTIZED, DecoderConfig, build_models, init_weights
from subspec_amd.utils import DraftParams
from subspec_amd.wandb_logger import wandb_logger

DEV = "cuda:0"
CFG = DecoderConfig(num_hidden_layers=4, hidden_size=256, num_attention_heads=2, num_key_value_heads=1,
                    head_dim=128, intermediate_size=512, vocab_size=2048)


def _weights(agreeing, seed=9):
    w = init_weights(CFG, seed, DEV)
    if agreeing:
        for layer in w["layers"]:
            for name in QUANTIZED:
                t = layer[name + ".weight"]
                layer[name + ".weight"] = quant.dequantize(*quant.quantize_int4_g64(t)).to(t.dtype)
    return w


def _assert_greedy_continuation(weights, seq, start, tag):
    """Teacher forcing through the target (resident, torch prefill path): every token from ``start`` on is the argmax
    of the logits at its prefix, or within what bf16 can tell apart of it (different tree shapes change the order of
    the attention sums, and this random model has many near-ties)."""
    kv = create_kv_cache("static", max_cache_len=512, config=CFG, device=DEV, dtype=torch.bfloat16)
    target, _, _ = build_models(CFG, kv, device=DEV, weights=weights)
    logits = target.prefill(seq[:-1].to(DEV), 0, all_logits=True).float().cpu()      # row t scores token t + 1
    scale = logits.abs().amax().item()
    exact = 0
    for t in range(start - 1, seq.numel() - 1):
        tok = int(seq[t + 1])
        if tok == int(logits[t].argmax()):
            exact += 1
        else:
            gap = float(logits[t].max() - logits[t, tok])
            assert gap <= 2e-2 * scale, (tag, t, tok, int(logits[t].argmax()), gap, scale)
    assert exact >= 0.85 * (seq.numel() - start), (tag, exact)


def _run(cls, weights, first_streamed, new_tokens=60, verify="exact", **gk):
    kv = create_kv_cache("static", max_cache_len=512, config=CFG, device=DEV, dtype=torch.bfloat16)
    target, draft, _ = build_models(CFG, kv, device=DEV, weights=weights, first_streamed=first_streamed)
    vk = dict(threshold=0.9, window_size=1, threshold_method="entropy") if verify == "lossy" else None
    gen = cls(target, None, SubSpecSDDraftModel(draft), DraftParams(temperature=0.2, max_depth=4, topk_len=4),
              generator_kwargs=dict(verify_method=verify, verify_kwargs=vk, **gk))
    prompt = torch.randint(0, CFG.vocab_size, (1, 32), generator=torch.Generator().manual_seed(4)).to(DEV)
    wandb_logger.clear_log_data()
    out = gen.generate(prompt, max_new_tokens=new_tokens, do_sample=False, past_key_values=kv)
    torch.cuda.synchronize()
    return out[0].cpu(), dict(wandb_logger.log_data), kv, gen


@pytest.mark.parametrize("agreeing", [True, False])
@pytest.mark.parametrize("first_streamed", [None, 2])
def test_v2_emits_what_v1_emits(agreeing, first_streamed):
    w = _weights(agreeing)
    ref, ref_log, ref_kv, _ = _run(SubSpecSDGenerator, w, first_streamed)
    _assert_greedy_continuation(w, ref, 32, "v1")
    for steps in (0, 1, 4, None):
        print("v2", agreeing, first_streamed, steps, flush=True)
        out, log, kv, gen = _run(SubSpecSDGeneratorV2, w, first_streamed, postspec_steps=steps)
        assert out.numel() == ref.numel() and torch.equal(out[:32], ref[:32])
        _assert_greedy_continuation(w, out, 32, (agreeing, first_streamed, steps))
        if steps == 0:
            assert torch.equal(out, ref)                     # without extension the two drivers are the same program
        assert kv.get_seq_length() == out.numel() - 1
        # the cache holds the rows of the emitted sequence: compare with a fresh prefill of it
        L = kv.get_seq_length()
        kv2 = create_kv_cache("static", max_cache_len=512, config=CFG, device=DEV, dtype=torch.bfloat16)
        t2, _, _ = build_models(CFG, kv2, device=DEV, weights=w)
        t2.prefill(out[:-1].to(DEV), 0)
        a, b = kv.cache.data[..., :L, :].float(), kv2.cache.data[..., :L, :].float()
        assert (a - b).abs().amax().item() <= 5e-2 * b.abs().amax().item()
        assert log["speculate_count"] + log["post_verify_count"] == log["n_iter"]
        assert abs(log["post_verify_rate"] * log["n_iter"] - log["post_verify_count"]) < 1e-6
        if steps == 0:
            assert log["post_verify_count"] == 0 and log["n_iter"] == ref_log["n_iter"]
        if agreeing and steps == 4:
            # fully accepted trees continue into the extension instead of being speculated afresh
            assert log["post_verify_count"] >= 3, log
            assert log["speculate_count"] < ref_log["n_iter"]


@pytest.mark.parametrize("cls,steps", [(SubSpecSDGenerator, None), (SubSpecSDGeneratorV2, 3), (SubSpecSDGeneratorV2, None)])
def test_deep_trees_beyond_one_window(cls, steps):
    """Depth 20 x 6 = 121 nodes (the shape of the reference's depth-48 x 6 trees at test size): the target decodes
    the tree in two windows of rows and the draft's masks take more than one word."""
    w = _weights(True)
    kv = create_kv_cache("static", max_cache_len=1024, config=CFG, device=DEV, dtype=torch.bfloat16)
    target, draft, _ = build_models(CFG, kv, device=DEV, weights=w, first_streamed=2)
    gk = {} if steps is None and cls is SubSpecSDGenerator else dict(postspec_steps=steps)
    gen = cls(target, None, SubSpecSDDraftModel(draft), DraftParams(temperature=0.2, max_depth=20, topk_len=6),
              generator_kwargs=dict(verify_method="exact", **gk))
    prompt = torch.randint(0, CFG.vocab_size, (1, 32), generator=torch.Generator().manual_seed(4)).to(DEV)
    wandb_logger.clear_log_data()
    out = gen.generate(prompt, max_new_tokens=120, do_sample=False, past_key_values=kv)[0].cpu()
    log = dict(wandb_logger.log_data)
    print("deep trees", cls.__name__, steps, log["n_iter"], log["avg_sampled"], flush=True)
    assert out.numel() == 152
    _assert_greedy_continuation(w, out, 32, (cls.__name__, steps))
    assert log["avg_sampled"] > 3.0, log
    L = kv.get_seq_length()
    assert L == out.numel() - 1
    kv2 = create_kv_cache("static", max_cache_len=512, config=CFG, device=DEV, dtype=torch.bfloat16)
    t2, _, _ = build_models(CFG, kv2, device=DEV, weights=w)
    t2.prefill(out[:-1].to(DEV), 0)
    a, b = kv.cache.data[..., :L, :].float(), kv2.cache.data[..., :L, :].float()
    assert (a - b).abs().amax().item() <= 5e-2 * b.abs().amax().item()


def test_v2_lossy_and_sampling_targets_run_through_the_same_loop():
    w = _weights(True)
    ref, _, _, _ = _run(SubSpecSDGenerator, w, 2, verify="lossy")
    out, log, _, _ = _run(SubSpecSDGeneratorV2, w, 2, verify="lossy", postspec_steps=3)
    assert out.numel() == ref.numel() and log["post_verify_count"] >= 1
    # lossy verification may accept other tokens when the tree is deeper, so only the shared prefix must agree
    same = (out[:40] == ref[:40]).float().mean().item()
    assert same >= 0.8, same
    kv = create_kv_cache("static", max_cache_len=512, config=CFG, device=DEV, dtype=torch.bfloat16)
    target, draft, _ = build_models(CFG, kv, device=DEV, weights=w, first_streamed=2)
    gen = SubSpecSDGeneratorV2(target, None, SubSpecSDDraftModel(draft), DraftParams(temperature=0.2, max_depth=4, topk_len=4),
                               generator_kwargs=dict(seed=5, postspec_steps=2))
    prompt = torch.randint(0, CFG.vocab_size, (1, 32), generator=torch.Generator().manual_seed(4)).to(DEV)
    a = gen.generate(prompt, max_new_tokens=30, do_sample=True, temperature=0.8, past_key_values=kv)
    assert a.shape[1] == 62 and kv.get_seq_length() == 61


def test_v2_rejects_trees_beyond_the_slot_limit():
    w = _weights(False)
    kv = create_kv_cache("static", max_cache_len=512, config=CFG, device=DEV, dtype=torch.bfloat16)
    target, draft, _ = build_models(CFG, kv, device=DEV, weights=w)
    gen = SubSpecSDGeneratorV2(target, None, SubSpecSDDraftModel(draft), DraftParams(max_depth=64, topk_len=8))
    with pytest.raises(ValueError):
        gen.generate(torch.zeros(1, 4, dtype=torch.long, device=DEV), max_new_tokens=4, do_sample=False, past_key_values=kv)


@pytest.mark.parametrize("verify", ["exact", "lossy"])
def test_v2_with_a_verify_cap_below_the_tree_size(verify):
    """``max_verify_tokens`` smaller than ``1 + max_depth * topk_len`` (17 nodes, cap 12): the v1 driver cuts the
    tree, the v2 driver must not (its draft keeps extending the uncut deepest level) -- the emitted tokens stay the
    target's greedy continuation, the extension is still taken, and the cache holds the emitted sequence's rows."""
    w = _weights(True)
    kv = create_kv_cache("static", max_cache_len=512, config=CFG, device=DEV, dtype=torch.bfloat16)
    target, draft, _ = build_models(CFG, kv, device=DEV, weights=w, first_streamed=2)
    vk = dict(threshold=0.9, window_size=1, threshold_method="entropy") if verify == "lossy" else None
    gen = SubSpecSDGeneratorV2(target, None, SubSpecSDDraftModel(draft),
                               DraftParams(temperature=0.2, max_depth=4, topk_len=4, max_verify_tokens=12),
                               generator_kwargs=dict(verify_method=verify, verify_kwargs=vk, postspec_steps=3))
    prompt = torch.randint(0, CFG.vocab_size, (1, 32), generator=torch.Generator().manual_seed(4)).to(DEV)
    wandb_logger.clear_log_data()
    out = gen.generate(prompt, max_new_tokens=60, do_sample=False, past_key_values=kv)[0].cpu()
    log = dict(wandb_logger.log_data)
    print("v2 with cap", verify, log["n_iter"], log["avg_sampled"], log["post_verify_count"], flush=True)
    assert out.numel() == 92 and kv.get_seq_length() == 91
    if verify == "exact":
        _assert_greedy_continuation(w, out, 32, "v2 cap")
    assert log["post_verify_count"] >= 2 and log["avg_sampled"] > 2.5, log
    kv2 = create_kv_cache("static", max_cache_len=512, config=CFG, device=DEV, dtype=torch.bfloat16)
    t2, _, _ = build_models(CFG, kv2, device=DEV, weights=w)
    t2.prefill(out[:-1].to(DEV), 0)
    a, b = kv.cache.data[..., :91, :].float(), kv2.cache.data[..., :91, :].float()
    assert (a - b).abs().amax().item() <= 5e-2 * b.abs().amax().item()
