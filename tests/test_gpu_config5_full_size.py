"""BASELINE config 5 as a whole, at its full size: a random-init Qwen2.5-7B-shaped decoder (28 layers, hidden 3584, 28 / 4
heads of 128, FFN 18944, vocabulary 152064), target bf16, substitute draft = the same weights int4 g64, depth-8 / k-8
tree capped at 64 nodes, prompt of 2048 random ids (the cycle of specdecodes/models/generators/subspec_sd.py:82-124).

The reference cannot run here, so the cycle is pinned by what defines lossless speculative decoding and layer streaming:
* with exact verification every emitted token is the target's greedy choice under teacher forcing (or tied with it as
  far as bf16 logits can tell);
* streaming layers 14-27 from pinned host memory changes nothing: the tokens and the K / V rows of the accepted
  sequence are bit-identical to the all-resident run;
* with a draft that agrees with its target (the target runs the draft's dequantized weights) the cycle accepts deep paths.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu

from subspec_amd import quant
from subspec_amd.cache import create_kv_cache
from subspec_amd.draft import SubSpecSDDraftModel
from subspec_amd.generator import SubSpecSDGenerator
from subspec_amd.model import QUANTIZED, DecoderConfig, build_models, init_weights
from subspec_amd.utils import DraftParams
from subspec_amd.wandb_logger import wandb_logger

DEV = "cuda:0"
PROMPT, NEW = 2048, 40


def _generate(cfg, weights, keep_layers, prompt, new_tokens=NEW):
    kv = create_kv_cache("static", max_cache_len=PROMPT + new_tokens + 72, config=cfg, device=DEV, dtype=torch.bfloat16)
    target, draft, _ = build_models(cfg, kv, device=DEV, first_streamed=keep_layers, weights=weights)
    gen = SubSpecSDGenerator(target, None, SubSpecSDDraftModel(draft),
                             DraftParams(temperature=0.2, max_depth=8, topk_len=8, max_verify_tokens=64),
                             generator_kwargs=dict(verify_method="exact"))
    wandb_logger.clear_log_data()
    out = gen.generate(prompt, max_new_tokens=new_tokens, do_sample=False, past_key_values=kv)
    torch.cuda.synchronize()
    log = dict(wandb_logger.log_data)
    rows = kv.cache.data[..., :kv.get_seq_length(), :].clone()        # K / V rows of the accepted sequence, every layer
    return out[0], log, rows, target, kv


def test_config5_cycle_at_full_size():
    cfg = DecoderConfig()
    assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.vocab_size) == (28, 3584, 152064)
    base = init_weights(cfg, 0, DEV)
    prompt = torch.randint(0, cfg.vocab_size, (1, PROMPT), generator=torch.Generator().manual_seed(0)).to(DEV)

    # ---- all layers resident
    print("config 5: resident run", flush=True)
    seq, log, rows, target, kv = _generate(cfg, base, cfg.num_hidden_layers, prompt)
    assert seq.numel() == PROMPT + NEW and log["n_tokens"] == NEW
    assert torch.equal(seq[:PROMPT], prompt[0])
    # teacher forcing through the same target, on the device, in chunks of the prefill path
    print("config 5: teacher forcing", flush=True)
    kv.reset()
    logits = target.prefill(seq[:-1], 0, all_logits=True)[PROMPT - 1:].float()       # row t scores token PROMPT + t
    emitted = seq[PROMPT:]
    scale = logits.abs().amax().item()
    top = logits.argmax(-1)
    gap = logits.amax(-1) - logits.gather(1, emitted.unsqueeze(1)).squeeze(1)
    exact = int((top == emitted).sum())
    print(f"config 5: {exact} of {NEW} tokens are the argmax under teacher forcing, largest gap {gap.max().item():.4f} "
          f"of a logit scale {scale:.3f}", flush=True)
    assert gap.max().item() <= 2e-2 * scale, (gap.max().item(), scale)
    assert exact >= 0.8 * NEW, exact
    del target, kv, logits
    torch.cuda.empty_cache()

    # ---- layers 14-27 streamed from pinned host memory: same tokens, same cache rows
    print("config 5: streamed run", flush=True)
    seq_s, log_s, rows_s, target_s, kv_s = _generate(cfg, base, 14, prompt)
    assert target_s.streamer is not None and target_s.streamer.bytes_streamed > 14 * 400e6 * log_s["n_iter"]
    assert torch.equal(seq_s, seq)
    assert rows_s.shape == rows.shape and torch.equal(rows_s, rows)
    del target_s, kv_s, rows_s, rows
    torch.cuda.empty_cache()

    # ---- a draft that agrees with its target accepts deep paths (at most 9 tokens per cycle)
    print("config 5: agreeing draft", flush=True)
    agree = {**base, "layers": [dict(w) for w in base["layers"]]}
    for w in agree["layers"]:
        for name in QUANTIZED:
            t = w[name + ".weight"]
            w[name + ".weight"] = quant.dequantize(*quant.quantize_int4_g64(t)).to(t.dtype)
    seq_a, log_a, _, _, _ = _generate(cfg, agree, cfg.num_hidden_layers, prompt, new_tokens=64)
    print("config 5: agreeing draft, tokens per cycle", log_a["avg_sampled"], flush=True)
    assert log_a["avg_sampled"] >= 7.0, log_a["avg_sampled"]
