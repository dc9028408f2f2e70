"""GPU: the plug-in seam end to end, in the order the reference's pipeline builder runs it (run/core/builder.py:318-369):
load_model_fn -> load_draft_model_fn -> recipe.generate_configurations -> apply_quantization(draft_model.model) ->
apply_offloading(model, device_map, draft_model=...) -> load_kv_cache_fn -> generator_cls(...).eval() -> generate.
The checkpoint is written by the test; nothing of the reference is imported."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from subspec_amd import registry as R
from subspec_amd.cache import create_kv_cache
from subspec_amd.model import build_models, load_hf_checkpoint
from subspec_amd.quant import HqqInt4Linear
from subspec_amd.wandb_logger import wandb_logger
from test_plugin_seam import StubRegistry, builder_stub, resolve, write_checkpoint

DEV = "cuda:0"
HF = {"model_type": "qwen2", "num_hidden_layers": 4, "hidden_size": 256, "num_attention_heads": 2, "num_key_value_heads": 1,
      "intermediate_size": 512, "vocab_size": 2048, "rms_norm_eps": 1e-6, "rope_theta": 1e6,
      "max_position_embeddings": 4096, "tie_word_embeddings": False}


def _greedy_continuation(path, seq, start, tag):
    """Teacher forcing through a resident target built straight from the checkpoint: every emitted token is the
    argmax at its prefix, or within what bf16 can tell apart of it."""
    cfg, w = load_hf_checkpoint(path, device=DEV)
    kv = create_kv_cache("static", max_cache_len=512, config=cfg, device=DEV, dtype=torch.bfloat16)
    target, _, _ = build_models(cfg, kv, device=DEV, weights=w)
    logits = target.prefill(seq[:-1].to(DEV), 0, all_logits=True).float().cpu()
    scale, exact = logits.abs().amax().item(), 0
    for t in range(start - 1, seq.numel() - 1):
        tok = int(seq[t + 1])
        if tok == int(logits[t].argmax()):
            exact += 1
        else:
            assert float(logits[t].max() - logits[t, tok]) <= 2e-2 * scale, (tag, t)
    assert exact >= 0.85 * (seq.numel() - start), (tag, exact)


@pytest.mark.parametrize("method", ["subspec_sd", "subspec_sd_v2"])
def test_builder_sequence_runs_the_cycle(tmp_path, method):
    path = str(tmp_path)
    write_checkpoint(path, hf=HF, seed=3)
    v2 = method.endswith("v2")
    # v2: three streamed layers through a ring of two slabs (the recipe's prefetch_slabs), v1: two through the default
    recipe = resolve("subspec_amd.recipes:Recipe")(**(dict(keep_first_n_layers_on_gpu=1, prefetch_slabs=2) if v2
                                                      else dict(keep_first_n_layers_on_gpu=2)))
    b = builder_stub(recipe, device=DEV)
    b.max_length = 160
    StubRegistry.entries.clear()
    R.register(StubRegistry, recipe=recipe, llm_path=path)
    entry = StubRegistry.entries[method]
    print("seam:", method, "load", flush=True)
    model, tokenizer = entry.load_model_fn(b, path)
    draft = entry.load_draft_model_fn(b, model, tokenizer, None)
    target_config, draft_config = recipe.generate_configurations(target_model=model, draft_model=draft, max_length=b.max_length,
                                                                 cpu_offload_gb=None, dtype=b.dtype, device=DEV)
    recipe.apply_quantization(draft.model, draft_config["quant_config"], b.dtype, DEV)
    off = recipe.apply_offloading(model, target_config["device_map"], draft_model=draft)
    assert (off.first_streamed, off.streamer.n, off.streamer.n_slabs) == ((1, 3, 2) if v2 else (2, 2, 2))
    # placement: resident layers and the draft's int4 tiles on the GPU, streamed layers alias their pinned slabs
    assert model.model.layers[0].mlp.up_proj.weight.device.type == "cuda" and model.lm_head.weight.device.type == "cuda"
    assert model.model.layers[3].mlp.up_proj.weight.device.type == "cpu" and model.model.layers[3].mlp.up_proj.weight.is_pinned()
    assert isinstance(draft.model.model.layers[3].self_attn.q_proj, HqqInt4Linear)
    assert draft.model.model.layers[3].self_attn.q_proj.wq.device.type == "cuda"
    kv, draft_kv = entry.load_kv_cache_fn(b, model, draft)
    assert draft_kv is None
    gen = resolve(entry.generator_cls)(target_model=model, tokenizer=tokenizer, draft_model=draft, draft_params=b.draft_params,
                                       cache_implementation="static", profiling=True, profiling_verbose=False,
                                       generator_kwargs=dict({"verify_method": "exact", "prefill_chunk_size": 16},
                                                             **({"postspec_steps": 2} if method.endswith("v2") else {}))).eval()
    prompt = torch.randint(0, HF["vocab_size"], (1, 32), generator=torch.Generator().manual_seed(4)).to(DEV)
    wandb_logger.clear_log_data()
    print("seam:", method, "generate", flush=True)
    out = gen.generate(prompt, max_new_tokens=40, do_sample=False, past_key_values=kv)[0].cpu()
    log = dict(wandb_logger.log_data)
    assert out.numel() == 72 and kv.get_seq_length() == 71 and log["n_tokens"] == 40
    assert off.streamer.bytes_streamed > 0 and gen.target_model.streamer is off.streamer
    assert gen.target_model.native_layers and gen.draft_model.decoder.native_layers
    _greedy_continuation(path, out, 32, method)
    # a second generate() over a fresh cache re-binds the same decoders
    kv2, _ = entry.load_kv_cache_fn(b, model, draft)
    out2 = gen.generate(prompt, max_new_tokens=40, do_sample=False, past_key_values=kv2)[0].cpu()
    assert torch.equal(out, out2)
