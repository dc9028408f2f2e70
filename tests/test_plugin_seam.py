"""CPU: the Python plug-in seam behind the reference's pipeline builder -- recipe classes resolved from
``class_path`` strings, the quantizer and offloader call conventions, the three loader functions and the registry
call -- exercised in the order run/core/builder.py:318-350 calls them, on a tiny checkpoint the test writes itself.
The reference is not imported; its lazy ``"module:Symbol"`` resolution (run/core/registry.py:8-34) and its
``ModelRegistry.register`` keyword names are restated by two small stand-ins."""
import importlib
import json
import os
from types import SimpleNamespace

import pytest
import torch
import torch.nn as nn
from safetensors.torch import save_file

from subspec_amd import quant
from subspec_amd.hf_model import CausalLM, layer_tensors, share_parameters
from subspec_amd.model import load_hf_checkpoint, quantize_layers
from subspec_amd.offloaders import Offloader, PrefetchOffloader, _uncovered
from subspec_amd.quant import HqqInt4Linear
from subspec_amd import registry as R
from subspec_amd.utils import DraftParams

HF = {"model_type": "qwen2", "num_hidden_layers": 3, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
      "intermediate_size": 128, "vocab_size": 48, "rms_norm_eps": 1e-5, "rope_theta": 10000.0,
      "max_position_embeddings": 128, "tie_word_embeddings": False}


def write_checkpoint(path, hf=HF, seed=0):
    g = torch.Generator().manual_seed(seed)
    H, D = hf["hidden_size"], hf["hidden_size"] // hf["num_attention_heads"]
    Q, KV, F, V = hf["num_attention_heads"] * D, hf["num_key_value_heads"] * D, hf["intermediate_size"], hf["vocab_size"]
    t = {"model.embed_tokens.weight": torch.randn(V, H, generator=g), "model.norm.weight": torch.rand(H, generator=g) + 0.5,
         "lm_head.weight": torch.randn(V, H, generator=g)}
    for i in range(hf["num_hidden_layers"]):
        p = f"model.layers.{i}."
        t[p + "input_layernorm.weight"] = torch.rand(H, generator=g) + 0.5
        t[p + "post_attention_layernorm.weight"] = torch.rand(H, generator=g) + 0.5
        for n, rows in (("q", Q), ("k", KV), ("v", KV)):
            t[p + f"self_attn.{n}_proj.weight"] = torch.randn(rows, H, generator=g) * 0.1
            t[p + f"self_attn.{n}_proj.bias"] = torch.randn(rows, generator=g) * 0.1
        t[p + "self_attn.o_proj.weight"] = torch.randn(H, Q, generator=g) * 0.1
        t[p + "mlp.gate_proj.weight"] = torch.randn(F, H, generator=g) * 0.1
        t[p + "mlp.up_proj.weight"] = torch.randn(F, H, generator=g) * 0.1
        t[p + "mlp.down_proj.weight"] = torch.randn(H, F, generator=g) * 0.1
    t = {k: v.to(torch.bfloat16) for k, v in t.items()}
    save_file(t, os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(hf, f)
    return t


def resolve(spec: str):
    """``"some.module:Symbol"`` -> the symbol, as the reference resolves recipe class paths and lazy registry entries."""
    module_name, _, symbol = spec.partition(":")
    return getattr(importlib.import_module(module_name), symbol)


class StubRegistry:
    entries = {}

    @classmethod
    def register(cls, name, generator_cls, draft_model_cls, default_config=None, load_model_fn=None,
                 load_draft_model_fn=None, load_kv_cache_fn=None, needs_draft_kv_cache=True):
        cls.entries[name] = SimpleNamespace(generator_cls=generator_cls, draft_model_cls=draft_model_cls,
                                            default_config=default_config or {}, load_model_fn=load_model_fn,
                                            load_draft_model_fn=load_draft_model_fn, load_kv_cache_fn=load_kv_cache_fn,
                                            needs_draft_kv_cache=needs_draft_kv_cache)


def builder_stub(recipe, device="cpu", **kw):
    return SimpleNamespace(recipe=recipe, dtype=torch.bfloat16, device=device, cache_implementation="static", max_length=96,
                           draft_params=DraftParams(temperature=0.2, max_depth=3, topk_len=4), cpu_offload_gb=None, **kw)


def test_recipe_quantizer_and_loaders_in_builder_order(tmp_path):
    t = write_checkpoint(str(tmp_path))
    recipe = resolve("subspec_amd.recipes:Recipe")(keep_first_n_layers_on_gpu=1)
    b = builder_stub(recipe)
    StubRegistry.entries.clear()
    R.register(StubRegistry, recipe=recipe, llm_path=str(tmp_path))
    entry = StubRegistry.entries["subspec_sd"]
    assert entry.needs_draft_kv_cache is False and entry.default_config["recipe"] is recipe
    assert resolve(entry.generator_cls).__name__ == "SubSpecSDGenerator"
    assert resolve(StubRegistry.entries["subspec_sd_v2"].generator_cls).__name__ == "SubSpecSDGeneratorV2"
    assert resolve(entry.draft_model_cls).__name__ == "SubSpecSDDraftModel"

    # builder.load_model_and_tokenizer / load_draft_model
    model, tokenizer = entry.load_model_fn(b, str(tmp_path))
    assert tokenizer is None and isinstance(model, nn.Module) and model.device.type == "cpu"
    assert len(model.model.layers) == 3 and model.config.model_type == "qwen2" and model.model.config is model.config
    names = dict(model.named_parameters())
    assert set(names) == set(t), set(names) ^ set(t)
    assert all(torch.equal(names[k], t[k]) for k in t)
    draft = entry.load_draft_model_fn(b, model, tokenizer, None)
    assert draft.model is not model and draft.model.model.norm.weight is model.model.norm.weight
    assert draft.model.model.layers[0].self_attn.q_proj is not model.model.layers[0].self_attn.q_proj
    assert draft.model.model.layers[0].self_attn.q_proj.weight is model.model.layers[0].self_attn.q_proj.weight

    # recipe.generate_configurations: 7 projections per layer quantized in the draft; layers 1.. of the target on the CPU
    target_config, draft_config = recipe.generate_configurations(target_model=model, draft_model=draft, max_length=96,
                                                                 cpu_offload_gb=None, dtype=torch.bfloat16, device="cuda:0")
    qc = draft_config["quant_config"]
    assert len(qc) == 21 and "model.layers.2.mlp.down_proj" in qc
    assert qc["model.layers.0.self_attn.q_proj"]["weight_quant_params"] == {"nbits": 4, "group_size": 64, "axis": 1}
    dm = target_config["device_map"]
    assert dm["model.embed_tokens"] == "cuda:0" and dm["lm_head"] == "cuda:0" and dm["model.layers.0.mlp.up_proj"] == "cuda:0"
    assert dm["model.layers.1.self_attn.k_proj"] == "cpu" and dm["model.layers.2.mlp.down_proj"] == "cpu"
    assert dm["model.layers.2.input_layernorm"] == "cuda:0" and not _uncovered(model, dm)

    # recipe.apply_quantization(draft_model.model, ...): the draft's projections become int4, the target's stay dense
    recipe.apply_quantization(draft.model, qc, torch.bfloat16, "cpu")
    for i in range(3):
        la, lt = draft.model.model.layers[i], model.model.layers[i]
        for mod, ref in ((la.self_attn.k_proj, lt.self_attn.k_proj), (la.mlp.down_proj, lt.mlp.down_proj)):
            assert isinstance(mod, HqqInt4Linear) and isinstance(ref, nn.Linear) and not isinstance(ref, HqqInt4Linear)
    # fused int4 layer == the tiles of the separately quantized projections side by side (each projection is its own
    # tensor to the quantizer, as in the reference: the proximal refinement stops per tensor), and with the plain
    # min/max rule it also equals quantizing the fused dense matrix (groups run along the input dimension of one row)
    cfg, fused = load_hf_checkpoint(str(tmp_path))
    parts = {"qkv_proj": [f"self_attn.{n}_proj" for n in "qkv"], "o_proj": ["self_attn.o_proj"],
             "gate_up_proj": ["mlp.gate_proj", "mlp.up_proj"], "down_proj": ["mlp.down_proj"]}
    plain = share_parameters(model)
    quant.HqqQuantizer.quantize_model(plain, {k: dict(v, optimize=False) for k, v in qc.items()}, torch.bfloat16, "cpu")
    want_plain = quantize_layers(fused["layers"], optimize=False)
    for i in range(3):
        got = layer_tensors(draft.model.model.layers[i], cfg, "cpu", torch.bfloat16)
        got_plain = layer_tensors(plain.model.layers[i], cfg, "cpu", torch.bfloat16)
        for key, names in parts.items():
            packed = [quant.pack_tiled(*quant.quantize_int4_g64(t[f"model.layers.{i}.{n}.weight"], optimize=True)) for n in names]
            assert torch.equal(got[key + ".wq"], torch.cat([p[0] for p in packed], 0)), (i, key)
            assert torch.equal(got[key + ".sz"], torch.cat([p[1] for p in packed], 0)), (i, key)
            assert got[key + ".out_features"] == want_plain[i][key + ".out_features"]
            assert torch.equal(got_plain[key + ".wq"], want_plain[i][key + ".wq"]), (i, key)
            assert torch.equal(got_plain[key + ".sz"], want_plain[i][key + ".sz"]), (i, key)
        assert torch.equal(got["qkv_proj.bias"], fused["layers"][i]["qkv_proj.bias"])
    # dense fused layout of the target == the checkpoint loader's, and the modules now alias the fused matrices
    got = layer_tensors(model.model.layers[0], cfg, "cpu", torch.bfloat16)
    for key, ref in fused["layers"][0].items():
        assert torch.equal(got[key], ref), key
    q = model.model.layers[0].self_attn.q_proj.weight
    assert q.data_ptr() == got["qkv_proj.weight"].data_ptr() and torch.equal(q, t["model.layers.0.self_attn.q_proj.weight"])

    # builder.load_kv_cache: one shared cache, max_length + the tree's rows
    kv, draft_kv = entry.load_kv_cache_fn(b, model, draft)
    assert draft_kv is None and kv.cache.max_cache_len == 96 + 13 and kv.get_seq_length() == 0
    assert kv.cache.data.shape == (3, 2, 1, 2, 109, 16)
    with pytest.raises(ValueError, match="max_length"):
        entry.load_kv_cache_fn(builder_stub(recipe, ) if False else SimpleNamespace(**dict(vars(b), max_length=None)), model, draft)

    # builder.load_generator: the reference's keyword arguments
    gen = resolve(entry.generator_cls)(target_model=model, tokenizer=tokenizer, draft_model=draft, draft_params=b.draft_params,
                                       cache_implementation="static", profiling=True, profiling_verbose=False,
                                       generator_kwargs={"verify_method": "lossy", "verify_kwargs": {"threshold": 0.3}})
    assert gen.eval() is gen and draft.draft_params is b.draft_params
    with pytest.raises(RuntimeError, match="GPU"):            # weights on the CPU: no CPU path, and it says so
        gen.generate(torch.zeros(1, 4, dtype=torch.long), max_new_tokens=2, past_key_values=kv)


def test_layer_offload_recipe_and_quantizer_config_forms(tmp_path):
    write_checkpoint(str(tmp_path))
    recipe = resolve("subspec_amd.recipes:LayerOffloadRecipe")(keep_first_n_layers_on_gpu=2)
    assert recipe.quantizer is None and recipe.offloader is Offloader
    model = CausalLM.from_pretrained(str(tmp_path))
    target_config, draft_config = recipe.generate_configurations(model, None, 64, None, torch.bfloat16, "cuda:0")
    assert draft_config is None and target_config["quant_config"] is None
    cpu = sorted(k for k, v in target_config["device_map"].items() if v == "cpu")
    assert len(cpu) == 7 and all(k.startswith("model.layers.2.") for k in cpu)
    assert recipe.apply_quantization(model, {}, torch.bfloat16, "cpu") is None           # no quantizer: skipped
    # quantizer: plain dict, hqq-shaped dict and attribute object are accepted; other bit widths are refused by name
    for cfgform in ({"nbits": 4, "group_size": 64, "axis": 1, "optimize": False},
                    {"weight_quant_params": {"nbits": 4, "group_size": 64, "axis": 1}},
                    SimpleNamespace(nbits=4, group_size=64, axis=1)):
        m = share_parameters(model)
        quant.HqqQuantizer.quantize_model(m, {"model.layers.0.mlp.up_proj": cfgform}, torch.bfloat16, "cpu")
        assert isinstance(m.model.layers[0].mlp.up_proj, HqqInt4Linear) and isinstance(model.model.layers[0].mlp.up_proj, nn.Linear)
    with pytest.raises(ValueError, match="model.layers.0.mlp.up_proj"):
        quant.HqqQuantizer.quantize_model(share_parameters(model), {"model.layers.0.mlp.up_proj": {"weight_quant_params": {"nbits": 8, "group_size": 64}}},
                                          torch.bfloat16, "cpu")
    # a fused matrix quantized in part cannot be expressed
    m = share_parameters(model)
    quant.HqqQuantizer.quantize_model(m, {"model.layers.0.self_attn.q_proj": {"nbits": 4}}, torch.bfloat16, "cpu")
    with pytest.raises(NotImplementedError, match="qkv_proj"):
        layer_tensors(m.model.layers[0], model.decoder_config, "cpu", torch.bfloat16)


def test_offloader_refuses_what_it_cannot_stream(tmp_path):
    write_checkpoint(str(tmp_path))
    model = CausalLM.from_pretrained(str(tmp_path))
    recipe = resolve("subspec_amd.recipes:Recipe")()
    dm = recipe.generate_configurations(model, None, 64, None, torch.bfloat16, "cuda:0")[0]["device_map"]
    assert sum(v == "cpu" for v in dm.values()) == 21                                       # every layer, as the reference's recipe
    with pytest.raises(ValueError, match="does not give any device"):
        PrefetchOffloader(model, device_map={k: v for k, v in dm.items() if k != "model.norm"})
    with pytest.raises(ValueError, match="map all seven or none"):
        PrefetchOffloader(model, device_map=dict(dm, **{"model.layers.1.mlp.up_proj": "cuda:0"}))
    resident_tail = dict(dm, **{k: "cuda:0" for k in dm if k.startswith("model.layers.2.")})
    with pytest.raises(ValueError, match="last layers"):
        PrefetchOffloader(model, device_map=resident_tail)
    with pytest.raises(ValueError, match="No CPU layer"):
        PrefetchOffloader(model, device_map={k: "cuda:0" for k in dm})
    with pytest.raises(ValueError, match="must sit on a GPU"):
        PrefetchOffloader(model, device_map={k: "cpu" if v == "cpu" else "cpu" for k, v in dm.items()})
    with pytest.raises(ValueError, match="only decoder-layer projections"):
        PrefetchOffloader(model, device_map=dict(dm, lm_head="cpu"))
