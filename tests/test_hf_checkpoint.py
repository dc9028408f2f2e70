"""CPU: ingestion of a local HuggingFace-style checkpoint directory (config.json + safetensors) into the
fused layer layout.  The checkpoint is written by the test itself with the Qwen2 / Llama tensor names."""
import json
import os

import pytest
import torch
from safetensors.torch import save_file

from subspec_amd.model import config_from_hf, layer_shapes, load_hf_checkpoint

HF = {"num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
      "intermediate_size": 96, "vocab_size": 50, "rms_norm_eps": 1e-5, "rope_theta": 10000.0,
      "max_position_embeddings": 128}


def _write(tmp_path, qkv_bias: bool, tied: bool, shards: int = 2):
    g = torch.Generator().manual_seed(0)
    H, D = HF["hidden_size"], HF["hidden_size"] // HF["num_attention_heads"]
    Q, KV, F, V = HF["num_attention_heads"] * D, HF["num_key_value_heads"] * D, HF["intermediate_size"], HF["vocab_size"]
    t = {"model.embed_tokens.weight": torch.randn(V, H, generator=g), "model.norm.weight": torch.rand(H, generator=g)}
    if not tied:
        t["lm_head.weight"] = torch.randn(V, H, generator=g)
    for i in range(HF["num_hidden_layers"]):
        p = f"model.layers.{i}."
        t[p + "input_layernorm.weight"] = torch.rand(H, generator=g)
        t[p + "post_attention_layernorm.weight"] = torch.rand(H, generator=g)
        for n, rows in (("q", Q), ("k", KV), ("v", KV)):
            t[p + f"self_attn.{n}_proj.weight"] = torch.randn(rows, H, generator=g)
            if qkv_bias:
                t[p + f"self_attn.{n}_proj.bias"] = torch.randn(rows, generator=g)
        t[p + "self_attn.o_proj.weight"] = torch.randn(H, Q, generator=g)
        t[p + "mlp.gate_proj.weight"] = torch.randn(F, H, generator=g)
        t[p + "mlp.up_proj.weight"] = torch.randn(F, H, generator=g)
        t[p + "mlp.down_proj.weight"] = torch.randn(H, F, generator=g)
    t = {k: v.to(torch.bfloat16) for k, v in t.items()}
    keys = sorted(t)
    for s in range(shards):
        save_file({k: t[k] for k in keys[s::shards]}, os.path.join(tmp_path, f"model-{s:05d}-of-{shards:05d}.safetensors"))
    with open(os.path.join(tmp_path, "config.json"), "w") as f:
        json.dump(dict(HF, tie_word_embeddings=tied), f)
    return t


@pytest.mark.parametrize("qkv_bias,tied", [(True, False), (False, True)])
def test_load_fuses_projections(tmp_path, qkv_bias, tied):
    t = _write(str(tmp_path), qkv_bias, tied)
    cfg, w = load_hf_checkpoint(str(tmp_path))
    assert cfg == config_from_hf(HF) and cfg.head_dim == 16 and cfg.q_size == 64 and cfg.kv_size == 32
    assert len(w["layers"]) == 2
    for i, lw in enumerate(w["layers"]):
        p = f"model.layers.{i}."
        for name, shape in layer_shapes(cfg).items():
            assert tuple(lw[name].shape) == tuple(shape), name
        q, k, v = lw["qkv_proj.weight"].split([cfg.q_size, cfg.kv_size, cfg.kv_size], 0)
        assert torch.equal(q, t[p + "self_attn.q_proj.weight"]) and torch.equal(k, t[p + "self_attn.k_proj.weight"])
        assert torch.equal(v, t[p + "self_attn.v_proj.weight"])
        gate, up = lw["gate_up_proj.weight"].chunk(2, 0)
        assert torch.equal(gate, t[p + "mlp.gate_proj.weight"]) and torch.equal(up, t[p + "mlp.up_proj.weight"])
        assert torch.equal(lw["o_proj.weight"], t[p + "self_attn.o_proj.weight"])
        assert torch.equal(lw["down_proj.weight"], t[p + "mlp.down_proj.weight"])
        if qkv_bias:
            assert torch.equal(lw["qkv_proj.bias"][:cfg.q_size], t[p + "self_attn.q_proj.bias"])
            assert torch.equal(lw["qkv_proj.bias"][-cfg.kv_size:], t[p + "self_attn.v_proj.bias"])
        else:
            assert int(lw["qkv_proj.bias"].abs().sum()) == 0
    assert torch.equal(w["embed"], t["model.embed_tokens.weight"]) and torch.equal(w["norm"], t["model.norm.weight"])
    assert torch.equal(w["lm_head"], t["model.embed_tokens.weight"] if tied else t["lm_head.weight"])


def test_missing_tensor_and_wrong_shape_are_reported(tmp_path):
    t = _write(str(tmp_path), True, False, shards=1)
    fn = os.path.join(str(tmp_path), "model-00000-of-00001.safetensors")
    broken = dict(t)
    del broken["model.layers.1.mlp.down_proj.weight"]
    save_file(broken, fn)
    with pytest.raises(KeyError):
        load_hf_checkpoint(str(tmp_path))
    broken = dict(t)
    broken["model.layers.0.self_attn.o_proj.weight"] = torch.zeros(8, 8, dtype=torch.bfloat16)
    save_file(broken, fn)
    with pytest.raises(ValueError):
        load_hf_checkpoint(str(tmp_path))
    os.remove(fn)
    with pytest.raises(FileNotFoundError):
        load_hf_checkpoint(str(tmp_path))
