"""Pins ``oracle/decoder.py`` against the library the reference actually runs: a HuggingFace Qwen2
decoder (transformers, random weights, nothing downloaded) called the way
``ClassicSDGeneratorBase._tree_decoding`` calls it (specdecodes/models/generators/classic_sd.py:75-109):
tree tokens as one sequence, ``position_ids = prefix + depth``, an additive 4-D mask that opens the
whole prefix and, among the tree slots, the row's own node and its ancestors
(cpu_tree.py:263-286 with ``invert=True``), on top of a KV cache holding the prefix.  fp32 on the CPU.
No GPU."""
import pytest
import torch

from oracle import decoder as od

transformers = pytest.importorskip("transformers")
from transformers import Qwen2Config, Qwen2ForCausalLM  # noqa: E402
from transformers.cache_utils import DynamicCache  # noqa: E402

H, F, HQ, HKV, D, V, LAYERS = 256, 512, 2, 1, 128, 512, 2


def hf_model(seed):
    torch.manual_seed(seed)
    cfg = Qwen2Config(vocab_size=V, hidden_size=H, intermediate_size=F, num_hidden_layers=LAYERS, num_attention_heads=HQ,
                      num_key_value_heads=HKV, max_position_embeddings=512, rope_theta=1e6, rms_norm_eps=1e-6,
                      tie_word_embeddings=False)
    cfg._attn_implementation = "eager"
    model = Qwen2ForCausalLM(cfg).eval()
    with torch.no_grad():                                   # norm weights away from their init of exactly 1
        for layer in model.model.layers:
            layer.input_layernorm.weight.mul_(1 + 0.3 * torch.randn(H))
            layer.post_attention_layernorm.weight.mul_(1 + 0.3 * torch.randn(H))
            for proj in (layer.self_attn.q_proj, layer.self_attn.k_proj, layer.self_attn.v_proj):
                proj.bias.normal_(0, 0.1)
    return model


def oracle_weights(model, i):
    sd = {k: v.detach().float() for k, v in model.state_dict().items()}
    pre = f"model.layers.{i}."
    return {"input_norm": sd[pre + "input_layernorm.weight"], "post_norm": sd[pre + "post_attention_layernorm.weight"],
            "qkv": torch.cat([sd[pre + f"self_attn.{n}_proj.weight"] for n in "qkv"]),
            "qkv_bias": torch.cat([sd[pre + f"self_attn.{n}_proj.bias"] for n in "qkv"]),
            "o": sd[pre + "self_attn.o_proj.weight"],
            "gate_up": torch.cat([sd[pre + "mlp.gate_proj.weight"], sd[pre + "mlp.up_proj.weight"]]),
            "down": sd[pre + "mlp.down_proj.weight"]}


def oracle_forward(model, tokens, positions, rows, anc_bits, prefix_len, caches):
    """Embedding -> all layers through the oracle -> hidden states per layer (before the final norm)."""
    x = model.model.embed_tokens.weight.detach().float()[tokens]
    hidden = [x]
    for i in range(LAYERS):
        x = od.decoder_layer(x, oracle_weights(model, i), caches[i][0], caches[i][1], positions, rows, anc_bits, prefix_len,
                             HQ, HKV, D, 1e-6, 1e6)
        hidden.append(x)
    return hidden


def tree_mask(parents, prefix):
    n = len(parents)
    mask = torch.full((1, 1, n, prefix + n), torch.finfo(torch.float32).min)
    mask[..., :prefix] = 0
    bits = []
    for i in range(n):
        j, b = i, 0
        while j >= 0:
            mask[0, 0, i, prefix + j] = 0
            b |= 1 << j
            j = parents[j]
        bits.append(b)
    return mask, bits


@pytest.mark.parametrize("seed", [0, 1])
def test_oracle_layer_equals_huggingface_qwen2_on_a_tree(seed):
    model = hf_model(seed)
    g = torch.Generator().manual_seed(seed)
    P = 11
    prefix = torch.randint(0, V, (P,), generator=g)
    parents = [-1, 0, 0, 1, 1, 2, 3, 3, 6]
    depth = [0, 1, 1, 2, 2, 2, 3, 3, 4]
    n = len(parents)
    tree = torch.randint(0, V, (n,), generator=g)
    mask, bits = tree_mask(parents, P)
    with torch.no_grad():
        cache = DynamicCache()
        pre = model(prefix[None], past_key_values=cache, use_cache=True, output_hidden_states=True)
        out = model(tree[None], past_key_values=cache, attention_mask=mask,
                    position_ids=torch.tensor([[P + d for d in depth]]), cache_position=torch.arange(P, P + n),
                    output_hidden_states=True, use_cache=True)
    # the oracle: prefix as a chain (row i sees slots 0..i, prefix length 0), then the tree rows
    caches = [(torch.zeros(HKV, 64, D), torch.zeros(HKV, 64, D)) for _ in range(LAYERS)]
    chain_bits = [(1 << (i + 1)) - 1 for i in range(P)]
    hid_pre = oracle_forward(model, prefix, torch.arange(P), torch.arange(P), chain_bits, 0, caches)
    hid = oracle_forward(model, tree, torch.tensor([P + d for d in depth]), torch.arange(P, P + n), bits, P, caches)
    for i in range(LAYERS):
        assert torch.allclose(hid_pre[i], pre.hidden_states[i][0], atol=2e-4, rtol=1e-4), ("prefix", i)
    for i in range(LAYERS):                                 # hidden_states[LAYERS] is post-norm in transformers
        assert torch.allclose(hid[i], out.hidden_states[i][0], atol=2e-4, rtol=1e-4), ("tree", i)
    final = od.rms_norm(hid[LAYERS], model.model.norm.weight.detach(), 1e-6)
    assert torch.allclose(final, out.hidden_states[LAYERS][0], atol=2e-4, rtol=1e-4)
    logits = final @ model.lm_head.weight.detach().T
    assert torch.allclose(logits, out.logits[0], atol=5e-4, rtol=1e-4)
    # the K / V rows the oracle wrote are the ones HuggingFace cached (rotary applied to K, V untouched)
    for i in range(LAYERS):
        layer = cache.layers[i] if hasattr(cache, "layers") else None
        keys = layer.keys if layer is not None else cache.key_cache[i]
        vals = layer.values if layer is not None else cache.value_cache[i]
        assert torch.allclose(caches[i][0][:, :P + n], keys[0], atol=2e-4, rtol=1e-4)
        assert torch.allclose(caches[i][1][:, :P + n], vals[0], atol=2e-4, rtol=1e-4)


def test_a_wrong_mask_or_position_is_detected():
    """The comparison above has teeth: siblings leaking into each other or depth-less positions change the result."""
    model = hf_model(3)
    g = torch.Generator().manual_seed(3)
    P, parents, depth = 5, [-1, 0, 0, 1], [0, 1, 1, 2]
    n = len(parents)
    prefix, tree = torch.randint(0, V, (P,), generator=g), torch.randint(0, V, (n,), generator=g)
    mask, bits = tree_mask(parents, P)
    with torch.no_grad():
        cache = DynamicCache()
        model(prefix[None], past_key_values=cache, use_cache=True)
        out = model(tree[None], past_key_values=cache, attention_mask=mask, position_ids=torch.tensor([[P + d for d in depth]]),
                    cache_position=torch.arange(P, P + n), output_hidden_states=True, use_cache=True)
    ref = out.hidden_states[1][0]

    def run(bits_, positions):
        caches = [(torch.zeros(HKV, 64, D), torch.zeros(HKV, 64, D)) for _ in range(LAYERS)]
        oracle_forward(model, prefix, torch.arange(P), torch.arange(P), [(1 << (i + 1)) - 1 for i in range(P)], 0, caches)
        return oracle_forward(model, tree, positions, torch.arange(P, P + n), bits_, P, caches)[1]

    good = run(bits, torch.tensor([P + d for d in depth]))
    assert torch.allclose(good, ref, atol=2e-4, rtol=1e-4)
    causal = [(1 << (i + 1)) - 1 for i in range(n)]          # node 2 would see its sibling 1
    assert not torch.allclose(run(causal, torch.tensor([P + d for d in depth])), ref, atol=2e-3, rtol=1e-3)
    assert not torch.allclose(run(bits, torch.arange(P, P + n)), ref, atol=2e-3, rtol=1e-3)   # slot index instead of depth
