"""TEST INFRASTRUCTURE ONLY (CPU oracle).  fp32 restatement of one decoder layer of the substitute
draft: the HuggingFace Qwen2 layer whose projections are the affine int4 linears installed by
``HqqQuantizer.quantize_model`` (specdecodes/helpers/quantizers/hqq/__init__.py:17-120, recipe
``specdecodes/helpers/recipes/subspec/hqq_4bit_postspec.py:17-58``), evaluated on tree rows with the
ancestor mask of ``cpu_tree.py:263-286``.  Everything is float32 on dequantized weights; the device
layer rounds intermediates to bf16, so comparisons use a relative tolerance.

Pinned by: the HuggingFace Qwen2 decoder itself (transformers is importable in the build image; a small
random-weight model, nothing downloaded), called as the reference calls it -- prefix in a KV cache, tree tokens
with ``position_ids = prefix + depth`` and the additive ancestor mask (generators/classic_sd.py:75-109): hidden
states of every layer, final logits and the cached K / V rows agree to 2e-4 in fp32
(tests/test_oracle_hf_layer.py, which also shows that a causal mask or slot-index positions are detected);
plus closed forms (rotary is a rotation, identity at position 0, relative).
"""
import torch


def rms_norm(x, w, eps):
    return w * (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps))


def rope(t, positions, theta):
    """t [n, heads, D], rotate-half form."""
    D = t.shape[-1]
    inv = 1.0 / (theta ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    ang = torch.outer(positions.float(), inv)
    cos, sin = torch.cat([ang, ang], -1).cos()[:, None], torch.cat([ang, ang], -1).sin()[:, None]
    rot = torch.cat([-t[..., D // 2:], t[..., :D // 2]], -1)
    return t * cos + rot * sin


def decoder_layer(x, w, k_cache, v_cache, positions, cache_rows, anc_bits, prefix_len, n_q_heads, n_kv_heads, head_dim,
                  eps, theta):
    """x [n, H] fp32; w: dict of fp32 dense weights (qkv [Q+2KV, H] + bias, o, gate_up [2F, H], down) and norm
    weights; k_cache / v_cache [Hkv, S, D] fp32, updated in place at cache_rows; anc_bits: python ints
    over tree slots (any number of slots).  Returns the new x."""
    n = x.shape[0]
    Q, KV = n_q_heads * head_dim, n_kv_heads * head_dim
    h = rms_norm(x, w["input_norm"], eps)
    qkv = h @ w["qkv"].T + (w["qkv_bias"] if w.get("qkv_bias") is not None else 0)
    q, k, v = qkv.split([Q, KV, KV], -1)
    q = rope(q.reshape(n, n_q_heads, head_dim), positions, theta)
    k = rope(k.reshape(n, n_kv_heads, head_dim), positions, theta)
    v = v.reshape(n, n_kv_heads, head_dim)
    k_cache[:, cache_rows] = k.transpose(0, 1)
    v_cache[:, cache_rows] = v.transpose(0, 1)
    rep = n_q_heads // n_kv_heads
    out = torch.zeros(n, n_q_heads, head_dim)
    if n <= 64:
        for i in range(n):
            keys = list(range(prefix_len)) + [prefix_len + j for j in range(int(anc_bits[i]).bit_length()) if (anc_bits[i] >> j) & 1]
            for hq in range(n_q_heads):
                kk, vv = k_cache[hq // rep, keys], v_cache[hq // rep, keys]
                p = torch.softmax(kk @ q[i, hq] / head_dim ** 0.5, 0)
                out[i, hq] = p @ vv
    else:
        # the same sums for many rows at once: scores of every row against prefix + slots, the keys a row may not see at
        # -inf (tests/test_oracle_decoder.py holds this form against the loop above)
        slots = max(int(b).bit_length() for b in anc_bits)
        allowed = torch.zeros(n, prefix_len + slots, dtype=torch.bool)
        allowed[:, :prefix_len] = True
        for i in range(n):
            for j in range(int(anc_bits[i]).bit_length()):
                if (anc_bits[i] >> j) & 1:
                    allowed[i, prefix_len + j] = True
        for hq in range(n_q_heads):
            kk, vv = k_cache[hq // rep, :prefix_len + slots], v_cache[hq // rep, :prefix_len + slots]
            s = (q[:, hq] @ kk.T / head_dim ** 0.5).masked_fill(~allowed, float("-inf"))
            out[:, hq] = torch.softmax(s, -1) @ vv
    x = x + out.reshape(n, Q) @ w["o"].T
    h = rms_norm(x, w["post_norm"], eps)
    gate, up = (h @ w["gate_up"].T).chunk(2, -1)
    return x + (torch.nn.functional.silu(gate) * up) @ w["down"].T
