"""Oracle: tree-masked GQA attention.  Test infrastructure only.

Follows what the reference executes for one tree-decoding forward
(specdecodes/models/generators/classic_sd.py:57-109 under run/pipelines/run_test.py:64):
HF ``sdpa_attention_forward`` on the math backend = ``repeat_kv`` + scaled-dot-product attention
with the additive mask ``(~allowed) * finfo.min`` over the whole static cache; the allowed set of
tree row i is the prefix plus ancestor-or-self slots (cpu_tree.py:263-286), everything beyond
prefix + n is masked (generators/classic_sd.py:33-55).  Evaluated in fp32 on the bf16/fp16 inputs.
"""
import torch
import torch.nn.functional as F


def allowed_mask(parents, prefix_len: int, cache_len: int) -> torch.Tensor:
    """bool [n, cache_len]: brute-force ancestor closure from the parent array."""
    n = len(parents)
    m = torch.zeros(n, cache_len, dtype=torch.bool)
    m[:, :prefix_len] = True
    for i in range(n):
        j = i
        while j >= 0:
            m[i, prefix_len + j] = True
            j = int(parents[j])
    return m


def tree_attention(q, k_cache, v_cache, parents, prefix_len: int, scale=None):
    """q [B, Hq, n, D], caches [B, Hkv, S, D] -> [B, n, Hq*D] (fp32), explicit softmax(QK^T)V."""
    B, Hq, n, D = q.shape
    Hkv, S = k_cache.shape[1], k_cache.shape[2]
    rep = Hq // Hkv
    k = k_cache.float().repeat_interleave(rep, dim=1)
    v = v_cache.float().repeat_interleave(rep, dim=1)
    scale = D ** -0.5 if scale is None else scale
    allowed = allowed_mask(parents, prefix_len, S)
    add = (~allowed).float() * torch.finfo(torch.float32).min
    scores = torch.matmul(q.float(), k.transpose(-1, -2)) * scale + add
    o = torch.matmul(torch.softmax(scores, dim=-1), v)
    return o.transpose(1, 2).reshape(B, n, Hq * D)


def tree_attention_sdpa(q, k_cache, v_cache, parents, prefix_len: int, scale=None):
    """The same through the library routine the reference calls."""
    B, Hq, n, D = q.shape
    Hkv, S = k_cache.shape[1], k_cache.shape[2]
    rep = Hq // Hkv
    k = k_cache.float().repeat_interleave(rep, dim=1)
    v = v_cache.float().repeat_interleave(rep, dim=1)
    add = (~allowed_mask(parents, prefix_len, S)).float() * torch.finfo(torch.float32).min
    o = F.scaled_dot_product_attention(q.float(), k, v, attn_mask=add[None, None], scale=scale)
    return o.transpose(1, 2).reshape(B, n, Hq * D)
