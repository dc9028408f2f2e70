"""Thin torch-tensor front ends of the C ABI: pointer extraction, shape checks, output allocation.

torch is used for device memory and the current stream only; all arithmetic happens in
libsubspec_hip.so.
"""
from __future__ import annotations

import ctypes
from typing import Dict, Optional

import torch

from . import _lib as L

_DT = {torch.float32: L.F32, torch.float16: L.F16, torch.bfloat16: L.BF16}


def _dtype_code(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {t.dtype}; expected float32, float16 or bfloat16") from None


def _require_gpu(*tensors: torch.Tensor) -> torch.device:
    dev = tensors[0].device
    for t in tensors:
        if t.device.type != "cuda":
            raise L.SubspecHipError("the HIP kernels need device tensors (no CPU fallback)")
        if t.device != dev:
            raise ValueError("all tensors must live on the same device")
    return dev


def _stream(dev: torch.device) -> int:
    return torch.cuda.current_stream(dev).cuda_stream


def tree_verify(
    logits: torch.Tensor,            # [B, rows, V] or [rows, V]
    token_ids: torch.Tensor,         # int32 [B, n] or [n], device
    parents: torch.Tensor,           # int32 [B, n] or [n], device
    *,
    root: int = 0,
    skip_nodes: int = 0,
    eos_token_id: Optional[int] = None,
    verify_method: str = "exact",
    threshold_method: str = "prob",
    threshold: float = 0.0,
    window_size: int = 1,
    exact_entropy: bool = False,
    workspace: Optional[torch.Tensor] = None,
    do_sample: bool = False,
    temperature: float = 1.0,
    seed: int = 0,
    offset: int = 0,
    out: Optional[Dict[str, torch.Tensor]] = None,
    static_scratch: bool = False,
    _prepared: Optional[list] = None,
) -> Dict[str, torch.Tensor]:
    """Runs the fused verifier; everything stays on the device (no synchronisation here).

    ``static_scratch=True`` calls ``subspec_tree_verify_static`` (greedy target only): the library's built-in scratch
    array takes the place of the workspace; with ``out`` (the dictionary an earlier call returned, same shapes)
    nothing at all is allocated.

    ``do_sample=True`` draws the target token of every row from ``softmax(logits / temperature)``
    (Philox stream ``seed`` / ``offset``) instead of taking the argmax.

    Returns device tensors: ``tokens`` / ``contexts`` int64 [B, n+1], ``counts`` int32 [B, 4]
    (emitted, accept_len, total_len, status) and the per-node ``target`` int64 / ``entropy`` /
    ``child_prob`` float32 [B, rows].
    """
    if logits.dim() == 2:
        logits = logits.unsqueeze(0)
    if token_ids.dim() == 1:
        token_ids, parents = token_ids.unsqueeze(0), parents.unsqueeze(0)
    if logits.dim() != 3 or token_ids.dim() != 2 or parents.shape != token_ids.shape:
        raise ValueError("expected logits [B, rows, V] and token_ids / parents [B, n]")
    dev = _require_gpu(logits, token_ids, parents)
    B, rows, V = logits.shape
    n = token_ids.shape[1]
    if token_ids.shape[0] != B:
        raise ValueError(f"batch mismatch: logits {B} vs tree arrays {token_ids.shape[0]}")
    method = {"exact": L.VERIFY_EXACT, "lossy": L.VERIFY_LOSSY}.get(str(verify_method or "exact").strip().lower())
    if method is None:
        raise ValueError(f"Unsupported verify_method: {verify_method!r} (supported: 'exact', 'lossy')")
    gate = {"entropy": L.GATE_ENTROPY, "prob": L.GATE_PROB}.get(str(threshold_method or "entropy").strip().lower())
    if gate is None:
        raise ValueError(f"Unsupported threshold_method: {threshold_method!r} (supported: 'entropy', 'prob')")
    logits = logits.contiguous()
    token_ids = token_ids.to(torch.int32).contiguous()
    parents = parents.to(torch.int32).contiguous()
    lib = L.lib()
    if static_scratch and do_sample:
        raise ValueError("static_scratch serves the greedy verifier only")
    if workspace is None and not static_scratch:
        need = lib.subspec_tree_verify_workspace(B, rows, V, _dtype_code(logits))
        workspace = torch.empty(need, dtype=torch.uint8, device=dev)
    if out is not None:
        want = {"tokens": ((B, n + 1), torch.int64), "contexts": ((B, n + 1), torch.int64), "counts": ((B, 4), torch.int32),
                "target": ((B, rows), torch.int64), "entropy": ((B, rows), torch.float32), "child_prob": ((B, rows), torch.float32)}
        for key, (shape, dtype) in want.items():
            # the kernels write these element types: a narrower tensor of the right shape would be overrun
            if (tuple(out[key].shape) != shape or out[key].dtype != dtype or out[key].device != dev
                    or not out[key].is_contiguous()):
                raise ValueError(f"out[{key!r}] must be a contiguous {dtype} tensor of shape {shape} on {dev}")
    out = out if out is not None else {
        "tokens": torch.empty((B, n + 1), dtype=torch.int64, device=dev),
        "contexts": torch.empty((B, n + 1), dtype=torch.int64, device=dev),
        "counts": torch.empty((B, 4), dtype=torch.int32, device=dev),
        "target": torch.empty((B, rows), dtype=torch.int64, device=dev),
        "entropy": torch.empty((B, rows), dtype=torch.float32, device=dev),    # every row is written (0 without the entropy gate)
        "child_prob": torch.empty((B, rows), dtype=torch.float32, device=dev),
    }
    head = (logits.data_ptr(), _dtype_code(logits), B, rows, V, token_ids.data_ptr(), parents.data_ptr(), n,
            int(root), int(skip_nodes), -1 if eos_token_id is None else int(eos_token_id),
            method, gate, float(threshold), int(window_size),
            L.ENTROPY_ALWAYS if exact_entropy else L.ENTROPY_GUARD)
    outs = (out["tokens"].data_ptr(), out["contexts"].data_ptr(), out["counts"].data_ptr(),
            out["target"].data_ptr(), out["entropy"].data_ptr(), out["child_prob"].data_ptr(), _stream(dev))
    if static_scratch:
        name, args = "subspec_tree_verify_static", (*head, *outs)
    else:
        tail = (workspace.data_ptr(), workspace.numel() * workspace.element_size(), *outs)
        if do_sample:
            mask = (1 << 64) - 1
            name, args = "subspec_tree_verify_sample", (*head, float(temperature), int(seed) & mask, int(offset) & mask, *tail)
        else:
            name, args = "subspec_tree_verify", (*head, *tail)
    if _prepared is not None:                            # PreparedTreeVerify: the caller launches, and keeps the tensors alive
        _prepared.extend((name, args, out, (logits, token_ids, parents, workspace)))
        return out
    L.check(getattr(lib, name)(*args), name)
    return out


class PreparedTreeVerify:
    """A ``tree_verify`` call whose checks, conversions and argument marshalling are done once.

    A decoding loop verifies into the same tensors cycle after cycle (the reference keeps static buffers for the same
    reason when it captures its draft step, draft_models/subspec_sd_fi.py:65-179): ``PreparedTreeVerify(logits,
    token_ids, parents, **kwargs)`` takes what ``tree_verify`` takes, allocates the workspace and the outputs once and
    holds references to all of them; every ``call()`` then only launches, on the stream that was current when the
    object was made, and returns the same output dictionary.  The tensors are read where they are: the caller writes
    new logits / tokens / parents INTO them between calls.  64 x 152064 fp32 rows: 12.6 us per call against 18 to 20
    through ``tree_verify(out=...)`` and 26 to 28 when the outputs are allocated per call.
    """

    def __init__(self, logits: torch.Tensor, token_ids: torch.Tensor, parents: torch.Tensor, **kwargs):
        if token_ids.dtype != torch.int32 or parents.dtype != torch.int32:
            raise ValueError("PreparedTreeVerify reads token_ids / parents in place: they must be int32 tensors")
        if not (logits.is_contiguous() and token_ids.is_contiguous() and parents.is_contiguous()):
            raise ValueError("PreparedTreeVerify reads its inputs in place: they must be contiguous")
        parts: list = []
        tree_verify(logits, token_ids, parents, _prepared=parts, **kwargs)
        self._name, args, self.out, self._keep = parts
        fn = getattr(L.lib(), self._name)
        self._fn = fn
        # converted once: ctypes would otherwise convert all 27 arguments on every call
        self._args = tuple(t(a) for t, a in zip(fn.argtypes, args))

    def call(self) -> Dict[str, torch.Tensor]:
        code = self._fn(*self._args)
        if code != 0:
            L.check(code, self._name)
        return self.out

    __call__ = call


def sample_tokens(logits: torch.Tensor, temperature: float = 1.0, seed: int = 0, offset: int = 0) -> torch.Tensor:
    """One token per row of ``logits [rows, V]`` drawn from ``softmax(logits / temperature)`` (rounded to the
    logits dtype) with the verifier's Philox race: ``GeneratorBase._sample_token(do_sample=True)`` for
    the rows outside a tree, e.g. the first token after the prefill
    (specdecodes/models/generators/base.py:116-132).  Returns int64 ``[rows]`` on the device."""
    lg = logits.reshape(-1, logits.shape[-1])
    rows = lg.shape[0]
    if rows > L.MAX_TREE_NODES:
        raise ValueError(f"at most {L.MAX_TREE_NODES} rows per call")
    # a parentless forest: no node has children, so the verifier only reports each row's draw
    tok = torch.zeros(rows, dtype=torch.int32, device=lg.device)
    par = torch.full((rows,), -1, dtype=torch.int32, device=lg.device)
    out = tree_verify(lg, tok, par, do_sample=True, temperature=temperature, seed=seed, offset=offset)
    return out["target"][0]


def kv_compact_(
    cache: torch.Tensor,             # [..., seq, head_dim], contiguous; every leading index is a slab
    contexts: torch.Tensor,          # int64 device tensor, kept rows relative to `offset`
    offset: int,
    count: Optional[int] = None,
    count_dev: Optional[torch.Tensor] = None,
    max_count: Optional[int] = None,
) -> torch.Tensor:
    """In place: ``cache[..., offset + j, :] = cache[..., offset + contexts[j], :]`` for j < count."""
    dev = _require_gpu(cache, contexts)
    if not cache.is_contiguous():
        raise ValueError("kv_compact_: cache must be contiguous")
    if contexts.dtype != torch.int64 or not contexts.is_contiguous():
        raise ValueError("kv_compact_: contexts must be a contiguous int64 tensor")
    seq, hd = cache.shape[-2], cache.shape[-1]
    row_bytes = hd * cache.element_size()
    n_slabs = cache.numel() // (seq * hd)
    if count_dev is None:
        count = int(contexts.numel()) if count is None else int(count)
    else:
        _require_gpu(count_dev)
        if count_dev.dtype != torch.int32:
            raise ValueError("kv_compact_: count_dev must be int32")
        count = 0
    if max_count is None:
        max_count = min(int(contexts.numel()), L.MAX_TREE_NODES) if count_dev is not None else count
    code = L.lib().subspec_kv_compact(
        cache.data_ptr(), None, n_slabs, seq * row_bytes, seq, row_bytes, int(offset), contexts.data_ptr(),
        None if count_dev is None else count_dev.data_ptr(), count, int(max_count), _stream(dev))
    L.check(code, "subspec_kv_compact")
    return cache


def topk_expand(sampled_probs: torch.Tensor, parent_probs: torch.Tensor, k: int,
                workspace: Optional[torch.Tensor] = None):
    """Global top-k over (leaves x vocab) of ``round(sampled_probs * parent_probs[..., None])``.

    ``sampled_probs`` [B, L, V], ``parent_probs`` [B, L] (same dtype).  Returns
    ``(token_ids int64 [B, k], topk_probs dtype [B, k], parent_indices int64 [B, k])`` on the device,
    sorted by value descending, equal values by flat index ascending.
    """
    if sampled_probs.dim() != 3 or parent_probs.shape != sampled_probs.shape[:2]:
        raise ValueError("expected sampled_probs [B, L, V] and parent_probs [B, L]")
    if parent_probs.dtype != sampled_probs.dtype:
        raise ValueError("sampled_probs and parent_probs must share a dtype")
    dev = _require_gpu(sampled_probs, parent_probs)
    B, Lv, V = sampled_probs.shape
    k = min(int(k), int(V))
    sampled_probs = sampled_probs.contiguous()
    parent_probs = parent_probs.contiguous()
    lib = L.lib()
    need = lib.subspec_topk_expand_workspace(B, Lv, V, k)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=dev)
    token_ids = torch.empty((B, k), dtype=torch.int64, device=dev)
    parents = torch.empty((B, k), dtype=torch.int64, device=dev)
    vals = torch.empty((B, k), dtype=sampled_probs.dtype, device=dev)
    code = lib.subspec_topk_expand(
        sampled_probs.data_ptr(), parent_probs.data_ptr(), _dtype_code(sampled_probs), B, Lv, V, k,
        workspace.data_ptr(), workspace.numel() * workspace.element_size(),
        token_ids.data_ptr(), vals.data_ptr(), parents.data_ptr(), _stream(dev))
    L.check(code, "subspec_topk_expand")
    return token_ids, vals, parents


def bits_to_words(bits, n_slots: int, device=None) -> torch.Tensor:
    """Python-int bitsets -> int64 tensor [n] (up to 64 slots) or [n, ceil(n_slots / 64)]: bit j of a row is
    bit j % 64 of word j // 64."""
    def signed(w):
        return w - (1 << 64) if w >= (1 << 63) else w
    mask = (1 << 64) - 1
    if n_slots <= 64:
        return torch.tensor([signed(int(b) & mask) for b in bits], dtype=torch.int64, device=device)
    if n_slots > L.MAX_TREE_NODES:
        raise ValueError(f"{n_slots} tree slots exceed the {L.MAX_TREE_NODES} the attention kernel masks")
    words = (n_slots + 63) // 64
    return torch.tensor([[signed((int(b) >> (64 * w)) & mask) for w in range(words)] for b in bits], dtype=torch.int64,
                        device=device)


def ancestor_bits_tensor(parents, device=None) -> torch.Tensor:
    """uint64 ancestor-or-self bitsets (as an int64 tensor, [n] or [n, ceil(n / 64)] above 64 nodes) from a parent
    array with parent < child."""
    bits = []
    for i, p in enumerate(parents):
        v = (1 << i) | (bits[int(p)] if int(p) >= 0 else 0)
        bits.append(v)
    return bits_to_words(bits, len(bits), device)


def tree_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, anc_bits: torch.Tensor,
                   prefix_len: int, scale: Optional[float] = None, workspace: Optional[torch.Tensor] = None,
                   n_tree_slots: Optional[int] = None):
    """``q`` [B, Hq, n, D], caches [B, Hkv, S, D] (tree K/V already written at rows prefix_len..),
    ``anc_bits`` int64 [n] (shared tree) or [B, n], with a trailing dimension of ceil(slots / 64) words when
    more than 64 tree slots are occupied: bit j = row may attend to tree slot j.  ``n_tree_slots`` (default n) is
    the number of occupied tree slots (<= 512); n may be as large (windows of 64 rows inside one launch).  Returns [B, n, Hq * D]."""
    dev = _require_gpu(q, k_cache, v_cache, anc_bits)
    if q.dim() != 4 or k_cache.dim() != 4 or v_cache.shape != k_cache.shape:
        raise ValueError("expected q [B, Hq, n, D] and k/v caches [B, Hkv, S, D]")
    if q.dtype != k_cache.dtype or q.dtype != v_cache.dtype:
        raise ValueError("q, k_cache and v_cache must share a dtype")
    B, Hq, n, D = q.shape
    Hkv, S = k_cache.shape[1], k_cache.shape[2]
    if k_cache.shape[0] != B or k_cache.shape[3] != D:
        raise ValueError("cache shape does not match q")
    if not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise ValueError("tree_attention: the KV caches must be contiguous [B, Hkv, S, D]")
    slots = n if n_tree_slots is None else int(n_tree_slots)
    words = (slots + 63) // 64
    rows_shape = anc_bits.shape[:-1] if words > 1 else anc_bits.shape       # [n] or [B, n]
    if anc_bits.dtype != torch.int64 or (words > 1 and anc_bits.shape[-1] != words) or len(rows_shape) not in (1, 2) \
            or rows_shape[-1] != n:
        raise ValueError("anc_bits must be int64 [n] / [B, n] (ceil(slots / 64) words per row, [..., n, words], above 64 "
                         "tree slots)")
    q = q.contiguous()
    anc_bits = anc_bits.contiguous()
    if len(rows_shape) == 2 and rows_shape[0] not in (1, B):
        raise ValueError("anc_bits batch dimension must be 1 or B")
    stride = n if (len(rows_shape) == 2 and rows_shape[0] == B and B > 1) else 0
    lib = L.lib()
    need = lib.subspec_tree_attention_workspace(B, Hq, Hkv, n, int(prefix_len), slots)
    if workspace is None and need > 256:
        workspace = torch.empty(need, dtype=torch.uint8, device=dev)
    out = torch.empty((B, n, Hq * D), dtype=q.dtype, device=dev)
    code = lib.subspec_tree_attention(
        q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), _dtype_code(q), B, Hq, Hkv, n, slots, D, S,
        int(prefix_len), anc_bits.data_ptr(), stride, float(D ** -0.5 if scale is None else scale),
        None if workspace is None else workspace.data_ptr(),
        0 if workspace is None else workspace.numel() * workspace.element_size(), _stream(dev))
    L.check(code, "subspec_tree_attention")
    return out


def _page_shape(pool_layer_or_pool: torch.Tensor, page_indices: torch.Tensor):
    if page_indices.dtype != torch.int32 or page_indices.dim() != 1 or not page_indices.is_contiguous():
        raise ValueError("page_indices must be a contiguous int32 vector")
    if not pool_layer_or_pool.is_contiguous() or pool_layer_or_pool.shape[-4] != 2:
        raise ValueError("expected a contiguous pool [..., max_pages, 2, page_len, kv_heads, head_dim]")
    return pool_layer_or_pool.shape[-5], pool_layer_or_pool.shape[-3], pool_layer_or_pool.shape[-2], pool_layer_or_pool.shape[-1]


def tree_attention_paged(q: torch.Tensor, pool_layer: torch.Tensor, page_indices: torch.Tensor, anc_bits: torch.Tensor,
                         prefix_len: int, scale: Optional[float] = None, workspace: Optional[torch.Tensor] = None,
                         n_tree_slots: Optional[int] = None):
    """``tree_attention`` over one request's pages: ``q`` [1, Hq, n, D], ``pool_layer``
    [max_pages, 2, page_len, Hkv, D] (one layer of ``KvCachePool.cache_data``), ``page_indices`` int32
    [n_pages] in sequence order; tree K/V already appended at rows prefix_len...  Returns [1, n, Hq * D]."""
    dev = _require_gpu(q, pool_layer, page_indices, anc_bits)
    if q.dim() != 4 or q.shape[0] != 1 or pool_layer.dim() != 5:
        raise ValueError("expected q [1, Hq, n, D] and a pool layer [max_pages, 2, page_len, Hkv, D]")
    max_pages, page_len, Hkv, D = _page_shape(pool_layer, page_indices)
    _, Hq, n, Dq = q.shape
    if Dq != D or q.dtype != pool_layer.dtype:
        raise ValueError("q and the pool must share head_dim and dtype")
    slots = n if n_tree_slots is None else int(n_tree_slots)
    words = (slots + 63) // 64
    if anc_bits.dtype != torch.int64 or anc_bits.numel() != n * words:
        raise ValueError("anc_bits must be int64 [n] ([n, ceil(slots / 64)] above 64 tree slots)")
    q, anc_bits = q.contiguous(), anc_bits.contiguous()
    lib = L.lib()
    need = lib.subspec_tree_attention_workspace(1, Hq, Hkv, n, int(prefix_len), slots)
    if workspace is None and need > 256:
        workspace = torch.empty(need, dtype=torch.uint8, device=dev)
    out = torch.empty((1, n, Hq * D), dtype=q.dtype, device=dev)
    code = lib.subspec_tree_attention_paged(
        q.data_ptr(), pool_layer.data_ptr(), page_indices.data_ptr(), page_indices.numel(), max_pages, page_len,
        out.data_ptr(), _dtype_code(q), Hq, Hkv, n, slots, D, int(prefix_len), anc_bits.data_ptr(),
        float(D ** -0.5 if scale is None else scale), None if workspace is None else workspace.data_ptr(),
        0 if workspace is None else workspace.numel() * workspace.element_size(), _stream(dev))
    L.check(code, "subspec_tree_attention_paged")
    return out


def kv_compact_paged_(pool: torch.Tensor, page_indices: torch.Tensor, contexts: torch.Tensor, offset: int,
                      count: Optional[int] = None, count_dev: Optional[torch.Tensor] = None,
                      max_count: Optional[int] = None) -> torch.Tensor:
    """In place, for every layer and K / V of ``pool`` [L, max_pages, 2, page_len, Hkv, D]:
    logical row offset + j <- logical row offset + contexts[j], j < count, rows addressed through ``page_indices``."""
    dev = _require_gpu(pool, page_indices, contexts)
    if pool.dim() != 6:
        raise ValueError("expected a pool [L, max_pages, 2, page_len, Hkv, D]")
    max_pages, page_len, Hkv, D = _page_shape(pool, page_indices)
    if contexts.dtype != torch.int64 or not contexts.is_contiguous():
        raise ValueError("kv_compact_paged_: contexts must be a contiguous int64 tensor")
    if count_dev is None:
        count = int(contexts.numel()) if count is None else int(count)
    else:
        _require_gpu(count_dev)
        if count_dev.dtype != torch.int32:
            raise ValueError("kv_compact_paged_: count_dev must be int32")
        count = 0
    if max_count is None:
        max_count = min(int(contexts.numel()), L.MAX_TREE_NODES) if count_dev is not None else count
    code = L.lib().subspec_kv_compact_paged(
        pool.data_ptr(), pool.shape[0], max_pages, page_len, Hkv * D * pool.element_size(), page_indices.data_ptr(),
        page_indices.numel(), int(offset), contexts.data_ptr(), None if count_dev is None else count_dev.data_ptr(), count,
        int(max_count), _stream(dev))
    L.check(code, "subspec_kv_compact_paged")
    return pool


def int4_linear(x: torch.Tensor, wq: torch.Tensor, sz: torch.Tensor, out_features: int,
                bias: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x`` [..., K] (bf16 / fp16; 64 rows per pass over the weights, more rows are more passes) times the tiled int4 weight
    (``wq`` int32, ``sz`` int32 as produced by ``subspec_amd.quant.pack_tiled``) -> [..., N]."""
    dev = _require_gpu(x, wq, sz)
    K = x.shape[-1]
    M = x.numel() // K
    N = int(out_features)
    if wq.dtype != torch.int32 or sz.dtype != torch.int32:
        raise ValueError("int4_linear: wq and sz must be int32 tensors in the tiled layout")
    if wq.numel() * 8 != N * K or sz.numel() * 64 != N * K:
        raise ValueError(f"int4_linear: packed weight does not describe a [{N}, {K}] matrix")
    x2 = x.reshape(M, K).contiguous()
    if bias is not None:
        if bias.dtype != x.dtype or bias.numel() != N:
            raise ValueError("int4_linear: bias must be [N] in the activation dtype")
        bias = bias.contiguous()
    lib = L.lib()
    need = lib.subspec_int4_linear_workspace(M, N, K)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=dev)
    y = torch.empty((M, N), dtype=x.dtype, device=dev)
    code = lib.subspec_int4_linear(
        x2.data_ptr(), wq.data_ptr(), sz.data_ptr(), None if bias is None else bias.data_ptr(), y.data_ptr(),
        _dtype_code(x2), M, N, K, 64, None if workspace is None else workspace.data_ptr(),
        0 if workspace is None else workspace.numel() * workspace.element_size(), _stream(dev))
    L.check(code, "subspec_int4_linear")
    return y.reshape(*x.shape[:-1], N)


# ---------------------------------------------------------------------------------------------- draft probabilities
def softmax_temperature(logits: torch.Tensor, temperature: float) -> torch.Tensor:
    """``torch.softmax(logits / temperature, -1)`` in the logits dtype (draft_models/classic_sd.py:10-16)."""
    dev = _require_gpu(logits)
    if not temperature > 0:
        raise ValueError("softmax_temperature: temperature must be positive")
    x = logits.contiguous()
    out = torch.empty_like(x)
    vocab = x.shape[-1]
    rows = x.numel() // vocab
    lib = L.lib()
    need = lib.subspec_softmax_temperature_workspace(rows, vocab)
    ws = torch.empty(need, dtype=torch.uint8, device=dev) if need else None
    code = lib.subspec_softmax_temperature(x.data_ptr(), out.data_ptr(), _dtype_code(x), rows, vocab, float(temperature),
                                           ws.data_ptr() if need else None, need, _stream(dev))
    L.check(code, "subspec_softmax_temperature")
    return out


# ---------------------------------------------------------------------------------------------- decoder layer
def temperature_warp(logits: torch.Tensor, temperature: float) -> torch.Tensor:
    """``logits / temperature`` in the logits dtype (TemperatureLogitsWarper; generators/base.py:57-58)."""
    dev = _require_gpu(logits)
    logits = logits.contiguous()
    out = torch.empty_like(logits)
    code = L.lib().subspec_temperature_warp(logits.data_ptr(), out.data_ptr(), _dtype_code(logits), logits.numel(),
                                            float(temperature), _stream(dev))
    L.check(code, "subspec_temperature_warp")
    return out


def decoder_layer_dims(dtype: torch.dtype, n_rows: int, hidden: int, intermediate: int, n_q_heads: int, n_kv_heads: int,
                       head_dim: int, kv_seq_stride: int, prefix_len: int, n_tree_slots: int, rms_eps: float,
                       rope_theta: float, rope_inv_freq: Optional[torch.Tensor] = None,
                       prefix_len_dev: Optional[torch.Tensor] = None, page_indices: Optional[torch.Tensor] = None,
                       max_pages: int = 0, page_len: int = 0) -> "L.DecoderLayerDims":
    """``rope_inv_freq``: float32 device tensor [head_dim / 2] (kept alive by the caller) with the inverse frequencies
    the caller's eager rotary uses; without it the kernel evaluates ``rope_theta ** (-2i / head_dim)`` itself.
    ``prefix_len_dev``: int64 device tensor of one element that holds the prefix length when the kernels run
    (``prefix_len`` is then its upper bound): layer calls captured into a graph.  ``page_indices``: int32 device page
    table of a paged cache (``k_cache`` of the layer call = one layer of the pool, ``kv_seq_stride`` = pages * page_len)."""
    code = {torch.bfloat16: L.BF16, torch.float16: L.F16}.get(dtype)
    if code is None:
        raise ValueError(f"decoder layer: dtype {dtype} not supported (bf16 / fp16 only)")
    table = None
    if rope_inv_freq is not None:
        if rope_inv_freq.dtype != torch.float32 or rope_inv_freq.numel() != head_dim // 2 or not rope_inv_freq.is_cuda \
                or not rope_inv_freq.is_contiguous():
            raise ValueError("decoder layer: rope_inv_freq must be a contiguous float32 device tensor of head_dim / 2 elements")
        table = rope_inv_freq.data_ptr()
    dyn = None
    if prefix_len_dev is not None:
        if prefix_len_dev.dtype != torch.int64 or prefix_len_dev.numel() != 1 or not prefix_len_dev.is_cuda:
            raise ValueError("decoder layer: prefix_len_dev must be an int64 device tensor of one element")
        dyn = prefix_len_dev.data_ptr()
    pages, n_pages = None, 0
    if page_indices is not None:
        if page_indices.dtype != torch.int32 or not page_indices.is_cuda or not page_indices.is_contiguous():
            raise ValueError("decoder layer: page_indices must be a contiguous int32 device tensor")
        pages, n_pages = page_indices.data_ptr(), page_indices.numel()
    return L.DecoderLayerDims(code, 0, n_rows, hidden, intermediate, n_q_heads, n_kv_heads, head_dim, kv_seq_stride,
                              prefix_len, n_tree_slots, rms_eps, rope_theta, table, dyn, pages, n_pages, int(max_pages),
                              int(page_len))


def decoder_layer_weights(w: dict) -> "L.DecoderLayerWeights":
    """Pointer table of one layer's tensors (``input_layernorm.weight``, ``qkv_proj.wq`` ... as produced by
    ``subspec_amd.model.quantize_layers``).  The caller keeps the tensors alive."""
    def ptr(name):
        t = w.get(name)
        return None if t is None else t.data_ptr()
    for name in ("qkv_proj.wq", "o_proj.wq", "gate_up_proj.wq", "down_proj.wq"):
        if name not in w:
            raise ValueError(f"decoder layer: {name} missing (the layer must be int4-packed)")
    return L.DecoderLayerWeights(ptr("input_layernorm.weight"), ptr("post_attention_layernorm.weight"),
                                 ptr("qkv_proj.wq"), ptr("qkv_proj.sz"), ptr("qkv_proj.bias"),
                                 ptr("o_proj.wq"), ptr("o_proj.sz"), ptr("gate_up_proj.wq"), ptr("gate_up_proj.sz"),
                                 ptr("down_proj.wq"), ptr("down_proj.sz"))


def dense_layer_weights(w: dict) -> "L.DenseLayerWeights":
    """Pointer table of one layer's dense tensors (``qkv_proj.weight`` ... in the fused layout of
    ``subspec_amd.model.init_weights``).  The caller keeps the tensors alive."""
    def ptr(name, required=True):
        t = w.get(name)
        if t is None:
            if required:
                raise ValueError(f"decoder layer: {name} missing")
            return None
        if not t.is_contiguous():
            raise ValueError(f"decoder layer: {name} must be contiguous")
        return t.data_ptr()
    return L.DenseLayerWeights(ptr("input_layernorm.weight"), ptr("post_attention_layernorm.weight"),
                               ptr("qkv_proj.weight"), ptr("qkv_proj.bias", False), ptr("o_proj.weight"),
                               ptr("gate_up_proj.weight"), ptr("down_proj.weight"))


def decoder_layer_workspace(dims: "L.DecoderLayerDims") -> int:
    need = L.lib().subspec_int4_decoder_layer_workspace(ctypes.byref(dims))
    if need == 0:
        raise ValueError("decoder layer: " + L.lib().subspec_last_error().decode("utf-8", "replace"))
    return int(need)


def int4_decoder_layer_(x: torch.Tensor, dims: "L.DecoderLayerDims", weights: "L.DecoderLayerWeights",
                        positions: torch.Tensor, cache_rows: torch.Tensor, anc_bits: torch.Tensor,
                        k_cache: torch.Tensor, v_cache: torch.Tensor, workspace: torch.Tensor) -> torch.Tensor:
    """In-place update of the residual stream ``x`` [n_rows, hidden] by one int4 decoder layer;
    ``positions`` / ``cache_rows`` int32 [n_rows], ``anc_bits`` int64 [n_rows], ``k_cache`` /
    ``v_cache`` [1, Hkv, S, D] views of this layer's cache."""
    dev = _require_gpu(x, positions, cache_rows, anc_bits, k_cache, v_cache, workspace)
    if positions.dtype != torch.int32 or cache_rows.dtype != torch.int32 or anc_bits.dtype != torch.int64:
        raise ValueError("decoder layer: positions / cache_rows must be int32 and anc_bits int64")
    if not (x.is_contiguous() and k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise ValueError("decoder layer: x and the layer's cache views must be contiguous")
    if x.shape != (dims.n_rows, dims.hidden) or positions.numel() != dims.n_rows or cache_rows.numel() != dims.n_rows \
            or anc_bits.numel() != dims.n_rows * ((dims.n_tree_slots + 63) // 64):
        raise ValueError("decoder layer: tensor shapes do not match the dimensions given")
    dense = isinstance(weights, L.DenseLayerWeights)
    fn = L.lib().subspec_dense_decoder_layer if dense else L.lib().subspec_int4_decoder_layer
    code = fn(ctypes.byref(dims), ctypes.byref(weights), x.data_ptr(), positions.data_ptr(), cache_rows.data_ptr(),
              anc_bits.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), workspace.data_ptr(),
              workspace.numel() * workspace.element_size(), _stream(dev))
    L.check(code, "subspec_dense_decoder_layer" if dense else "subspec_int4_decoder_layer")
    return x


decoder_layer_ = int4_decoder_layer_     # either weight storage: the pointer table's type selects the entry point


def int4_gate_up_silu(x: torch.Tensor, wq: torch.Tensor, sz: torch.Tensor, intermediate_size: int,
                      bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``silu(gate) * up`` of a SwiGLU MLP from the fused gate|up int4 weight (``2 * intermediate_size`` rows, gate rows
    first) in one launch: ``x`` [..., K] (at most 64 rows) -> [..., intermediate_size]."""
    dev = _require_gpu(x, wq, sz)
    K = x.shape[-1]
    M = x.numel() // K
    N = 2 * int(intermediate_size)
    if wq.dtype != torch.int32 or sz.dtype != torch.int32:
        raise ValueError("int4_gate_up_silu: wq and sz must be int32 tensors in the tiled layout")
    if wq.numel() * 8 != N * K or sz.numel() * 64 != N * K:
        raise ValueError(f"int4_gate_up_silu: packed weight does not describe a [{N}, {K}] matrix")
    x2 = x.reshape(M, K).contiguous()
    if bias is not None:
        if bias.dtype != x.dtype or bias.numel() != N:
            raise ValueError("int4_gate_up_silu: bias must be [2 * intermediate_size] in the activation dtype")
        bias = bias.contiguous()
    act = torch.empty((M, N // 2), dtype=x.dtype, device=dev)
    code = L.lib().subspec_int4_gate_up_silu(x2.data_ptr(), wq.data_ptr(), sz.data_ptr(),
                                            None if bias is None else bias.data_ptr(), act.data_ptr(), _dtype_code(x2),
                                            M, N, K, _stream(dev))
    L.check(code, "subspec_int4_gate_up_silu")
    return act.reshape(*x.shape[:-1], N // 2)


def dense_gate_up_silu(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``silu(gate) * up`` from a dense fused weight [2F, K] (gate rows first) in one launch: x [..., K] (at most 384
    rows) -> [..., F]."""
    dev = _require_gpu(x, weight)
    N, K = weight.shape
    if x.shape[-1] != K or x.dtype != weight.dtype or N % 2:
        raise ValueError("dense_gate_up_silu: x [..., K] and weight [2F, K] must agree in K and dtype")
    M = x.numel() // K
    x2 = x.reshape(M, K).contiguous()
    weight = weight.contiguous()
    if bias is not None:
        if bias.dtype != x.dtype or bias.numel() != N:
            raise ValueError("dense_gate_up_silu: bias must be [2F] in the activation dtype")
        bias = bias.contiguous()
    act = torch.empty((M, N // 2), dtype=x.dtype, device=dev)
    code = L.lib().subspec_dense_gate_up_silu(x2.data_ptr(), weight.data_ptr(), None if bias is None else bias.data_ptr(),
                                             act.data_ptr(), _dtype_code(x2), M, N, K, _stream(dev))
    L.check(code, "subspec_dense_gate_up_silu")
    return act.reshape(*x.shape[:-1], N // 2)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``weight * (x * rsqrt(mean(x^2) + eps)).to(x.dtype)`` over the last dimension in one launch
    (bf16 / fp16; hidden a multiple of 8, at most 16384)."""
    dev = _require_gpu(x, weight)
    H = x.shape[-1]
    if weight.numel() != H or weight.dtype != x.dtype:
        raise ValueError("rms_norm: weight must be [hidden] in the activation dtype")
    x2 = x.reshape(-1, H).contiguous()
    y = torch.empty_like(x2)
    code = L.lib().subspec_rms_norm(x2.data_ptr(), weight.contiguous().data_ptr(), y.data_ptr(), _dtype_code(x2),
                                    x2.shape[0], H, float(eps), _stream(dev))
    L.check(code, "subspec_rms_norm")
    return y.reshape(x.shape)


def dense_linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``F.linear(x, weight, bias)`` for at most 384 rows of bf16 / fp16 activations: x [..., K], weight [N, K]
    (N a multiple of 16; of 32 above 64 rows)."""
    dev = _require_gpu(x, weight)
    N, K = weight.shape
    if x.shape[-1] != K or x.dtype != weight.dtype:
        raise ValueError("dense_linear: x [..., K] and weight [N, K] must agree in K and dtype")
    M = x.numel() // K
    x2 = x.reshape(M, K).contiguous()
    weight = weight.contiguous()
    if bias is not None:
        if bias.dtype != x.dtype or bias.numel() != N:
            raise ValueError("dense_linear: bias must be [N] in the activation dtype")
        bias = bias.contiguous()
    lib = L.lib()
    need = lib.subspec_dense_linear_workspace(M, N, K)
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    y = torch.empty((M, N), dtype=x.dtype, device=dev)
    code = lib.subspec_dense_linear(x2.data_ptr(), weight.data_ptr(), None if bias is None else bias.data_ptr(), y.data_ptr(),
                                    _dtype_code(x), M, N, K, ws.data_ptr(), need, _stream(dev))
    L.check(code, "subspec_dense_linear")
    return y.reshape(*x.shape[:-1], N)
