"""Minimal Qwen2-shaped decoder used by the cycle driver: RMSNorm, rotary embeddings, GQA attention
against the shared static KV cache, SwiGLU MLP.  Random-init weights of the real shapes; nothing is
downloaded.

Plain library work (bf16 GEMMs, norms, rotary, the causal prefill attention) goes through torch;
the hot-path pieces are the HIP kernels: tree-masked attention for every tree forward, int4
GEMV / GEMM for the draft's projections, layer streaming for the target's offloaded layers.
q/k/v and gate/up are stored fused (rows concatenated), which leaves every output row and its
quantization groups unchanged.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Callable, Dict, List, Optional

import torch
import torch.nn.functional as F

from . import ops, quant
from .cache import KVManager
from .offload import LayerSlabLayout, LayerStreamer


@dataclass
class DecoderConfig:
    num_hidden_layers: int = 28
    hidden_size: int = 3584
    num_attention_heads: int = 28
    num_key_value_heads: int = 4
    head_dim: int = 128
    intermediate_size: int = 18944
    vocab_size: int = 152064
    rms_norm_eps: float = 1e-6
    rope_theta: float = 1e6
    max_position_embeddings: int = 32768

    @property
    def q_size(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_key_value_heads * self.head_dim


def layer_shapes(cfg: DecoderConfig) -> Dict[str, tuple]:
    H, F_ = cfg.hidden_size, cfg.intermediate_size
    return {
        "input_layernorm.weight": (H,),
        "qkv_proj.weight": (cfg.q_size + 2 * cfg.kv_size, H),
        "qkv_proj.bias": (cfg.q_size + 2 * cfg.kv_size,),
        "o_proj.weight": (H, cfg.q_size),
        "post_attention_layernorm.weight": (H,),
        "gate_up_proj.weight": (2 * F_, H),
        "down_proj.weight": (H, F_),
    }


QUANTIZED = ("qkv_proj", "o_proj", "gate_up_proj", "down_proj")


def init_weights(cfg: DecoderConfig, seed: int, device, dtype=torch.bfloat16) -> dict:
    g = torch.Generator(device=device).manual_seed(seed)

    def rnd(*shape, std=0.02):
        return (torch.randn(*shape, generator=g, device=device, dtype=torch.float32) * std).to(dtype)

    layers = []
    for _ in range(cfg.num_hidden_layers):
        w = {}
        for name, shape in layer_shapes(cfg).items():
            if name.endswith("layernorm.weight"):
                w[name] = torch.ones(shape, device=device, dtype=dtype)
            elif name.endswith(".bias"):
                w[name] = rnd(*shape, std=0.02)
            else:
                w[name] = rnd(*shape)
        layers.append(w)
    return {"embed": rnd(cfg.vocab_size, cfg.hidden_size), "layers": layers,
            "norm": torch.ones(cfg.hidden_size, device=device, dtype=dtype),
            "lm_head": rnd(cfg.vocab_size, cfg.hidden_size)}


def quantize_layers(layers: List[Dict[str, torch.Tensor]], optimize: bool = False) -> List[Dict[str, torch.Tensor]]:
    """int4 g64 copies of the four projections of every layer (norms and biases are shared); ``optimize``
    refines the zero points as hqq does by default (quant.refine_zero_proximal)."""
    out = []
    for w in layers:
        q = {k: v for k, v in w.items() if not any(k == n + ".weight" for n in QUANTIZED)}
        for n in QUANTIZED:
            wq, sz = quant.pack_tiled(*quant.quantize_int4_g64(w[n + ".weight"], optimize=optimize))
            q[n + ".wq"], q[n + ".sz"] = wq, sz
            q[n + ".out_features"] = w[n + ".weight"].shape[0]
        out.append(q)
    return out


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    if x.is_cuda and x.dtype != torch.float32 and x.shape[-1] % 8 == 0 and x.shape[-1] <= 16384:
        return ops.rms_norm(x, weight, eps)                  # one launch instead of seven
    xf = x.float()
    xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return weight * xf.to(x.dtype)


def _linear(w: Dict[str, torch.Tensor], name: str, x: torch.Tensor) -> torch.Tensor:
    bias = w.get(name + ".bias")
    if name + ".wq" in w:
        return ops.int4_linear(x, w[name + ".wq"], w[name + ".sz"], w[name + ".out_features"], bias)
    return F.linear(x, w[name + ".weight"], bias)


class Decoder:
    """One decoder stack over a shared KV cache.  ``layers[i]`` holds either bf16 weights or int4
    packed weights; layers from ``first_streamed`` on are fetched through ``streamer``."""

    def __init__(self, cfg: DecoderConfig, embed, layers, norm, lm_head, kv: KVManager,
                 streamer: Optional[LayerStreamer] = None, first_streamed: Optional[int] = None):
        self.cfg, self.embed, self.layers, self.norm, self.lm_head, self.kv = cfg, embed, layers, norm, lm_head, kv
        self.streamer = streamer
        self.first_streamed = cfg.num_hidden_layers if first_streamed is None else first_streamed
        self.device, self.dtype = embed.device, embed.dtype
        self._native = None
        self.use_native_layers = True            # False: run every module through its own torch / library call
        self._inv_freq = 1.0 / (cfg.rope_theta ** (torch.arange(0, cfg.head_dim, 2, device=self.device, dtype=torch.float32)
                                                   / cfg.head_dim))
        self._rope_len = 0
        self._rope_tables(kv.cache.max_cache_len + 8)

    def bind_cache(self, kv: KVManager) -> None:
        """Run over another cache from now on (the builder creates the cache after the models)."""
        if kv is not self.kv:
            self.kv = kv
            self._native = None                      # whether the one-call layers apply depends on the cache layout
        self._rope_tables(kv.cache.max_cache_len + 8)

    def _rope_tables(self, n: int) -> None:
        """cos / sin of positions 0 .. n - 1 (rebuilt when a growing cache passes their length)."""
        if n <= self._rope_len:
            return
        freqs = torch.outer(torch.arange(n, device=self.device, dtype=torch.float32), self._inv_freq)
        self.cos = torch.cat([freqs, freqs], -1).cos()
        self.sin = torch.cat([freqs, freqs], -1).sin()
        self._rope_len = n

    # ------------------------------------------------------------------ native layers
    @property
    def native_layers(self) -> bool:
        """True when the stack can run through the library's decoder-layer entry points (one host call
        per layer instead of one per module): every layer int4-packed, or every layer dense 16-bit."""
        if self._native is None:
            packed = [("qkv_proj.wq" in w) for w in self.layers]
            # either cache layout: contiguous per-layer caches, or the page pool (rows written and read through the table)
            self._native = (bool(self.layers) and (all(packed) or not any(packed)) and self.dtype != torch.float32
                            and (self.kv.cache.contiguous or hasattr(self.kv.cache, "pool")))
            if self._native:
                self._native_packed = packed[0]      # int4 layers: windows of at most 64 rows
                make = ops.decoder_layer_weights if packed[0] else ops.dense_layer_weights
                self._native_make = make
                resident = min(self.first_streamed, len(self.layers))
                self._native_weights = [make(w) for w in self.layers[:resident]]
                self._native_ws = {}
        return self._native

    def _run_native_layers(self, x, positions, rows, anc_bits, prefix_len: int, slots: int,
                           prefix_len_dev: Optional[torch.Tensor] = None, fresh: bool = False) -> torch.Tensor:
        """``fresh``: ``x`` is a tensor of the caller's own making (the layers work in place and may keep it)."""
        cfg, cache = self.cfg, self.kv.cache
        n = x.shape[0]
        paged = not cache.contiguous
        if paged:
            table = cache.table()
            paging = dict(page_indices=table, max_pages=cache.pool.max_pages, page_len=cache.page_len)
            stride = table.numel() * cache.page_len
            layer_kv = lambda i: (cache.pool.cache_data[i], cache.pool.cache_data[i])
        else:
            paging, stride = {}, cache.max_cache_len
            layer_kv = lambda i: (cache.k(i), cache.v(i))
        dims = ops.decoder_layer_dims(self.dtype, n, cfg.hidden_size, cfg.intermediate_size, cfg.num_attention_heads,
                                      cfg.num_key_value_heads, cfg.head_dim, stride, int(prefix_len),
                                      int(slots), cfg.rms_norm_eps, cfg.rope_theta, self._inv_freq,
                                      prefix_len_dev=prefix_len_dev, **paging)
        need = ops.decoder_layer_workspace(dims)
        ws = self._native_ws.get("ws")
        if ws is None or ws.numel() < need:
            ws = self._native_ws["ws"] = torch.empty(need, dtype=torch.uint8, device=self.device)
        x = x if fresh and x.is_contiguous() else x.contiguous().clone()
        pos32, rows32 = positions.to(torch.int32), rows.to(torch.int32)          # no copies when they are int32 already
        bits = anc_bits.to(torch.int64).contiguous()
        for i, w in enumerate(self._native_weights):
            ops.decoder_layer_(x, dims, w, pos32, rows32, bits, *layer_kv(i), ws)
        if self.streamer is not None and self.streamer.n:
            base = self.first_streamed

            def step(j, w):                       # w: views into the device slab that holds layer base + j right now
                ops.decoder_layer_(x, dims, self._native_make(w), pos32, rows32, bits, *layer_kv(base + j), ws)

            self.streamer.run(step)
        return x

    # ------------------------------------------------------------------ pieces
    def _rope(self, t: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """t: [n, heads, D]"""
        cos = self.cos[positions].unsqueeze(1).to(t.dtype)
        sin = self.sin[positions].unsqueeze(1).to(t.dtype)
        half = t.shape[-1] // 2
        rot = torch.cat([-t[..., half:], t[..., :half]], -1)
        return t * cos + rot * sin

    def _layer(self, i: int, w: Dict[str, torch.Tensor], x: torch.Tensor, positions: torch.Tensor,
               rows: torch.Tensor, attn: Callable[[int, torch.Tensor], torch.Tensor]) -> torch.Tensor:
        cfg = self.cfg
        n = x.shape[0]
        h = rms_norm(x, w["input_layernorm.weight"], cfg.rms_norm_eps)
        qkv = _linear(w, "qkv_proj", h)
        q, k, v = qkv.split([cfg.q_size, cfg.kv_size, cfg.kv_size], dim=-1)
        q = self._rope(q.reshape(n, cfg.num_attention_heads, cfg.head_dim), positions)
        k = self._rope(k.reshape(n, cfg.num_key_value_heads, cfg.head_dim), positions)
        v = v.reshape(n, cfg.num_key_value_heads, cfg.head_dim)
        self.kv.cache.write(i, rows, k.transpose(0, 1).unsqueeze(0), v.transpose(0, 1).unsqueeze(0))
        a = attn(i, q.transpose(0, 1).unsqueeze(0).contiguous())          # [1, Hq, n, D] -> [n, Hq*D]
        x = x + _linear(w, "o_proj", a)
        h = rms_norm(x, w["post_attention_layernorm.weight"], cfg.rms_norm_eps)
        gate, up = _linear(w, "gate_up_proj", h).chunk(2, dim=-1)
        return x + _linear(w, "down_proj", F.silu(gate) * up)

    def _run_layers(self, x, positions, rows, attn) -> torch.Tensor:
        state = {"x": x}
        for i in range(min(self.first_streamed, len(self.layers))):
            state["x"] = self._layer(i, self.layers[i], state["x"], positions, rows, attn)
        if self.streamer is not None and self.streamer.n:
            base = self.first_streamed

            def step(j, w):
                state["x"] = self._layer(base + j, w, state["x"], positions, rows, attn)

            self.streamer.run(step)
        return state["x"]

    def logits(self, x: torch.Tensor) -> torch.Tensor:
        """Final norm and the language-model head (HuggingFace ``lm_head`` inside the draft and target forwards,
        specdecodes/models/draft_models/classic_sd.py:10-16, generators/classic_sd.py:102-109).  Up to 64 rows the
        1.09 GB head streams through the dense kernels of this package (152064 x 3584 bf16: 170 us at 8 rows, 198 us at 32
        against 232 / 255 us for the vendor GEMM; 204 us at 64 rows, where the two are level); wider inputs keep the
        vendor GEMM (128 rows: 236 against 261 us)."""
        h = rms_norm(x, self.norm, self.cfg.rms_norm_eps)
        rows = h.numel() // h.shape[-1]
        V, H = self.lm_head.shape
        if (h.is_cuda and rows <= 64 and h.dtype in (torch.bfloat16, torch.float16) and H % 64 == 0
                and (V % 32 == 0 if rows > 32 else V % 16 == 0 and V * H * 2 < (1 << 31)) and self.lm_head.is_contiguous()):
            return ops.dense_linear(h, self.lm_head)
        return F.linear(h, self.lm_head)

    # ------------------------------------------------------------------ forwards
    def prefill(self, token_ids: torch.Tensor, start: int, all_logits: bool = False) -> torch.Tensor:
        """Causal forward of ``token_ids`` [n] at cache rows start..start+n-1; returns the last logits [1, V]
        (``all_logits``: the logits of every position [n, V], e.g. to score a sequence by teacher forcing)."""
        n = token_ids.numel()
        self.kv.cache.ensure(start + n)
        self._rope_tables(start + n)
        positions = torch.arange(start, start + n, device=self.device)
        cfg = self.cfg
        rep = cfg.num_attention_heads // cfg.num_key_value_heads

        def attn(i, q):
            k, v = self.kv.cache.prefix_kv(i, start + n)
            k, v = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)
            mask = torch.ones(n, start + n, dtype=torch.bool, device=self.device).tril(diagonal=start)
            o = F.scaled_dot_product_attention(q, k, v, attn_mask=mask)
            return o.transpose(1, 2).reshape(n, cfg.q_size)

        x = self._run_layers(self.embed[token_ids], positions, positions, attn)
        return self.logits(x if all_logits else x[-1:])

    def tree_forward(self, token_ids: torch.Tensor, depths: Optional[torch.Tensor], anc_bits: torch.Tensor, prefix_len: int,
                     first_slot: int = 0, n_tree_slots: Optional[int] = None,
                     prefix_len_dev: Optional[torch.Tensor] = None,
                     positions32: Optional[torch.Tensor] = None, rows32: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Forward of tree nodes occupying cache rows prefix_len+first_slot.. ; ``depths`` are the node
        depths (rotary position = prefix_len + depth), ``anc_bits`` int64 [n] bitsets over tree
        slots ([n, ceil(slots / 64)] words above 64 slots).  Up to 64 rows (int4 layers) or 384 rows (dense layers: a
        whole 289-node tree in the target) go through the one-call layers, every weight matrix read once for all
        rows; a larger window runs module by module on library GEMMs with only attention on this library's kernel.
        Returns logits [n, V].

        ``prefix_len_dev`` (int64 device tensor of one element): the prefix length is taken from the device when the
        kernels run and ``prefix_len`` is only its upper bound -- nothing on the host side depends on the actual
        value, so the call can be captured into a graph and replayed as the sequence grows (one-call layers only).

        ``positions32`` / ``rows32`` (int32 [n], both or neither): rotary positions and cache rows the caller has worked
        out already -- a draft that grows a tree level by level derives them for all levels of a speculation at once
        instead of with five small launches per level; ``depths`` is then unused (one-call layers only)."""
        n = token_ids.numel()
        slots = first_slot + n if n_tree_slots is None else n_tree_slots
        self.kv.cache.ensure(prefix_len + max(slots, first_slot + n))
        self._rope_tables(prefix_len + max(slots, first_slot + n) + 8)
        cfg = self.cfg
        native = self.use_native_layers and self.native_layers and slots <= ops.L.MAX_TREE_NODES
        if native and n > 64:                        # dense layers only, projection widths in tiles of 32
            native = (n <= 384 and not self._native_packed and cfg.q_size % 32 == 0 and cfg.kv_size % 32 == 0
                      and cfg.hidden_size % 32 == 0)
        if prefix_len_dev is not None and not native:
            raise ValueError("a device-side prefix length needs the one-call decoder layers (at most 64 rows; 384 for dense layers)")
        if positions32 is not None and rows32 is not None:
            if native:
                return self.logits(self._run_native_layers(self.embed[token_ids], positions32, rows32, anc_bits, prefix_len,
                                                           slots, prefix_len_dev=prefix_len_dev, fresh=True))
            positions, rows = positions32.long(), rows32.long()
        elif depths is None:
            raise ValueError("tree_forward needs `depths`, or positions32 and rows32")
        elif prefix_len_dev is not None:
            positions = depths.to(self.device) + prefix_len_dev
            rows = torch.arange(first_slot, first_slot + n, device=self.device) + prefix_len_dev
        else:
            positions = depths.to(self.device) + prefix_len
            rows = torch.arange(prefix_len + first_slot, prefix_len + first_slot + n, device=self.device)
        if native:
            return self.logits(self._run_native_layers(self.embed[token_ids], positions, rows, anc_bits, prefix_len, slots,
                                                       prefix_len_dev=prefix_len_dev))

        def attn(i, q):
            return self.kv.cache.tree_attention(i, q, anc_bits, prefix_len, slots).reshape(n, cfg.q_size)

        return self.logits(self._run_layers(self.embed[token_ids], positions, rows, attn))


def config_from_hf(config: dict) -> DecoderConfig:
    """``DecoderConfig`` from the fields of a HuggingFace ``config.json`` (Qwen2 / Llama family)."""
    heads = int(config["num_attention_heads"])
    return DecoderConfig(
        num_hidden_layers=int(config["num_hidden_layers"]), hidden_size=int(config["hidden_size"]),
        num_attention_heads=heads, num_key_value_heads=int(config.get("num_key_value_heads", heads)),
        head_dim=int(config.get("head_dim") or int(config["hidden_size"]) // heads),
        intermediate_size=int(config["intermediate_size"]), vocab_size=int(config["vocab_size"]),
        rms_norm_eps=float(config.get("rms_norm_eps", 1e-6)), rope_theta=float(config.get("rope_theta", 1e4)),
        max_position_embeddings=int(config.get("max_position_embeddings", 32768)))


def load_hf_checkpoint(path: str, device="cpu", dtype=torch.bfloat16):
    """Weights of a LOCAL HuggingFace checkpoint directory (``config.json`` + ``*.safetensors``, Qwen2 or
    Llama naming) in this package's fused layout: ``qkv_proj = q|k|v`` rows, ``gate_up_proj = gate|up`` rows.
    Returns ``(DecoderConfig, weights)`` with ``weights`` as produced by ``init_weights``.

    The reference loads the same checkpoints by model name through ``AutoModelForCausalLM.from_pretrained``
    (run/core/builder.py:94-103); nothing is downloaded here and only safetensors files are read."""
    import glob
    import json
    import os

    from safetensors import safe_open

    with open(os.path.join(path, "config.json")) as f:
        hf = json.load(f)
    cfg = config_from_hf(hf)
    tensors: Dict[str, torch.Tensor] = {}
    files = sorted(glob.glob(os.path.join(path, "*.safetensors")))
    if not files:
        raise FileNotFoundError(f"no .safetensors file in {path}")
    for fn in files:
        with safe_open(fn, framework="pt", device="cpu") as sf:
            for key in sf.keys():
                tensors[key] = sf.get_tensor(key)

    return cfg, weights_from_tensors(cfg, tensors, device, dtype, where=f"the checkpoint in {path}")


def weights_from_tensors(cfg: DecoderConfig, tensors: Dict[str, torch.Tensor], device="cpu", dtype=torch.bfloat16,
                         where: str = "the state dict") -> dict:
    """HuggingFace-named tensors (``model.layers.N.self_attn.q_proj.weight`` ..., Qwen2 or Llama) -> this package's
    fused layout (``qkv_proj = q|k|v`` rows, ``gate_up_proj = gate|up`` rows), as produced by ``init_weights``."""
    def take(name: str, required: bool = True) -> Optional[torch.Tensor]:
        t = tensors.get(name)
        if t is None:
            if required:
                raise KeyError(f"{name} missing from {where}")
            return None
        return t.detach().to(device=device, dtype=dtype)

    layers = []
    for i in range(cfg.num_hidden_layers):
        pre = f"model.layers.{i}."
        w = {"input_layernorm.weight": take(pre + "input_layernorm.weight"),
             "post_attention_layernorm.weight": take(pre + "post_attention_layernorm.weight"),
             "qkv_proj.weight": torch.cat([take(pre + f"self_attn.{n}_proj.weight") for n in "qkv"], 0),
             "o_proj.weight": take(pre + "self_attn.o_proj.weight"),
             "gate_up_proj.weight": torch.cat([take(pre + "mlp.gate_proj.weight"), take(pre + "mlp.up_proj.weight")], 0),
             "down_proj.weight": take(pre + "mlp.down_proj.weight")}
        biases = [take(pre + f"self_attn.{n}_proj.bias", required=False) for n in "qkv"]
        # Qwen2 has q/k/v biases, Llama has none: a zero bias keeps one layer layout for both
        sizes = (cfg.q_size, cfg.kv_size, cfg.kv_size)
        w["qkv_proj.bias"] = torch.cat([b if b is not None else torch.zeros(n, device=device, dtype=dtype)
                                        for b, n in zip(biases, sizes)], 0)
        for name, shape in layer_shapes(cfg).items():
            if name in w and tuple(w[name].shape) != tuple(shape):
                raise ValueError(f"layer {i}: {name} has shape {tuple(w[name].shape)}, expected {tuple(shape)}")
        layers.append(w)
    embed = take("model.embed_tokens.weight")
    head = take("lm_head.weight", required=False)
    if head is None:                                              # tie_word_embeddings
        head = embed
    return {"embed": embed, "layers": layers, "norm": take("model.norm.weight"), "lm_head": head}


def build_models(cfg: DecoderConfig, kv: KVManager, seed: int = 0, device="cuda:0", dtype=torch.bfloat16,
                 first_streamed: Optional[int] = None, weights: Optional[dict] = None, hqq_optimize: bool = False,
                 n_slabs: int = 4):
    """Target (bf16, layers >= first_streamed in pinned host memory) and substitute draft (same
    weights, int4 g64, resident) over one shared KV cache.  ``n_slabs``: device slabs of the streaming ring, i.e.
    how many layers the copies may run ahead of the compute stream (``LayerStreamer``)."""
    w = init_weights(cfg, seed, device, dtype) if weights is None else weights     # e.g. from load_hf_checkpoint
    draft_layers = quantize_layers(w["layers"], optimize=hqq_optimize)
    streamer = None
    layers = w["layers"]
    if first_streamed is not None and first_streamed < cfg.num_hidden_layers:
        layout = LayerSlabLayout(layer_shapes(cfg), dtype)
        host = [{k: v.cpu() for k, v in layers[i].items()} for i in range(first_streamed, cfg.num_hidden_layers)]
        streamer = LayerStreamer(layout, host, device, n_slabs=n_slabs)
        layers = layers[:first_streamed]
    target = Decoder(cfg, w["embed"], layers, w["norm"], w["lm_head"], kv, streamer, first_streamed)
    draft = Decoder(cfg, w["embed"], draft_layers, w["norm"], w["lm_head"], kv)
    return target, draft, w
