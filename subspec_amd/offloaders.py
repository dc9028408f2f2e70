"""Offloaders with the reference's call convention ``cls(model, device_map=..., draft_model=...)``
(specdecodes/helpers/recipes/base_recipe.py:54-63), for HuggingFace-shaped modules.

``PrefetchOffloader`` stands for specdecodes/helpers/offloaders/prefetch_offloader_postspec.py:54-241 (asynchronous
copies on a side stream, post-speculation in the waits) and ``Offloader`` for the synchronous
specdecodes/helpers/offloaders/offloader.py:40-89; here both place the weights the same way and stream them through
``subspec_amd.offload.LayerStreamer`` (the synchronous one with a ring of two slabs, which serialises copy and
compute as its reference does only by accident of the hook order; results are identical).

What an offloader does to the model:
  * modules whose ``device_map`` entry is ``"cpu"`` are decoder-layer projections; a layer is streamed when ALL
    seven of its projections are (``LayerOffloadRecipe``: layers ``keep_first_n_layers_on_gpu ..``; the SubSpec
    recipe: every layer).  Streamed layers must form the tail of the stack; anything else is refused with the
    reason (the slab ring visits layers in order and a forward starts with the resident ones);
  * each streamed layer becomes ONE pinned host slab in the fused layout (q|k|v, gate|up; its two norm gains ride
    along), and the module's parameters are re-pointed at views of that slab, so the weights exist once in host
    memory;
  * every other parameter moves to the device named for ``model.embed_tokens``;
  * the result is recorded on the module (``model._subspec_offload``) for ``hf_model.as_decoder``.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch
import torch.nn as nn

from .hf_model import ATTN, MLP, _hf_config_of
from .model import layer_shapes
from .offload import LayerSlabLayout, LayerStreamer


def _uncovered(model: nn.Module, device_map: Dict[str, object]):
    names = list(model.state_dict().keys())
    if "" in device_map:
        return []
    keys = tuple(device_map.keys())
    return [n for n in names if not any(n == k or n.startswith(k + ".") for k in keys)]


class OffloadState:
    def __init__(self, device, first_streamed: int, streamer: Optional[LayerStreamer]):
        self.device, self.first_streamed, self.streamer = torch.device(device), first_streamed, streamer


class PrefetchOffloader:
    n_slabs = 4

    def __init__(self, model: nn.Module, device_map: Dict[str, object], draft_model=None, n_slabs: Optional[int] = None,
                 **_unused):
        if n_slabs is not None:
            self.n_slabs = int(n_slabs)                  # ring depth: layers the copies may run ahead (default of the class)
        missing = _uncovered(model, device_map)
        if missing:
            raise ValueError("The device_map provided does not give any device for the following parameters: "
                             + ", ".join(missing))
        if "model.embed_tokens" not in device_map:
            raise ValueError("device_map must name the device of model.embed_tokens (the GPU the model runs on)")
        self.gpu_device = torch.device(device_map["model.embed_tokens"])
        if self.gpu_device.type != "cuda":
            raise ValueError(f"model.embed_tokens is mapped to {self.gpu_device}: the resident part must sit on a GPU")
        self.draft_model = draft_model
        cfg = _hf_config_of(model)
        n_layers = len(model.model.layers)

        def on_cpu(name: str) -> bool:
            return str(device_map.get(name, self.gpu_device)) == "cpu"

        streamed = []
        for i in range(n_layers):
            flags = [on_cpu(f"model.layers.{i}.self_attn.{n}") for n in ATTN] + [on_cpu(f"model.layers.{i}.mlp.{n}") for n in MLP]
            if any(flags) and not all(flags):
                raise ValueError(f"layer {i}: some of its projections are mapped to the CPU and some are not; a layer is "
                                 "streamed as one slab, so map all seven or none")
            streamed.append(all(flags))
        stray = [k for k, v in device_map.items() if str(v) == "cpu" and ".layers." not in k]
        if stray:
            raise ValueError(f"only decoder-layer projections can be offloaded, not {stray}")
        if not any(streamed):
            raise ValueError("No CPU layer found in the model.")
        first = streamed.index(True)
        if not all(streamed[first:]):
            raise ValueError("streamed layers must be the last layers of the stack (layers "
                             f"{[i for i, s in enumerate(streamed) if s]} were mapped to the CPU)")
        self.first_streamed = first

        dtype = model.model.embed_tokens.weight.dtype
        layout = LayerSlabLayout(layer_shapes(cfg), dtype)
        host_layers = [self._fused_host_layer(model.model.layers[i], cfg, dtype) for i in range(first, n_layers)]
        self.streamer = LayerStreamer(layout, host_layers, self.gpu_device, n_slabs=self.n_slabs)
        del host_layers
        for j, i in enumerate(range(first, n_layers)):             # the module now aliases its pinned slab
            self._alias(model.model.layers[i], layout.views(self.streamer.host[j]), cfg)
        # everything else to the GPU (parameters shared with the draft move with it: their storage is swapped in place)
        for name, mod in model.named_modules():
            if name.startswith("model.layers.") and int(name.split(".")[2]) >= first:
                continue
            for p in list(mod.parameters(recurse=False)) + list(mod.buffers(recurse=False)):
                if p.device != self.gpu_device and not p.is_meta:
                    p.data = p.data.to(self.gpu_device)
        model._subspec_offload = OffloadState(self.gpu_device, first, self.streamer)
        model._subspec_decoder = None

    @staticmethod
    def _fused_host_layer(layer: nn.Module, cfg, dtype) -> Dict[str, torch.Tensor]:
        a, m = layer.self_attn, layer.mlp
        for mod in (a.q_proj, a.k_proj, a.v_proj, a.o_proj, m.gate_proj, m.up_proj, m.down_proj):
            if not isinstance(mod, nn.Linear):
                raise TypeError(f"a streamed layer must hold dense nn.Linear projections, found {type(mod).__name__}")
        biases = [getattr(p, "bias", None) for p in (a.q_proj, a.k_proj, a.v_proj)]
        sizes = (cfg.q_size, cfg.kv_size, cfg.kv_size)
        return {"input_layernorm.weight": layer.input_layernorm.weight.data,
                "qkv_proj.weight": torch.cat([a.q_proj.weight.data, a.k_proj.weight.data, a.v_proj.weight.data], 0),
                "qkv_proj.bias": torch.cat([b.data if b is not None else torch.zeros(n, dtype=dtype) for b, n in zip(biases, sizes)], 0),
                "o_proj.weight": a.o_proj.weight.data,
                "post_attention_layernorm.weight": layer.post_attention_layernorm.weight.data,
                "gate_up_proj.weight": torch.cat([m.gate_proj.weight.data, m.up_proj.weight.data], 0),
                "down_proj.weight": m.down_proj.weight.data}

    @staticmethod
    def _alias(layer: nn.Module, views: Dict[str, torch.Tensor], cfg) -> None:
        a, m = layer.self_attn, layer.mlp
        q, k, v = views["qkv_proj.weight"].split([cfg.q_size, cfg.kv_size, cfg.kv_size], 0)
        bq, bk, bv = views["qkv_proj.bias"].split([cfg.q_size, cfg.kv_size, cfg.kv_size], 0)
        gate, up = views["gate_up_proj.weight"].chunk(2, 0)
        for mod, w, b in ((a.q_proj, q, bq), (a.k_proj, k, bk), (a.v_proj, v, bv), (a.o_proj, views["o_proj.weight"], None),
                          (m.gate_proj, gate, None), (m.up_proj, up, None), (m.down_proj, views["down_proj.weight"], None)):
            mod.weight.data = w
            if b is not None and getattr(mod, "bias", None) is not None:
                mod.bias.data = b
        layer.input_layernorm.weight.data = views["input_layernorm.weight"]
        layer.post_attention_layernorm.weight.data = views["post_attention_layernorm.weight"]


class Offloader(PrefetchOffloader):
    """The synchronous offloader's placement (offloader.py:40-89) with the smallest ring."""
    n_slabs = 2

    def __init__(self, model: nn.Module, device_map: Dict[str, object], record_stream: bool = False, draft_model=None):
        super().__init__(model, device_map, draft_model=draft_model)
