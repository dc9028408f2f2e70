"""Recipes loadable from the reference's YAML ``recipe: {class_path, kwargs}`` entries (run/core/config_utils.py:23-62),
e.g. ``class_path: subspec_amd.recipes:Recipe`` or ``subspec_amd.recipes:LayerOffloadRecipe`` with
``kwargs: {keep_first_n_layers_on_gpu: 14}``.

Same three methods and return shapes as the reference's ``QuantOffloadRecipe``
(specdecodes/helpers/recipes/base_recipe.py:5-63): ``generate_configurations(target_model, draft_model, max_length,
cpu_offload_gb, dtype, device) -> (target_config, draft_config)`` with optional ``"device_map"`` / ``"quant_config"``
entries, ``apply_quantization(model, quant_config, dtype, device)``, ``apply_offloading(model, device_map,
draft_model=None)``; ``quantizer`` / ``offloader`` are class attributes of the instance, ``None`` = skip.
"""
from __future__ import annotations

import logging
from typing import Any, Dict, Optional, Tuple

from .offloaders import Offloader, PrefetchOffloader
from .quant import HqqQuantizer

PROJECTIONS = ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "self_attn.o_proj",
               "mlp.gate_proj", "mlp.up_proj", "mlp.down_proj")


def BaseQuantizeConfig(nbits: int = 4, group_size: int = 64, axis: int = 1, **extra) -> Dict[str, Any]:
    """Per-layer quantization config in the shape hqq's function of this name returns (a dict with
    ``weight_quant_params``), reduced to what this build's quantizer reads."""
    return {"weight_quant_params": {"nbits": int(nbits), "group_size": int(group_size), "axis": int(axis), **extra},
            "scale_quant_params": None, "zero_quant_params": None}


def _module_devices(model, device, on_cpu) -> Dict[str, Any]:
    """Device of every parameter- or buffer-holding module: ``"cpu"`` for the names in ``on_cpu``, else ``device``
    (recipes/subspec/hqq_4bit_postspec.py:37-46)."""
    device_map: Dict[str, Any] = {}
    for name, _ in model.named_parameters():
        owner = ".".join(name.split(".")[:-1])
        device_map[owner] = "cpu" if owner in on_cpu else device
    for name, _ in model.named_buffers():
        device_map[".".join(name.split(".")[:-1])] = device
    device_map.setdefault("lm_head", device)
    return device_map


class QuantOffloadRecipe:
    def __init__(self):
        self.quantizer = None
        self.offloader = None

    def generate_configurations(self, target_model: Any, draft_model: Any, max_length: int, cpu_offload_gb: Optional[int],
                                dtype: Any, device: str) -> Tuple[Dict[str, Any], Dict[str, Any]]:
        return {}, {}

    def apply_quantization(self, model: Any, quant_config: Dict[str, Any], dtype: Any, device: str):
        if self.quantizer is None:
            logging.info("No quantizer provided; skipping quantization.")
            return None
        return self.quantizer.quantize_model(model, quant_config, dtype, device)

    def apply_offloading(self, model: Any, device_map: Dict[str, Any], draft_model: Any = None):
        if self.offloader is None:
            logging.info("No offloader provided; skipping offloading.")
            return None
        return self.offloader(model, device_map=device_map, draft_model=draft_model)


class Recipe(QuantOffloadRecipe):
    """SubSpec: the draft is the target with every attention and MLP projection in 4-bit, group 64 along the input
    dimension; the target keeps 16-bit weights, and the projections of ``keep_first_n_layers_on_gpu ..`` are held in
    host memory and streamed (recipes/subspec/hqq_4bit_postspec.py:10-58 offloads every quantized layer, i.e.
    ``keep_first_n_layers_on_gpu = 0``, the default here too)."""

    def __init__(self, keep_first_n_layers_on_gpu: int = 0, nbits: int = 4, group_size: int = 64,
                 prefetch_slabs: Optional[int] = None):
        super().__init__()
        self.quantizer = HqqQuantizer
        self.offloader = PrefetchOffloader
        self.keep_first_n_layers_on_gpu = int(keep_first_n_layers_on_gpu)
        self.nbits, self.group_size = int(nbits), int(group_size)
        # Device slabs of the streaming ring (None: the offloader's default of 4).  The copies of the next forward run
        # that many layers ahead, through verification and speculation; with a deep draft tree (the reference's
        # depth 48: 100 ms of speculation per cycle) a deeper ring keeps the link busy for all of it, at 466 MB of HBM
        # per slab at the Qwen2.5-7B shape.
        self.prefetch_slabs = prefetch_slabs

    def apply_offloading(self, model, device_map, draft_model=None):
        if self.prefetch_slabs is None:
            return super().apply_offloading(model, device_map, draft_model=draft_model)
        return self.offloader(model, device_map=device_map, draft_model=draft_model, n_slabs=self.prefetch_slabs)

    def generate_configurations(self, target_model, draft_model, max_length, cpu_offload_gb, dtype, device):
        layer_cnt = len(target_model.model.layers)
        per_layer = BaseQuantizeConfig(nbits=self.nbits, group_size=self.group_size, axis=1)
        quant_config = {f"model.layers.{i}.{p}": per_layer for i in range(layer_cnt) for p in PROJECTIONS}
        start = max(0, min(self.keep_first_n_layers_on_gpu, layer_cnt))
        on_cpu = {f"model.layers.{i}.{p}" for i in range(start, layer_cnt) for p in PROJECTIONS}
        target_config = {"device_map": _module_devices(target_model, device, on_cpu)} if on_cpu else {}
        return target_config, {"quant_config": quant_config}


class LayerOffloadRecipe(QuantOffloadRecipe):
    """Offload all decoder layers after the first N, no quantization (recipes/offload/layer_offload.py:9-56)."""

    def __init__(self, keep_first_n_layers_on_gpu: int = 0):
        super().__init__()
        self.quantizer = None
        self.offloader = Offloader
        self.keep_first_n_layers_on_gpu = int(keep_first_n_layers_on_gpu)

    def generate_configurations(self, target_model, draft_model, max_length, cpu_offload_gb, dtype, device):
        layer_cnt = len(target_model.model.layers)
        start = max(0, min(self.keep_first_n_layers_on_gpu, layer_cnt))
        on_cpu = {f"model.layers.{i}.{p}" for i in range(start, layer_cnt) for p in PROJECTIONS}
        return {"device_map": _module_devices(target_model, device, on_cpu), "quant_config": None}, None
