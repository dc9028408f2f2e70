"""The model objects the reference's builder passes around, and their conversion into this package's decoders.

The reference's pipeline builder (run/core/builder.py:86-350) handles a HuggingFace ``*ForCausalLM`` module: the
recipe reads ``model.model.layers`` and ``named_parameters()`` (recipes/subspec/hqq_4bit_postspec.py:17-58), the
quantizer replaces ``nn.Linear`` modules by name (quantizers/hqq/__init__.py:17-120), the offloader is called as
``cls(model, device_map=..., draft_model=...)`` (recipes/base_recipe.py:54-63), the draft shares the target's
parameters (draft_models/subspec_sd.py:11-45), and the generator finally receives both.  ``CausalLM`` is a module
tree with exactly those names (``model.embed_tokens``, ``model.layers.N.self_attn.{q,k,v,o}_proj``,
``model.layers.N.mlp.{gate,up,down}_proj``, the two layer norms, ``model.norm``, ``lm_head``) read from a LOCAL
checkpoint directory, so recipes, quantizer and offloader written against the reference's conventions work on it
unchanged; a real ``transformers`` Qwen2 / Llama module has the same names and is accepted as well.

``as_decoder`` turns such a module (dense, or with ``HqqInt4Linear`` projections, resident or partly streamed) into
the ``Decoder`` the cycle drivers run: q|k|v and gate|up rows fused, int4 tiles concatenated, streamed layers left
in their pinned slabs.
"""
from __future__ import annotations

import json
import os
from types import SimpleNamespace
from typing import Dict, List, Optional

import torch
import torch.nn as nn

from .model import DecoderConfig, Decoder, config_from_hf, layer_shapes
from .quant import HqqInt4Linear

ATTN = ("q_proj", "k_proj", "v_proj", "o_proj")
MLP = ("gate_proj", "up_proj", "down_proj")


class RMSNormWeight(nn.Module):
    """Holder of a norm gain under the name ``weight`` (the arithmetic lives in the HIP kernels)."""

    def __init__(self, weight: torch.Tensor, eps: float):
        super().__init__()
        self.weight = nn.Parameter(weight, requires_grad=False)
        self.variance_epsilon = eps


def _linear(weight: torch.Tensor, bias: Optional[torch.Tensor]) -> nn.Linear:
    lin = nn.Linear(weight.shape[1], weight.shape[0], bias=bias is not None, device="meta")
    lin.weight = nn.Parameter(weight, requires_grad=False)
    if bias is not None:
        lin.bias = nn.Parameter(bias, requires_grad=False)
    return lin


class _Attention(nn.Module):
    pass


class _MLP(nn.Module):
    pass


class _Layer(nn.Module):
    pass


class _Body(nn.Module):
    @property
    def dtype(self) -> torch.dtype:
        return self.embed_tokens.weight.dtype


class CausalLM(nn.Module):
    """HuggingFace-shaped decoder-only model holding weights only (no forward of its own: the cycle drivers run it
    through ``as_decoder``)."""

    def __init__(self, hf_config: dict, tensors: Dict[str, torch.Tensor]):
        super().__init__()
        self.decoder_config = config_from_hf(hf_config)
        cfg = self.decoder_config
        self.config = SimpleNamespace(**dict(hf_config, head_dim=cfg.head_dim,
                                             model_type=hf_config.get("model_type", "qwen2")))

        def take(name, required=True):
            t = tensors.get(name)
            if t is None and required:
                raise KeyError(f"{name} missing from the checkpoint")
            return t

        body = _Body()
        body.config = self.config
        body.embed_tokens = nn.Embedding(cfg.vocab_size, cfg.hidden_size, device="meta")
        body.embed_tokens.weight = nn.Parameter(take("model.embed_tokens.weight"), requires_grad=False)
        layers = []
        for i in range(cfg.num_hidden_layers):
            p = f"model.layers.{i}."
            layer, attn, mlp = _Layer(), _Attention(), _MLP()
            for n in ATTN:
                setattr(attn, n, _linear(take(p + f"self_attn.{n}.weight"), take(p + f"self_attn.{n}.bias", False)))
            for n in MLP:
                setattr(mlp, n, _linear(take(p + f"mlp.{n}.weight"), take(p + f"mlp.{n}.bias", False)))
            layer.self_attn, layer.mlp = attn, mlp
            layer.input_layernorm = RMSNormWeight(take(p + "input_layernorm.weight"), cfg.rms_norm_eps)
            layer.post_attention_layernorm = RMSNormWeight(take(p + "post_attention_layernorm.weight"), cfg.rms_norm_eps)
            layers.append(layer)
        body.layers = nn.ModuleList(layers)
        body.norm = RMSNormWeight(take("model.norm.weight"), cfg.rms_norm_eps)
        self.model = body
        head = take("lm_head.weight", False)
        self.lm_head = _linear(head if head is not None else body.embed_tokens.weight.data, None)
        if head is None:                                              # tie_word_embeddings
            self.lm_head.weight = body.embed_tokens.weight

    @property
    def dtype(self) -> torch.dtype:
        return self.model.dtype

    @property
    def device(self) -> torch.device:
        return self.model.embed_tokens.weight.device

    def forward(self, *args, **kwargs):
        raise RuntimeError("CausalLM holds weights only; run it through SubSpecSDGenerator (subspec_amd.hf_model.as_decoder)")

    @classmethod
    def from_pretrained(cls, path: str, torch_dtype: torch.dtype = torch.bfloat16, device_map="cpu", **_unused) -> "CausalLM":
        """Reads ``config.json`` and every ``*.safetensors`` file of a LOCAL directory (nothing is downloaded; the
        reference's ``AutoModelForCausalLM.from_pretrained(model_path, torch_dtype, device_map)``,
        run/core/builder.py:94-103)."""
        import glob

        from safetensors import safe_open
        if not os.path.isdir(path):
            raise FileNotFoundError(f"{path} is not a local checkpoint directory (model names cannot be downloaded here)")
        with open(os.path.join(path, "config.json")) as f:
            hf = json.load(f)
        files = sorted(glob.glob(os.path.join(path, "*.safetensors")))
        if not files:
            raise FileNotFoundError(f"no .safetensors file in {path}")
        device = "cpu" if device_map in (None, "cpu", "auto") else device_map
        tensors = {}
        for fn in files:
            with safe_open(fn, framework="pt", device="cpu") as sf:
                for key in sf.keys():
                    tensors[key] = sf.get_tensor(key).to(device=device, dtype=torch_dtype)
        return cls(hf, tensors)


def share_parameters(model: nn.Module) -> nn.Module:
    """A second module tree over the SAME parameter tensors (what the reference's ``share_param_deepcopy`` gives the
    substitute draft, draft_models/subspec_sd.py:11-21): modules are new objects, so replacing a projection of the
    copy by a quantized module leaves the original alone, while every parameter that is not replaced stays shared."""
    import copy
    memo = {id(t): t for t in list(model.parameters()) + list(model.buffers())}
    return copy.deepcopy(model, memo)


# ---------------------------------------------------------------------------------------------- conversion
def _hf_config_of(model: nn.Module) -> DecoderConfig:
    if isinstance(getattr(model, "decoder_config", None), DecoderConfig):
        return model.decoder_config
    cfg = model.config
    d = cfg.to_dict() if hasattr(cfg, "to_dict") else dict(vars(cfg))
    return config_from_hf(d)


def _fused_dense(parts: List[nn.Linear], device, dtype) -> torch.Tensor:
    """Rows of several projections in one matrix; the modules' parameters are then re-pointed at row ranges of it,
    so that the weights exist once."""
    fused = torch.cat([p.weight.data.to(device=device, dtype=dtype) for p in parts], 0).contiguous()
    row = 0
    for p in parts:
        n = p.weight.shape[0]
        p.weight.data = fused[row:row + n]
        row += n
    return fused


def layer_tensors(layer: nn.Module, cfg: DecoderConfig, device, dtype) -> Dict[str, torch.Tensor]:
    """One layer of an HF-shaped module in this package's fused layout: dense (``*.weight``) or int4
    (``*.wq`` / ``*.sz`` / ``*.out_features``), as ``model.init_weights`` / ``model.quantize_layers`` produce."""
    a, m = layer.self_attn, layer.mlp
    out: Dict[str, torch.Tensor] = {
        "input_layernorm.weight": layer.input_layernorm.weight.data.to(device=device, dtype=dtype),
        "post_attention_layernorm.weight": layer.post_attention_layernorm.weight.data.to(device=device, dtype=dtype)}
    groups = {"qkv_proj": [a.q_proj, a.k_proj, a.v_proj], "o_proj": [a.o_proj],
              "gate_up_proj": [m.gate_proj, m.up_proj], "down_proj": [m.down_proj]}
    for name, parts in groups.items():
        packed = [isinstance(p, HqqInt4Linear) for p in parts]
        if any(packed) and not all(packed):
            raise NotImplementedError(f"{name}: its projections share one fused matrix, so they must be quantized together")
        if packed[0]:
            out[name + ".wq"] = torch.cat([p.wq.to(device) for p in parts], 0).contiguous() if len(parts) > 1 else parts[0].wq.to(device)
            out[name + ".sz"] = torch.cat([p.sz.to(device) for p in parts], 0).contiguous() if len(parts) > 1 else parts[0].sz.to(device)
            out[name + ".out_features"] = sum(int(p.out_features) for p in parts)
        else:
            out[name + ".weight"] = _fused_dense(parts, device, dtype) if len(parts) > 1 else \
                parts[0].weight.data.to(device=device, dtype=dtype).contiguous()
    biases = [getattr(p, "bias", None) for p in groups["qkv_proj"]]
    sizes = (cfg.q_size, cfg.kv_size, cfg.kv_size)
    out["qkv_proj.bias"] = torch.cat([b.data.to(device=device, dtype=dtype) if b is not None else
                                      torch.zeros(n, device=device, dtype=dtype) for b, n in zip(biases, sizes)], 0)
    if not packed[0]:
        for name, shape in layer_shapes(cfg).items():
            if tuple(out[name].shape) != tuple(shape):
                raise ValueError(f"{name} has shape {tuple(out[name].shape)}, expected {tuple(shape)}")
    return out


def as_decoder(model, kv) -> Decoder:
    """``Decoder`` over the shared cache ``kv`` for a model handed over by the builder.  A ``Decoder`` is returned
    as it is (re-bound to ``kv``); an HF-shaped module is converted once and the result kept on the module.  Layers
    an offloader put into pinned slabs (``subspec_amd.offloaders``) stay there and are streamed."""
    if isinstance(model, Decoder):
        model.bind_cache(kv)
        return model
    dec = getattr(model, "_subspec_decoder", None)
    if dec is not None:
        dec.bind_cache(kv)
        return dec
    if not isinstance(model, nn.Module) or not hasattr(model, "model") or not hasattr(model.model, "layers"):
        raise TypeError(f"{type(model).__name__} is neither a subspec_amd Decoder nor a HuggingFace-shaped causal LM")
    cfg = _hf_config_of(model)
    off = getattr(model, "_subspec_offload", None)            # set by subspec_amd.offloaders
    device = off.device if off is not None else model.model.embed_tokens.weight.device
    if torch.device(device).type != "cuda":
        raise RuntimeError("the model's resident weights are not on a GPU: apply the recipe's offloader, or load the model "
                           "to the device (there is no CPU path)")
    dtype = model.model.embed_tokens.weight.dtype
    first_streamed = off.first_streamed if off is not None else cfg.num_hidden_layers
    layers = [layer_tensors(model.model.layers[i], cfg, device, dtype) for i in range(first_streamed)]
    head = model.lm_head.weight.data if getattr(model, "lm_head", None) is not None else model.model.embed_tokens.weight.data
    dec = Decoder(cfg, model.model.embed_tokens.weight.data.to(device), layers, model.model.norm.weight.data.to(device),
                  head.to(device), kv, off.streamer if off is not None else None, first_streamed)
    model._subspec_decoder = dec
    return dec
