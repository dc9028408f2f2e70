"""What the reference's ``ModelRegistry.register`` stores for a method (run/core/registry.py:71-97), for this build:
``load_model_fn(builder, model_path)``, ``load_draft_model_fn(builder, target_model, tokenizer, draft_model_path)``,
``load_kv_cache_fn(builder, target_model, draft_model)`` with the signatures ``GeneratorPipelineBuilder`` calls them
with (run/core/builder.py:86-160), and ``register(ModelRegistry)``, which makes the exact registration calls.

Nothing here imports the reference; ``builder`` is duck-typed: the attributes read are ``dtype``, ``device``,
``recipe``, ``cache_implementation``, ``max_length``, ``draft_params`` -- the ones the reference's default loaders
read (builder.py:94-103,119-131,146-198).
"""
from __future__ import annotations

import os
from typing import Any, Optional, Tuple

import torch

from .cache import create_kv_cache
from .hf_model import CausalLM, _hf_config_of
from .utils import DraftParams

METHODS = {
    "subspec_sd": ("subspec_amd.generator:SubSpecSDGenerator", "subspec_amd.draft:SubSpecSDDraftModel"),
    "subspec_sd_v2": ("subspec_amd.generator_v2:SubSpecSDGeneratorV2", "subspec_amd.draft:SubSpecSDDraftModel"),
}


def load_model_fn(builder: Any, model_path: str):
    """(model, tokenizer) from a LOCAL checkpoint directory.  The model is loaded to the CPU when the recipe has an
    offloader (which then places it), else to ``builder.device`` -- the rule of builder.py:96-97.  The tokenizer is
    read from the same directory when its files are there; a directory with weights only yields ``None`` (the
    generator then needs ``eos_token_id`` from its caller and rejects ``stop_strings``)."""
    recipe = getattr(builder, "recipe", None)
    offloaded = bool(recipe is not None and getattr(recipe, "offloader", None))
    model = CausalLM.from_pretrained(model_path, torch_dtype=getattr(builder, "dtype", torch.bfloat16),
                                     device_map="cpu" if offloaded else getattr(builder, "device", "cuda:0"))
    tokenizer = None
    if any(os.path.exists(os.path.join(model_path, f)) for f in ("tokenizer.json", "tokenizer.model", "vocab.json")):
        from transformers import AutoTokenizer
        tokenizer = AutoTokenizer.from_pretrained(model_path, local_files_only=True)
    return model, tokenizer


def load_draft_model_fn(builder: Any, target_model: Any, tokenizer: Any, draft_model_path: Optional[str] = None):
    """The substitute draft: a second module tree over the target's parameters, which the recipe's quantizer then
    turns into int4 (``draft_model_cls.from_pretrained(draft_model_path, target_model=..., torch_dtype=...,
    eos_token_id=..., device_map=...)``, builder.py:119-131; SubSpec has no draft checkpoint, the path is unused)."""
    from .draft import SubSpecSDDraftModel
    return SubSpecSDDraftModel.from_pretrained(draft_model_path, target_model=target_model,
                                               torch_dtype=getattr(builder, "dtype", torch.bfloat16),
                                               eos_token_id=getattr(tokenizer, "eos_token_id", None),
                                               device_map=getattr(builder, "device", "cuda:0"))


def _verify_headroom(draft_params: Any) -> int:
    """Rows beyond ``max_length`` that one cycle's tree may occupy (the rule of builder.py:152-190)."""
    if not draft_params:
        return 0
    get = draft_params.get if isinstance(draft_params, dict) else lambda k, d=None: getattr(draft_params, k, d)
    for key in ("max_verify_tokens", "max_sample_tokens"):
        if get(key) is not None:
            return int(get(key))
    if get("max_depth") is not None and get("topk_len") is not None:
        return int(get("max_depth")) * int(get("topk_len")) + 1
    return 0


def load_kv_cache_fn(builder: Any, target_model: Any, draft_model: Any) -> Tuple[Any, None]:
    """(past_key_values, None): ONE cache shared by target and draft (``needs_draft_kv_cache=False``,
    run/core/presets.py:153), as ``KVManager`` over this build's single-tensor layout."""
    impl = getattr(builder, "cache_implementation", "static")
    cfg = _hf_config_of(target_model)
    device = getattr(builder, "device", "cuda:0")
    dtype = getattr(target_model, "dtype", None) or getattr(builder, "dtype", torch.bfloat16)
    max_length = getattr(builder, "max_length", None)
    if impl == "dynamic":
        return create_kv_cache("dynamic", max_cache_len=max_length, config=cfg, device=device, dtype=dtype), None
    if max_length is None:
        raise ValueError("max_length should be set for static cache.")
    rows = int(max_length) + _verify_headroom(getattr(builder, "draft_params", None))
    return create_kv_cache(impl, max_cache_len=rows, max_batch_size=1, config=cfg, device=device, dtype=dtype), None


def register(model_registry: Any, recipe: Any = None, llm_path: Optional[str] = None) -> None:
    """Registers ``subspec_sd`` and ``subspec_sd_v2`` on the reference's ``ModelRegistry`` class (passed in, so this
    module does not import it)."""
    from .recipes import Recipe
    for name, (generator_cls, draft_model_cls) in METHODS.items():
        model_registry.register(
            name=name, generator_cls=generator_cls, draft_model_cls=draft_model_cls,
            default_config={"recipe": recipe if recipe is not None else Recipe(), "llm_path": llm_path},
            load_model_fn=load_model_fn, load_draft_model_fn=load_draft_model_fn, load_kv_cache_fn=load_kv_cache_fn,
            needs_draft_kv_cache=False)
