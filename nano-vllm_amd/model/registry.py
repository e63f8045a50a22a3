"""Model registry: config.json -> (configuration, model class), by architecture name.

A checkpoint directory names its design in config.json, either as ``"architecture": "<Name>"`` or in the
Hugging Face form ``"architectures": ["<Name>ForCausalLM"]``.  `build_model` reads it, builds the registered model
in the requested dtype on the device and loads ``*.safetensors`` from the same directory.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, fields
from typing import Callable

import torch


@dataclass
class Entry:
    make_config: Callable[[dict], object]
    make_model: Callable[..., torch.nn.Module]         # (config, dtype=, device=) -> model


_REGISTRY: dict[str, Entry] = {}


def register(names, make_config, make_model) -> None:
    for n in ([names] if isinstance(names, str) else names):
        _REGISTRY[n] = Entry(make_config, make_model)


def architectures() -> list[str]:
    return sorted(_REGISTRY)


def architecture_of(config: dict) -> str:
    name = config.get("architecture")
    if name is None:
        archs = config.get("architectures") or []
        name = archs[0] if archs else None
    if name is None:
        raise ValueError("config.json names no architecture")
    if name not in _REGISTRY:
        raise ValueError(f"unknown architecture {name!r}; known: {architectures()}")
    return name


def read_config(model_dir: str) -> dict:
    with open(os.path.join(model_dir, "config.json")) as f:
        return json.load(f)


def build_model(model_dir: str, dtype: torch.dtype = torch.bfloat16, device="cuda", load_weights: bool = True,
                **model_kwargs):
    """Returns (model, config object) for the checkpoint directory."""
    from ..utils.loader import load_model
    raw = read_config(model_dir)
    entry = _REGISTRY[architecture_of(raw)]
    cfg = entry.make_config(raw)
    model = entry.make_model(cfg, dtype=dtype, device=device, **model_kwargs)
    if load_weights:
        load_model(model, model_dir)
    return model, cfg


# ---- the registered designs ------------------------------------------------------------------------------------
def _qwen3_config(raw: dict):
    from .qwen3 import ModelConfig
    known = {f.name for f in fields(ModelConfig)}
    kw = {k: v for k, v in raw.items() if k in known}
    if "head_dim" not in kw and "hidden_size" in raw and "num_attention_heads" in raw:
        kw["head_dim"] = raw["hidden_size"] // raw["num_attention_heads"]
    return ModelConfig(**kw)


def _qwen3_model(cfg, dtype=torch.bfloat16, device="cuda", **kw):
    from .qwen3 import Qwen3ForCausalLM
    if dtype != torch.bfloat16:
        raise ValueError("the Qwen3 / Llama path runs in bfloat16 only")
    return Qwen3ForCausalLM(cfg, **kw).to(device=device, dtype=dtype)


def _buvalix_config(raw: dict):
    from .buvalix import BuvalixConfig
    return BuvalixConfig.from_dict(raw)


def _buvalix_model(cfg, dtype=torch.bfloat16, device="cuda", **kw):
    from .buvalix import BuvalixForCausalLM
    return BuvalixForCausalLM(cfg, dtype=dtype, device=device, **kw)


def _benarax_config(raw: dict):
    from .benarax import BenaraxConfig
    return BenaraxConfig.from_dict(raw)


def _benarax_model(cfg, dtype=torch.bfloat16, device="cuda", **kw):
    from .benarax import BenaraxForCausalLM
    return BenaraxForCausalLM(cfg, dtype=dtype, device=device, **kw)


def _divadra_config(raw: dict):
    from .divadra import DivadraConfig
    return DivadraConfig.from_dict(raw)


def _divadra_model(cfg, dtype=torch.bfloat16, device="cuda", **kw):
    from .divadra import DivadraForCausalLM
    return DivadraForCausalLM(cfg, dtype=dtype, device=device, **kw)


def _tutedra_config(raw: dict):
    from .tutedra import TutedraConfig
    return TutedraConfig.from_dict(raw)


def _tutedra_model(cfg, dtype=torch.bfloat16, device="cuda", **kw):
    from .tutedra import TutedraForCausalLM
    return TutedraForCausalLM(cfg, dtype=dtype, device=device, **kw)


register(["Qwen3ForCausalLM", "Qwen3"], _qwen3_config, lambda cfg, **kw: _qwen3_model(cfg, **kw))
register(["LlamaForCausalLM", "Llama"], lambda raw: _qwen3_config({**raw, "qk_norm": False}),
         lambda cfg, **kw: _qwen3_model(cfg, **kw))
register(["Buvalix", "BuvalixForCausalLM"], _buvalix_config, _buvalix_model)
register(["Benarax", "BenaraxForCausalLM"], _benarax_config, _benarax_model)
register(["Divadra", "DivadraForCausalLM"], _divadra_config, _divadra_model)
register(["Tutedra", "TutedraForCausalLM"], _tutedra_config, _tutedra_model)
