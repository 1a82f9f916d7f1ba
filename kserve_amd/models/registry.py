"""Model registry: config.json -> (config class, model class).

A model directory names its design either with the HuggingFace keys
(``architectures`` / ``model_type``) or with a single ``architecture`` key.
Model classes are imported lazily so that choosing one design does not
import (or compile) the others.
"""

from __future__ import annotations

import json
import os
from typing import Callable, Dict, Tuple

# architecture name -> (config loader path, model class path, native modules)
_REGISTRY: Dict[str, Tuple[str, str, Tuple[str, ...]]] = {}


def register(name: str, config_cls: str, model_cls: str, native: Tuple[str, ...]):
    _REGISTRY[name.lower()] = (config_cls, model_cls, native)


def _resolve(path: str):
    mod, _, attr = path.rpartition(".")
    import importlib

    return getattr(importlib.import_module(mod), attr)


_LLAMA = (
    "kserve_amd.engine.config.ModelConfig",
    "kserve_amd.models.llama.LlamaForCausalLM",
    ("kserve_amd_C",),
)
for _name in (
    "llama", "mistral", "mixtral", "qwen2",
    "LlamaForCausalLM", "MistralForCausalLM", "MixtralForCausalLM",
    "Qwen2ForCausalLM",
):
    register(_name, *_LLAMA)
register(
    "Merulorn",
    "kserve_amd.engine.config.HybridModelConfig",
    "kserve_amd.models.merulorn.MerulornForCausalLM",
    ("kserve_amd_seq_C",),
)
register(
    "Desalix",
    "kserve_amd.engine.config.HybridModelConfig",
    "kserve_amd.models.desalix.DesalixForCausalLM",
    ("kserve_amd_seq_C",),
)
register(
    "Voborax",
    "kserve_amd.engine.config.HybridModelConfig",
    "kserve_amd.models.voborax.VoboraxForCausalLM",
    ("kserve_amd_seq_C",),
)
register(
    "Laperax",
    "kserve_amd.engine.config.HybridModelConfig",
    "kserve_amd.models.laperax.LaperaxForCausalLM",
    ("kserve_amd_seq_C",),
)


def architecture_of(config_json: dict) -> str:
    if "architecture" in config_json:
        return str(config_json["architecture"])
    archs = config_json.get("architectures") or []
    if archs:
        return str(archs[0])
    return str(config_json.get("model_type", "llama"))


def lookup(name: str):
    try:
        return _REGISTRY[name.lower()]
    except KeyError:
        raise ValueError(
            f"unknown model architecture {name!r}; known: {sorted(_REGISTRY)}"
        ) from None


def load_model_config(model_dir: str):
    """Read ``model_dir/config.json`` into the config class of its design."""
    path = os.path.join(model_dir, "config.json")
    with open(path) as f:
        cfg = json.load(f)
    config_cls, _, _ = lookup(architecture_of(cfg))
    return _resolve(config_cls).from_hf_config(path)


def native_modules_for(model_dir: str) -> Tuple[str, ...]:
    """Names of the compiled extension modules the design runs on."""
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    return lookup(architecture_of(cfg))[2]


def model_class_for(config) -> Callable:
    """Model class for an in-memory config object."""
    name = getattr(config, "architecture", None) or "llama"
    return _resolve(lookup(name)[1])


def build_model(config, device: str = "cpu", dtype=None):
    return model_class_for(config)(config, dtype=dtype, device=device)
