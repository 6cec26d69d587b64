"""The one registry from an architecture's name to its configuration and plan.

``config.json["architectures"][0]`` selects the entry. The reference never
reads that key (it serves one pinned checkpoint, engine/dryft_qwen3/config.py:55-70);
here it is the only place where a model is chosen.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable

from ..config.base import ConfigError
from ..config.plan import ModelPlan


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: Any                       # has from_dict(raw) and to_dict()
    plan: Callable[[Any], ModelPlan]        # typed config -> ModelPlan


_REGISTRY: dict[str, Architecture] = {}
_MODEL_TYPES: dict[str, str] = {}      # config.json "model_type" -> architecture name, for files without "architectures"


def register_architecture(name: str, config_class: Any, plan: Callable[[Any], ModelPlan],
                          model_type: str | None = None) -> None:
    if name in _REGISTRY:
        raise ValueError(f"architecture {name!r} is already registered")
    _REGISTRY[name] = Architecture(name, config_class, plan)
    if model_type is not None:
        _MODEL_TYPES[model_type] = name


def known_architectures() -> list[str]:
    return sorted(_REGISTRY)


def resolve_architecture(raw_config: dict[str, Any]) -> Architecture:
    names = raw_config.get("architectures")
    if names is None and raw_config.get("model_type") in _MODEL_TYPES:
        names = [_MODEL_TYPES[raw_config["model_type"]]]          # a config.json that only says model_type
    if not isinstance(names, list) or not names or not isinstance(names[0], str):
        raise ConfigError("config.json", [
            f"architectures: expected a list naming the model class, got {names!r}; known: {known_architectures()}"])
    arch = _REGISTRY.get(names[0])
    if arch is None:
        raise ConfigError("config.json", [
            f"architectures: {names[0]!r} is not registered; known: {known_architectures()}"])
    return arch


_PRESET_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "presets")


def preset_names() -> list[str]:
    return sorted(f[:-5] for f in os.listdir(_PRESET_DIR) if f.endswith(".json"))


def load_preset(name: str) -> dict:
    """A named ``config.json`` shipped as data: sizes live in the file, not in code, and the file's own
    ``architectures`` entry says which registered model it is for."""
    path = os.path.join(_PRESET_DIR, name + ".json")
    if not os.path.isfile(path):
        raise KeyError(f"unknown preset {name!r}; known: {preset_names()}")
    with open(path, "r", encoding="utf-8") as f:
        return json.load(f)


from . import qwen3 as _qwen3  # noqa: E402,F401  (registers Qwen3ForCausalLM)
