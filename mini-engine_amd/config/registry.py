"""One registry from an architecture's name to the functions that describe it.

The name is ``config.json``'s ``architectures[0]``. When that key is absent the ``model_type`` key
is looked up instead (the reference keys on ``model_type`` and takes ``qwen3`` when it is absent too,
``src/mini_engine/model.py:37``).
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Any, Callable

from .specs import ModelPlan


@dataclass(frozen=True)
class ArchitectureEntry:
    name: str
    config_from_dict: Callable[..., Any]
    config_from_folder: Callable[[str], Any]
    plan_from_config: Callable[[Any], ModelPlan]
    model_types: tuple[str, ...] = field(default_factory=tuple)


_ARCHITECTURES: dict[str, ArchitectureEntry] = {}
_DEFAULT_MODEL_TYPE = "qwen3"
_MODEL_TYPE_TO_NAME = {"qwen3": "Qwen3ForCausalLM"}


def register_architecture(entry: ArchitectureEntry) -> None:
    _ARCHITECTURES[entry.name] = entry
    for t in entry.model_types:
        _MODEL_TYPE_TO_NAME[t] = entry.name


def architecture_names() -> list[str]:
    return sorted(_ARCHITECTURES)


def get_architecture(name: str) -> ArchitectureEntry:
    if name not in _ARCHITECTURES:
        raise ValueError(
            f"unknown architecture {name!r}; registered: {', '.join(architecture_names()) or '(none)'}"
        )
    return _ARCHITECTURES[name]


def architecture_name_of(cfg: dict[str, Any]) -> str:
    archs = cfg.get("architectures")
    if archs:
        return str(archs[0])
    model_type = cfg.get("model_type", _DEFAULT_MODEL_TYPE)
    if model_type not in _MODEL_TYPE_TO_NAME:
        raise ValueError(f"config.json names no architecture and model_type={model_type!r} is unknown")
    return _MODEL_TYPE_TO_NAME[model_type]


def read_config_json(folder: str) -> dict[str, Any]:
    path = os.path.join(folder, "config.json")
    if not os.path.exists(path):
        raise FileNotFoundError(f"{folder!r} holds no config.json")
    with open(path) as f:
        return json.load(f)


def plan_from_folder(folder: str) -> tuple[Any, ModelPlan]:
    """(typed architecture config, model plan) of the model folder, chosen by its config.json."""
    entry = get_architecture(architecture_name_of(read_config_json(folder)))
    config = entry.config_from_folder(folder)
    return config, entry.plan_from_config(config)
