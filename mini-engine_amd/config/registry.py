"""One registry from an architecture's name to the functions that describe it.

The name is ``config.json``'s ``architectures[0]``. When that key is absent the ``model_type`` key
is looked up among the model types that the registered entries claim (the reference keys on
``model_type``, ``src/mini_engine/model.py:37``); an entry may also claim configs that name neither
(``default_for_unnamed``, as the reference takes a config without ``model_type`` for its one model).
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
    default_for_unnamed: bool = False  # takes a config.json that names neither architectures nor model_type


_ARCHITECTURES: dict[str, ArchitectureEntry] = {}
_MODEL_TYPE_TO_NAME: dict[str, str] = {}
_UNNAMED: list[str] = []


def register_architecture(entry: ArchitectureEntry) -> None:
    _ARCHITECTURES[entry.name] = entry
    for t in entry.model_types:
        _MODEL_TYPE_TO_NAME[t] = entry.name
    if entry.default_for_unnamed and entry.name not in _UNNAMED:
        _UNNAMED.append(entry.name)


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
    model_type = cfg.get("model_type")
    if model_type is None:
        if len(_UNNAMED) != 1:
            raise ValueError("config.json names neither an architecture nor a model_type")
        return _UNNAMED[0]
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
