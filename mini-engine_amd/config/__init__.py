from .engine_config import EngineConfig
from .registry import (
    ArchitectureEntry,
    architecture_name_of,
    architecture_names,
    get_architecture,
    plan_from_folder,
    read_config_json,
    register_architecture,
)
from .specs import AttentionSpec, GatedMlpSpec, LayerSpec, ModelPlan, NormSpec, RotarySpec

__all__ = [
    "ArchitectureEntry",
    "AttentionSpec",
    "EngineConfig",
    "GatedMlpSpec",
    "LayerSpec",
    "ModelPlan",
    "NormSpec",
    "RotarySpec",
    "architecture_name_of",
    "architecture_names",
    "get_architecture",
    "plan_from_folder",
    "read_config_json",
    "register_architecture",
]
