"""The Qwen3 dense decoder: its ``config.json`` keys, and the plan that assembles it from parts.

Formulas and key handling follow the reference's ``src/mini_engine/model.py``:

* keys read, defaults and the three rejections: ``model.py:35-56``
  (``model_type`` must be ``qwen3``; ``rope_parameters.rope_type`` must be ``default``;
  ``use_sliding_window`` must be falsy; ``head_dim`` defaults to ``hidden_size // num_attention_heads``;
  ``rope_theta`` comes from ``rope_parameters`` first, then the top level, then 10000.0);
* layer contents: attention with per-head q/k RMSNorm and rotate-half RoPE ``model.py:93-119``,
  SwiGLU feed-forward ``model.py:122-131``, pre-norm residual block ``model.py:134-151``,
  embedding / final norm / optionally tied head ``model.py:154-170``;
* checkpoint tensor names are the module names of ``model.py:97-103, 125-127, 137-140, 157-159, 168``;
* end-of-sequence ids: ``generation_config.json`` first, else ``config.json``
  (``engine.py:130-133``), normalised like ``engine.py:302-307``.
"""

from __future__ import annotations

import json
import os
from dataclasses import asdict, dataclass
from typing import Any

from ..config.registry import ArchitectureEntry, register_architecture
from ..config.specs import AttentionSpec, GatedMlpSpec, LayerSpec, ModelPlan, NormSpec, RotarySpec

ARCHITECTURE = "Qwen3ForCausalLM"


@dataclass(frozen=True)
class Qwen3Config:
    """The numbers of ``config.json`` that the forward pass uses, under their own key names."""

    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    tie_word_embeddings: bool
    eos_token_ids: tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, cfg: dict[str, Any], eos: Any = None) -> "Qwen3Config":
        model_type = cfg.get("model_type", "qwen3")
        if model_type != "qwen3":
            raise ValueError(f"only qwen3 is supported by this architecture entry, got model_type={model_type!r}")
        rope = cfg.get("rope_parameters") or cfg.get("rope_scaling") or {}
        rope_type = rope.get("rope_type", rope.get("type", "default"))
        if rope_type != "default":
            raise ValueError(f"only default RoPE is supported, got rope_type={rope_type!r}")
        if cfg.get("use_sliding_window", False):
            raise ValueError("sliding-window attention is not supported for Qwen3 (use_sliding_window is set)")
        if cfg.get("attention_bias", False):
            raise ValueError("attention_bias=true is not supported: every projection is bias-free")
        missing = [
            k
            for k in (
                "vocab_size",
                "hidden_size",
                "intermediate_size",
                "num_hidden_layers",
                "num_attention_heads",
                "num_key_value_heads",
                "rms_norm_eps",
                "max_position_embeddings",
                "tie_word_embeddings",
            )
            if k not in cfg
        ]
        if missing:
            raise ValueError(f"config.json lacks required keys: {', '.join(missing)}")
        heads = int(cfg["num_attention_heads"])
        kv_heads = int(cfg["num_key_value_heads"])
        head_dim = cfg.get("head_dim") or int(cfg["hidden_size"]) // heads
        if heads % kv_heads != 0:
            raise ValueError(f"num_attention_heads={heads} is not a multiple of num_key_value_heads={kv_heads}")
        if int(head_dim) % 2 != 0:
            raise ValueError(f"head_dim={head_dim} must be even for rotate-half RoPE")
        theta = rope.get("rope_theta", cfg.get("rope_theta", 10000.0))
        if eos is None:
            eos = cfg.get("eos_token_id")
        return cls(
            vocab_size=int(cfg["vocab_size"]),
            hidden_size=int(cfg["hidden_size"]),
            intermediate_size=int(cfg["intermediate_size"]),
            num_hidden_layers=int(cfg["num_hidden_layers"]),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=int(head_dim),
            rms_norm_eps=float(cfg["rms_norm_eps"]),
            rope_theta=float(theta),
            max_position_embeddings=int(cfg["max_position_embeddings"]),
            tie_word_embeddings=bool(cfg["tie_word_embeddings"]),
            eos_token_ids=as_id_tuple(eos),
        )

    @classmethod
    def from_folder(cls, folder: str) -> "Qwen3Config":
        with open(os.path.join(folder, "config.json")) as f:
            cfg = json.load(f)
        eos = None
        gen_path = os.path.join(folder, "generation_config.json")
        if os.path.exists(gen_path):
            with open(gen_path) as f:
                eos = json.load(f).get("eos_token_id")
        return cls.from_dict(cfg, eos)

    def to_config_json(self) -> dict[str, Any]:
        """A ``config.json`` dictionary that :meth:`from_dict` reads back to an equal object."""
        d = asdict(self)
        eos = d.pop("eos_token_ids")
        d["architectures"] = [ARCHITECTURE]
        d["model_type"] = "qwen3"
        d["use_sliding_window"] = False
        d["attention_bias"] = False
        d["hidden_act"] = "silu"
        d["eos_token_id"] = None if not eos else (eos[0] if len(eos) == 1 else list(eos))
        return d


def as_id_tuple(eos: Any) -> tuple[int, ...]:
    if eos is None:
        return ()
    if isinstance(eos, int):
        return (eos,)
    return tuple(int(e) for e in eos)


def plan_from_config(cfg: Qwen3Config) -> ModelPlan:
    """Every layer: attention (q/k norm, rotary, all keys visible) then SwiGLU, pre-norm."""
    rotary = RotarySpec(rotary_dim=cfg.head_dim, theta=cfg.rope_theta)
    layers = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}"
        layers.append(
            LayerSpec(
                mixer=AttentionSpec(
                    hidden_size=cfg.hidden_size,
                    num_heads=cfg.num_attention_heads,
                    num_kv_heads=cfg.num_key_value_heads,
                    head_dim=cfg.head_dim,
                    scale=cfg.head_dim**-0.5,
                    qk_norm_eps=cfg.rms_norm_eps,
                    window=0,
                    position=rotary,
                ),
                ffn=GatedMlpSpec(
                    hidden_size=cfg.hidden_size, intermediate_size=cfg.intermediate_size, activation="silu"
                ),
                mixer_norm=NormSpec(dim=cfg.hidden_size, eps=cfg.rms_norm_eps),
                ffn_norm=NormSpec(dim=cfg.hidden_size, eps=cfg.rms_norm_eps),
                mixer_prefix=f"{p}.self_attn",
                ffn_prefix=f"{p}.mlp",
                mixer_norm_name=f"{p}.input_layernorm.weight",
                ffn_norm_name=f"{p}.post_attention_layernorm.weight",
                arrangement="pre_norm",
            )
        )
    return ModelPlan(
        architecture=ARCHITECTURE,
        vocab_size=cfg.vocab_size,
        hidden_size=cfg.hidden_size,
        layers=tuple(layers),
        order=tuple(range(cfg.num_hidden_layers)),
        final_norm=NormSpec(dim=cfg.hidden_size, eps=cfg.rms_norm_eps),
        embed_name="model.embed_tokens.weight",
        final_norm_name="model.norm.weight",
        head_name="lm_head.weight",
        tie_word_embeddings=cfg.tie_word_embeddings,
        max_position_embeddings=cfg.max_position_embeddings,
        eos_token_ids=cfg.eos_token_ids,
    )


register_architecture(
    ArchitectureEntry(
        name=ARCHITECTURE,
        config_from_dict=Qwen3Config.from_dict,
        config_from_folder=Qwen3Config.from_folder,
        plan_from_config=plan_from_config,
        model_types=("qwen3",),
        default_for_unnamed=True,
    )
)
