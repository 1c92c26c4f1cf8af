"""Typed descriptions of the parts a decoder is assembled from.

A model is described by data only: a tuple of :class:`LayerSpec` (what each layer is made of), an
execution ``order`` (a list of layer indices, which may name a layer twice), and a few model-wide
sizes. Nothing in here knows an architecture's name; an architecture module turns its own
``config.json`` keys into these specs (see ``models/qwen3.py``).

Every spec is a frozen dataclass with a ``kind`` string. The part registries in
``parts/base.py`` map ``kind`` to the class that implements it, so a new kind of mixer,
feed-forward, norm or position encoding is added by registering a (spec, implementation) pair; no
spec in this file has to change for that.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any


@dataclass(frozen=True)
class NormSpec:
    """Root-mean-square norm over the last ``dim`` elements: ``x * rsqrt(mean(x^2) + eps) * w``."""

    dim: int
    eps: float
    kind: str = "rmsnorm"


@dataclass(frozen=True)
class RotarySpec:
    """Rotate-half rotary position encoding over the first ``rotary_dim`` elements of each head.

    ``inv_freq[j] = theta ** (-2j / rotary_dim)``; pairs are ``(j, j + rotary_dim/2)``.
    """

    rotary_dim: int
    theta: float
    kind: str = "rotary"


@dataclass(frozen=True)
class AttentionSpec:
    """Causal grouped-query attention over a paged key/value cache.

    ``window == 0`` means every earlier key is visible; ``window == w`` means a query at position
    ``p`` sees keys ``p-w+1 .. p``. ``qk_norm_eps`` is ``None`` when q and k are not normalised per
    head. ``position`` is ``None`` for a mixer without position encoding. ``cache_from`` names
    another layer (index into ``ModelPlan.layers``) whose keys and values this layer reads instead
    of writing its own.
    """

    hidden_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float
    qk_norm_eps: float | None = None
    window: int = 0
    position: Any | None = None
    cache_from: int | None = None
    kind: str = "attention"

    @property
    def kv_elements_per_token(self) -> int:
        """Key and value elements one token occupies in this layer's own pages (none when it reads another's)."""
        return 0 if self.cache_from is not None else 2 * self.num_kv_heads * self.head_dim


@dataclass(frozen=True)
class GatedMlpSpec:
    """Dense gated feed-forward: ``down(act(gate(x)) * up(x))`` without biases; ``activation`` is "silu" or
    "gelu_tanh"."""

    hidden_size: int
    intermediate_size: int
    activation: str = "silu"
    kind: str = "gated_mlp"


@dataclass(frozen=True)
class LayerSpec:
    """One residual block: which mixer, which feed-forward, which norms, and how they are arranged.

    ``arrangement == "pre_norm"``: ``x += mixer(norm1(x)); x += ffn(norm2(x))``.
    The ``*_prefix`` / ``*_name`` strings are the checkpoint names of this layer's tensors.
    """

    mixer: Any
    ffn: Any
    mixer_norm: Any
    ffn_norm: Any
    mixer_prefix: str
    ffn_prefix: str
    mixer_norm_name: str
    ffn_norm_name: str
    arrangement: str = "pre_norm"


@dataclass(frozen=True)
class ModelPlan:
    """Everything the generic decoder needs to build itself."""

    architecture: str
    vocab_size: int
    hidden_size: int
    layers: tuple[LayerSpec, ...]
    order: tuple[int, ...]
    final_norm: Any
    embed_name: str
    final_norm_name: str
    head_name: str
    tie_word_embeddings: bool
    max_position_embeddings: int
    eos_token_ids: tuple[int, ...] = field(default_factory=tuple)
    embedding_multiplier: float | None = None  # the looked-up rows are multiplied by it (None: as they are)
    logit_scale: float | None = None  # the logits are multiplied by it (None: as they are)

    def __post_init__(self) -> None:
        n = len(self.layers)
        if not self.order:
            raise ValueError("ModelPlan.order is empty")
        for i in self.order:
            if not 0 <= i < n:
                raise ValueError(f"ModelPlan.order names layer {i}, but there are {n} layers")
