"""Interfaces of the parts a decoder layer is assembled from, and the registries that map a spec's
``kind`` to its implementation.

A part is built from its spec alone (plus the compute dtype and device); it never learns which model
it is in. The four interfaces:

``Norm``               ``weight_wants(name)``, ``load(tensors, name)``, ``weight`` / ``eps`` used by the
                       fused residual-add-and-norm of the block.
``PositionEncoding``   ``tables(num_positions)`` returns what the mixer's kernels read (for rotating
                       encodings: the float32 table of cosines and sines by position).
``Mixer``              ``weight_wants(prefix)``, ``load(tensors, prefix)``, ``cache_need()``,
                       ``forward(h, batch, cache) -> [T, hidden]``.
``FeedForward``        ``weight_wants(prefix)``, ``load(tensors, prefix)``, ``forward(h, batch) -> [T, hidden]``.

A mixer or feed-forward class may set ``takes_normed_input = True``; its ``forward`` is then handed a
``NormedInput`` (the residual add and the norm not yet evaluated) instead of a tensor and passes it
to ``ops.kernels.linear`` as the input of its first matrix product, which fuses both into that
product for decode-sized batches (``h.materialize()`` gives the tensor where it is needed).

A part of the package also has ``emit(program, h, ...)``, which writes its operations into the step program that
every step runs; a part without it enters that program as a call of its ``forward`` (``engine/program.py``).

A part class that sets ``graph_safe = True`` promises that its ``forward`` can be captured into a graph for
decode steps (see :class:`Part`); rows that pad a replayed batch carry the spare page and the spare state
slot, which belong to no request.

``h`` is the normed input [T, hidden] in the compute dtype, ``batch`` a ``StepBatch`` (token
positions, item boundaries, block tables per cache group, state slots), ``cache`` the binding
(``KVBinding`` / ``StateBinding`` / None) of this run of the layer: a layer that the order names
twice has a cache for each run. A mixer states what it needs kept between steps through
``cache_need()``:

* ``KVCacheNeed``: paged keys and values (heads, head size, window; 0 = all keys);
* ``StateNeed``: a fixed-size tensor per live request (a slot);
* ``None``: nothing.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable

import torch

from ..weights.loader import TensorWant


@dataclass(frozen=True)
class KVCacheNeed:
    num_kv_heads: int
    head_dim: int
    window: int = 0  # 0: every earlier key stays needed


@dataclass(frozen=True)
class StateNeed:
    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class KVBinding:
    """What a mixer with paged keys/values is given: its cache group and this layer's pages."""

    group: int
    k_cache: torch.Tensor  # [pages, kv_heads, block_size, head_dim]
    v_cache: torch.Tensor  # [pages, kv_heads, head_dim, block_size]
    block_size: int


@dataclass
class StateBinding:
    """What a mixer with per-request state is given: one row per slot (the last row is a spare)."""

    state: torch.Tensor  # [slots + 1, *shape]


class Part:
    # Whether the part's ``forward`` may run inside a graph capture of a decode step (every item one token)
    # and be replayed with other indices: it reads positions, state slots and block tables from the batch's
    # device tensors only (never from ``batch.starts`` / ``qlens`` / ``slots_host``, which a replay does not
    # update), does not wait for the device and allocates nothing but torch tensors. Parts defined outside
    # the package say so themselves; a model with a part that does not is stepped without graphs.
    graph_safe = False

    def __init__(self, spec: Any, dtype: torch.dtype, device: torch.device):
        self.spec, self.dtype, self.device = spec, dtype, device

    def weight_wants(self, prefix: str) -> dict[str, TensorWant]:
        return {}

    def load(self, tensors: dict[str, torch.Tensor], prefix: str) -> None:
        pass


class Norm(Part):
    def as_fused(self) -> tuple[torch.Tensor, float] | None:
        """``(weight float32 [dim], eps)`` when the norm is ``x * rsqrt(mean(x^2) + eps) * weight``: the block
        then lets the residual add and the norm ride on a neighbouring kernel. None for any other
        norm: the block adds the residual with a kernel of its own and calls the part."""
        return None

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """The norm of the float32 residual stream ``[T, dim]``, in the compute dtype."""
        raise NotImplementedError


class PositionEncoding(Part):
    def tables(self, num_positions: int = 1) -> Any:
        """What the mixer's kernels read for positions ``0 .. num_positions - 1``. For encodings that
        rotate pairs ``(j, j + r/2)`` of the first ``r`` elements of each head: a contiguous float32
        tensor ``[P >= num_positions, 2, r/2]`` of cosines and sines on the part's device. It is not
        allocated anew inside a graph capture: keep and hand back a table that is large enough."""
        raise NotImplementedError


class Mixer(Part):
    def cache_need(self) -> KVCacheNeed | StateNeed | None:
        return None

    def cache_source(self) -> int | None:
        """Index of another layer whose cache this mixer reads instead of owning one."""
        return None

    def forward(self, h: torch.Tensor, batch: Any, cache: Any = None) -> torch.Tensor:
        """``h`` is the normed input [T, H] (or a lazy one that a part may take as the prologue of its
        first product); the result [T, H] is the delta that the block adds to the residual stream. It
        may be any object that the add-and-norm kernel takes as a delta: a tensor in the compute dtype,
        or partial sums that kernel adds up (see ``ops.kernels.linear(..., as_delta=True)``)."""
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, h: torch.Tensor, batch: Any) -> torch.Tensor:
        """As :meth:`Mixer.forward`, without a cache."""
        raise NotImplementedError


class Registry:
    """Kinds of one sort of part, by name. A spec names its kind in the attribute ``key`` (``kind`` for parts,
    ``arrangement`` for the block that puts them together)."""

    def __init__(self, what: str, key: str = "kind"):
        self.what, self.key = what, key
        self._by_kind: dict[str, Callable[..., Part]] = {}

    def register(self, kind: str, factory: Callable[..., Part]) -> None:
        self._by_kind[kind] = factory

    def build(self, spec: Any, dtype: torch.dtype, device: torch.device) -> Part:
        kind = getattr(spec, self.key, None)
        if kind not in self._by_kind:
            raise ValueError(f"no {self.what} registered for {self.key} {kind!r}; known: {sorted(self._by_kind)}")
        return self._by_kind[kind](spec, dtype, device)

    def kinds(self) -> list[str]:
        return sorted(self._by_kind)


MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
NORMS = Registry("norm")
POSITION_ENCODINGS = Registry("position encoding")
BLOCK_ARRANGEMENTS = Registry("block arrangement", key="arrangement")
