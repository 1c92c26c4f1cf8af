"""Device storage behind the page tables: for every run of a layer (a position in the model's
order) that owns a cache, one tensor of key pages and one of value pages, or one tensor of state
rows for a mixer with per-request state.

Runs whose mixers state the same need (heads, head size, window) form one group and share one
block table per request. A page id indexes every run of its group at once. Each group has one page
more than the manager hands out: rows that pad a replayed graph write there.

Layout of a layer's pages: keys ``[pages, kv_heads, block_size, head_dim]`` and values transposed,
``[pages, kv_heads, head_dim, block_size]``, so that the matrix cores read both along the
contiguous direction (keys along head_dim for q.k, values along the keys for p.v).
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ..parts.base import KVBinding, KVCacheNeed, StateBinding, StateNeed
from .block_manager import GroupSpec


@dataclass
class CacheLayout:
    groups: list[GroupSpec]
    group_needs: list[KVCacheNeed]
    layer_group: dict[int, int]  # run (position in the order) -> group index, for runs that own pages
    state_layers: dict[int, StateNeed]  # run -> its state need

    @property
    def has_state(self) -> bool:
        return bool(self.state_layers)


def plan_layout(decoder) -> CacheLayout:
    """Group the runs of a decoder by what their mixers need."""
    needs: list[KVCacheNeed] = []
    layer_group: dict[int, int] = {}
    state_layers: dict[int, StateNeed] = {}
    for i, layer in enumerate(decoder.plan.order):
        if decoder.cache_owner[i] != i:
            continue
        need = decoder.blocks[layer].mixer.cache_need()
        if isinstance(need, KVCacheNeed):
            if need not in needs:
                needs.append(need)
            layer_group[i] = needs.index(need)
        elif isinstance(need, StateNeed):
            state_layers[i] = need
        elif need is not None:
            raise TypeError(f"layer {i}: unknown cache need {need!r}")
    groups = [GroupSpec(window=n.window) for n in needs] or [GroupSpec()]
    return CacheLayout(groups, needs, layer_group, state_layers)


class CacheStorage:
    def __init__(self, decoder, layout: CacheLayout, num_blocks: int, block_size: int, num_state_slots: int,
                 dtype: torch.dtype, device: torch.device):
        self.layout, self.block_size, self.dtype = layout, block_size, dtype
        self.spare_block = num_blocks  # never handed out by the manager
        self.spare_slot = num_state_slots
        self.kv: dict[int, tuple[torch.Tensor, torch.Tensor]] = {}
        self.state: dict[int, torch.Tensor] = {}
        for i, g in layout.layer_group.items():
            need = layout.group_needs[g]
            k = torch.zeros((num_blocks + 1, need.num_kv_heads, block_size, need.head_dim), dtype=dtype, device=device)
            v = torch.zeros((num_blocks + 1, need.num_kv_heads, need.head_dim, block_size), dtype=dtype, device=device)
            self.kv[i] = (k, v)
        for i, need in layout.state_layers.items():
            self.state[i] = torch.zeros((num_state_slots + 1, *need.shape), dtype=need.dtype, device=device)
        for r, owner in enumerate(decoder.cache_owner):
            if owner in self.kv:
                k, v = self.kv[owner]
                decoder.bindings[r] = KVBinding(layout.layer_group[owner], k, v, block_size)
            elif r in self.state:
                decoder.bindings[r] = StateBinding(self.state[r])

    def kv_bytes_per_token(self) -> int:
        """Bytes of keys and values one token occupies over all runs that own pages."""
        elem = torch.empty((), dtype=self.dtype).element_size()
        return sum(2 * self.layout.group_needs[g].num_kv_heads * self.layout.group_needs[g].head_dim * elem
                   for g in self.layout.layer_group.values())

    def zero_state(self, slots: list[int]) -> None:
        if self.state and slots:
            idx = torch.tensor(slots, dtype=torch.long, device=next(iter(self.state.values())).device)
            for s in self.state.values():
                s.index_fill_(0, idx, 0)
