"""The cache manager as Python sees it: pages in pools per cache group, a block table per request
and group, prefix digests with an eviction order, and slots for fixed-size per-request state.

All of it lives in the native host core (``csrc/host/pages.cpp``); :class:`BlockManager` is a view of
that core under the reference's method names (``src/mini_engine/block_manager.py:59-140``). What the
core does, in short: token ``i`` of a request lives in slot ``table[i // bs] * bs + i % bs``; a full
computed block carries the chained digest ``blake2b-128(parent, u32le(token)...)``; a page nobody holds
keeps its content and digest and waits in the free order, at the back when it has a digest and at
the front when it has none, and only loses them when it is taken for new content; a request's pages
are given back last page first; growing a table is all or nothing over every group and the state
slot, and a cached page that is taken out of the free order counts against the free pages; the last
token of a prompt is never served from the cache.

Beyond the reference: several *groups* of layers, each with a pool and a table of its own. A window
group gives pages back once no later query can see them (the table entry becomes -1). Prefix hits
are only offered when every group keeps all keys and no layer has per-request state, and a hit has
to be present in every group's pool.
"""

from __future__ import annotations

from collections.abc import Sequence as Seq
from dataclasses import dataclass

from ..engine.core import HostCore, chain_digest

ROOT_HASH = b""


def hash_block(parent: bytes, token_ids: Seq[int]) -> bytes:
    """Chained block digest, the same in every process (reference ``block_manager.py:26-32``)."""
    return chain_digest(parent, token_ids)


@dataclass(frozen=True)
class GroupSpec:
    """One cache group: ``window == 0`` keeps every key; ``window == w`` keeps the last ``w``."""

    window: int = 0
    num_blocks: int | None = None  # None: the manager's default


class PoolView:
    """One group's pages, read from the core on every access (for tests and diagnostics)."""

    def __init__(self, core: HostCore, group: int, num_blocks: int):
        self._core, self.group, self.num_blocks = core, group, num_blocks

    def _snapshot(self) -> dict:
        return self._core.pool(self.group, self.num_blocks)

    @property
    def ref_counts(self) -> list[int]:
        return self._snapshot()["holders"]

    @property
    def free_pool(self) -> list[int]:
        """Pages nobody holds, in the order they will be taken."""
        return self._snapshot()["free_order"]

    @property
    def block_hash(self) -> list[bytes | None]:
        return self._snapshot()["digests"]

    @property
    def hash_to_block(self) -> dict[bytes, int]:
        return {d: p for p, d in enumerate(self._snapshot()["digests"]) if d is not None}

    @property
    def num_evictions(self) -> int:
        return self._snapshot()["evictions"]


class SlotsView:
    def __init__(self, core: HostCore, num_slots: int):
        self._core, self.num_slots = core, num_slots

    @property
    def in_use(self) -> set[int]:
        return {i for i, taken in enumerate(self._core.slots_taken()) if taken}

    @property
    def free(self) -> list[int]:
        return [i for i, taken in enumerate(self._core.slots_taken()) if not taken]


class BlockManager:
    def __init__(self, num_blocks: int, block_size: int, enable_prefix_caching: bool = True,
                 groups: Seq[GroupSpec] = (GroupSpec(),), num_state_slots: int = 0, has_state: bool = False,
                 core: HostCore | None = None):
        if num_blocks < 1 or block_size < 1:
            raise ValueError("num_blocks and block_size must be positive")
        if not groups:
            raise ValueError("at least one cache group is needed")
        self.num_blocks, self.block_size, self.groups = num_blocks, block_size, tuple(groups)
        sizes = [g.num_blocks or num_blocks for g in self.groups]
        self.core = core or HostCore(block_size, [(g.window, n) for g, n in zip(self.groups, sizes)],
                                     enable_prefix_caching, num_state_slots, has_state)
        self.pools = [PoolView(self.core, g, n) for g, n in enumerate(sizes)]
        self.slots = SlotsView(self.core, num_state_slots) if num_state_slots > 0 else None
        self.has_state = has_state

    def new_sequence(self, token_ids, params=None):
        from ..engine.sequence import Sequence

        return Sequence(token_ids, params, core=self.core)

    # ---- queries
    @property
    def enable_prefix_caching(self) -> bool:
        return bool(self.core.pages_info()[1])

    @property
    def num_free_blocks(self) -> int:
        return int(self.core.pages_info()[2])

    @property
    def num_evictions(self) -> int:
        return int(self.core.pages_info()[3])

    # the first group under the reference's names
    @property
    def ref_counts(self) -> list[int]:
        return self.pools[0].ref_counts

    @property
    def free_pool(self) -> list[int]:
        return self.pools[0].free_pool

    @property
    def block_hash(self) -> list[bytes | None]:
        return self.pools[0].block_hash

    @property
    def hash_to_block(self) -> dict[bytes, int]:
        return self.pools[0].hash_to_block

    def blocks_needed(self, num_tokens: int) -> int:
        return -(-num_tokens // self.block_size)

    def fits(self, num_tokens: int) -> bool:
        """Whether a request of this many tokens could ever hold the pages a step of it needs."""
        return self.core.can_ever_hold(num_tokens)

    def match_prefix(self, token_ids: Seq[int]):
        """Pages of the longest run of cached full blocks that prefix ``token_ids`` and that every
        group still has: a list of page ids with one group (the reference's form), else one list
        per group."""
        hits = self.core.match(list(token_ids))
        return hits[0] if len(hits) == 1 else hits

    # ---- changes
    def _per_group(self, cached) -> list[list[int]] | None:
        if not cached:
            return None
        if len(self.pools) == 1 and isinstance(cached[0], int):
            return [list(cached)]
        return [list(c) for c in cached]

    def try_allocate(self, seq, num_tokens: int, cached_blocks=()) -> bool:
        """Grow every table of ``seq`` to hold ``num_tokens`` tokens and give it a state slot if it
        has none; False, with nothing changed, if any group lacks the space. ``cached_blocks`` (from
        :meth:`match_prefix`, only for a sequence with empty tables) are shared, not allocated."""
        seq.bind(self.core)
        return self.core.grow(seq._handle, num_tokens, self._per_group(cached_blocks))

    def free(self, seq) -> None:
        seq.bind(self.core)
        self.core.drop(seq._handle)

    def release_passed(self, seq) -> int:
        return self.core.drop_passed(seq.bind(self.core)._handle)

    def register_computed_blocks(self, seq) -> None:
        self.core.note_computed(seq.bind(self.core)._handle)

    def reset_prefix_cache(self) -> None:
        self.core.forget_digests()
