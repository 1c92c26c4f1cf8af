"""Paged cache bookkeeping: page pools per cache group, block tables, prefix hashes, LRU eviction,
and slots for fixed-size per-request state. Pure Python, no tensors.

Behaviour of one pool follows the reference's ``src/mini_engine/block_manager.py``:
token ``i`` lives in slot ``table[i // bs] * bs + i % bs`` (``:3-5``); a full computed block gets the
chained hash ``blake2b(parent ‖ u32le(token)...)`` (``:26-35``); a free page keeps its content and
hash and is only evicted when a fresh page is taken and nothing unhashed is left (``:144-152``);
pages are freed tail first (``:107-118``); allocation is all-or-nothing and a revived cached page
counts against the free capacity (``:83-105``); the last token of a prompt is never served from the
cache (``:62-79``).

Added here: several *groups* of layers, each with a pool of its own and a table of its own per
request. A group may be a window group: pages that lie wholly before
``num_computed_tokens - window + 1`` are given back after each step and their table entries become
-1. Prefix hits are only offered when every group keeps all keys and no layer has per-request
state; a hit has to be present in every group's pool.
"""

from __future__ import annotations

import hashlib
from collections import OrderedDict
from collections.abc import Sequence as Seq
from dataclasses import dataclass
from typing import TYPE_CHECKING

if TYPE_CHECKING:
    from ..engine.sequence import Sequence

ROOT_HASH = b""


def hash_block(parent: bytes, token_ids: Seq[int]) -> bytes:
    """Chained, process-independent block hash (reference ``block_manager.py:26-32``)."""
    h = hashlib.blake2b(parent, digest_size=16)
    for t in token_ids:
        h.update(int(t).to_bytes(4, "little", signed=False))
    return h.digest()


@dataclass(frozen=True)
class GroupSpec:
    """One cache group: ``window == 0`` keeps every key; ``window == w`` keeps the last ``w``."""

    window: int = 0
    num_blocks: int | None = None  # None: the manager's default


class PagePool:
    """Pages of one group: reference counts, hashes, and the ordered pool of free pages."""

    def __init__(self, num_blocks: int):
        self.num_blocks = num_blocks
        self.ref_counts = [0] * num_blocks
        self.block_hash: list[bytes | None] = [None] * num_blocks
        self.hash_to_block: dict[bytes, int] = {}
        # Pages with ref_count == 0 in eviction order (front = taken first). Unhashed pages are
        # kept at the front since they hold nothing reusable.
        self.free_pool: OrderedDict[int, None] = OrderedDict((i, None) for i in range(num_blocks))
        self.num_evictions = 0

    def take_fresh(self) -> int:
        block, _ = self.free_pool.popitem(last=False)
        h = self.block_hash[block]
        if h is not None:  # evict: its content is about to be overwritten
            del self.hash_to_block[h]
            self.block_hash[block] = None
            self.num_evictions += 1
        self.ref_counts[block] = 1
        return block

    def share(self, block: int) -> None:
        if self.ref_counts[block] == 0:
            del self.free_pool[block]
        self.ref_counts[block] += 1

    def release(self, block: int) -> None:
        self.ref_counts[block] -= 1
        assert self.ref_counts[block] >= 0, "double free"
        if self.ref_counts[block] == 0:
            self.free_pool[block] = None
            if self.block_hash[block] is None:
                self.free_pool.move_to_end(block, last=False)

    def reset_hashes(self) -> None:
        for h, b in self.hash_to_block.items():
            assert self.block_hash[b] == h
            self.block_hash[b] = None
        self.hash_to_block.clear()


class StateSlots:
    """Indices of fixed-size per-request state: taken at admission, given back at finish or preemption."""

    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self.free: list[int] = list(range(num_slots - 1, -1, -1))
        self.in_use: set[int] = set()

    def take(self) -> int | None:
        if not self.free:
            return None
        s = self.free.pop()
        self.in_use.add(s)
        return s

    def give_back(self, slot: int) -> None:
        assert slot in self.in_use, "state slot freed twice"
        self.in_use.remove(slot)
        self.free.append(slot)


class BlockManager:
    def __init__(
        self,
        num_blocks: int,
        block_size: int,
        enable_prefix_caching: bool = True,
        groups: Seq[GroupSpec] = (GroupSpec(),),
        num_state_slots: int = 0,
        has_state: bool = False,
    ):
        if num_blocks < 1 or block_size < 1:
            raise ValueError("num_blocks and block_size must be positive")
        if not groups:
            raise ValueError("at least one cache group is needed")
        self.num_blocks = num_blocks
        self.block_size = block_size
        self.groups = tuple(groups)
        self.pools = [PagePool(g.num_blocks or num_blocks) for g in self.groups]
        self.slots = StateSlots(num_state_slots) if num_state_slots > 0 else None
        self.has_state = has_state
        shareable = all(g.window == 0 for g in self.groups) and not has_state
        self.enable_prefix_caching = bool(enable_prefix_caching) and shareable

    # --------------------------------------------- the first group under the reference's names
    @property
    def ref_counts(self) -> list[int]:
        return self.pools[0].ref_counts

    @property
    def block_hash(self) -> list[bytes | None]:
        return self.pools[0].block_hash

    @property
    def hash_to_block(self) -> dict[bytes, int]:
        return self.pools[0].hash_to_block

    @property
    def free_pool(self) -> "OrderedDict[int, None]":
        return self.pools[0].free_pool

    @property
    def num_evictions(self) -> int:
        return sum(p.num_evictions for p in self.pools)

    # ---------------------------------------------------------------------------------- queries
    @property
    def num_free_blocks(self) -> int:
        return min(len(p.free_pool) for p in self.pools)

    def blocks_needed(self, num_tokens: int) -> int:
        return -(-num_tokens // self.block_size)

    def fits(self, num_tokens: int) -> bool:
        """Whether a request of this many tokens could ever hold its pages at once."""
        need = self.blocks_needed(num_tokens)
        for g, p in zip(self.groups, self.pools):
            if g.window == 0 and need > p.num_blocks:
                return False
        return True

    def match_prefix(self, token_ids: Seq[int]) -> list[list[int]] | list[int]:
        """Longest run of cached full blocks that prefix ``token_ids``, present in every group.

        Only the first ``len - 1`` tokens are eligible: at least one token must be computed to get
        logits for the next one. Returns page ids of the first group when there is one group (the
        reference's form), else one list per group.
        """
        hits: list[list[int]] = [[] for _ in self.pools]
        if self.enable_prefix_caching:
            parent = ROOT_HASH
            bs = self.block_size
            for i in range((len(token_ids) - 1) // bs):
                parent = hash_block(parent, token_ids[i * bs : (i + 1) * bs])
                blocks = [p.hash_to_block.get(parent) for p in self.pools]
                if any(b is None for b in blocks):
                    break
                for h, b in zip(hits, blocks):
                    h.append(b)
        return hits[0] if len(self.pools) == 1 else hits

    # -------------------------------------------------------------------------------- mutations
    def _per_group(self, cached) -> list[list[int]]:
        if not cached:
            return [[] for _ in self.pools]
        if len(self.pools) == 1 and (not cached or isinstance(cached[0], int)):
            return [list(cached)]
        return [list(c) for c in cached]

    def try_allocate(self, seq: "Sequence", num_tokens: int, cached_blocks=()) -> bool:
        """Grow every table of ``seq`` to hold ``num_tokens`` tokens, and give it a state slot if it
        has none. All-or-nothing: returns False and changes nothing if any group lacks space.

        ``cached_blocks`` (from :meth:`match_prefix`, only for a sequence with empty tables) are
        shared rather than allocated.
        """
        while len(seq.block_tables) < len(self.pools):
            seq.block_tables.append([])
        need = self.blocks_needed(num_tokens)
        if not cached_blocks and (self.slots is None or seq.state_slot >= 0):
            for table in seq.block_tables:
                if len(table) < need:
                    break
            else:
                return True  # the usual decode step: the last page still has room
        cached = self._per_group(cached_blocks)
        if any(cached) and any(seq.block_tables):
            raise ValueError("cached blocks can only seed an empty block table")
        plans = []
        for pool, table, hit in zip(self.pools, seq.block_tables, cached):
            num_new = need - len(table) - len(hit)
            # Reviving a cached page that sits in the free pool consumes free capacity too.
            num_revived = sum(1 for b in hit if pool.ref_counts[b] == 0)
            if max(num_new, 0) + num_revived > len(pool.free_pool):
                return False
            plans.append(num_new)
        if self.slots is not None and seq.state_slot < 0 and not self.slots.free:
            return False

        for pool, table, hit, num_new in zip(self.pools, seq.block_tables, cached, plans):
            for b in hit:
                pool.share(b)
                table.append(b)
            for _ in range(num_new):
                table.append(pool.take_fresh())
        if self.slots is not None and seq.state_slot < 0:
            seq.state_slot = self.slots.take()
        return True

    def free(self, seq: "Sequence") -> None:
        """Drop the sequence's references and its state slot. Pages are freed in reverse so that,
        among pages freed together, the tail of a sequence is evicted before its head."""
        for pool, table in zip(self.pools, seq.block_tables):
            for b in reversed(table):
                if b >= 0:
                    pool.release(b)
            table.clear()
        seq.table_epoch += 1
        seq.block_hashes.clear()
        if self.slots is not None and seq.state_slot >= 0:
            self.slots.give_back(seq.state_slot)
        seq.state_slot = -1

    def release_passed(self, seq: "Sequence") -> int:
        """Give back the pages of window groups that no later query of ``seq`` can see: a query at
        position ``p >= num_computed_tokens`` sees keys ``>= p - window + 1``. Returns how many."""
        freed = 0
        for g, pool, table in zip(self.groups, self.pools, seq.block_tables):
            if g.window <= 0:
                continue
            first_needed = seq.num_computed_tokens - g.window + 1
            for i in range(min(len(table), max(first_needed, 0) // self.block_size)):
                if table[i] >= 0:
                    pool.release(table[i])
                    table[i] = -1
                    seq.table_epoch += 1
                    freed += 1
        return freed

    def register_computed_blocks(self, seq: "Sequence") -> None:
        """Hash every block of ``seq`` that has become full and computed since the last call."""
        if not self.enable_prefix_caching:
            return
        bs = self.block_size
        for i in range(len(seq.block_hashes), seq.num_computed_tokens // bs):
            parent = seq.block_hashes[-1] if seq.block_hashes else ROOT_HASH
            h = hash_block(parent, seq.token_ids[i * bs : (i + 1) * bs])
            seq.block_hashes.append(h)
            for pool, table in zip(self.pools, seq.block_tables):
                block = table[i]
                # If another page already holds this content (two identical prompts admitted in
                # the same step), keep the existing entry; ours stays an unhashed private copy.
                if pool.block_hash[block] is None and h not in pool.hash_to_block:
                    pool.block_hash[block] = h
                    pool.hash_to_block[h] = block

    def reset_prefix_cache(self) -> None:
        for pool in self.pools:
            pool.reset_hashes()
