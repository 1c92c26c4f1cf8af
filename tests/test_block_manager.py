"""The cache manager (the native host core behind its Python view) without tensors. The first part
restates the vectors the reference's own tests hold (``tests/test_block_manager.py``, cited per
test); the second part covers what is added here: groups with windows, state slots, and random
orders of requests under which no page may be lost, held twice or freed twice."""

from __future__ import annotations

import random

import pytest

from mini_engine_amd.cache import ROOT_HASH, BlockManager, GroupSpec, hash_block
from mini_engine_amd.engine.sequence import Sequence

BS = 4


def computed(bm: BlockManager, tokens: list[int]) -> Sequence:
    """Admit a sequence through the prefix cache and mark its prompt computed."""
    seq = Sequence(tokens)
    cached = bm.match_prefix(seq.token_ids)
    assert bm.try_allocate(seq, len(seq), cached)
    seq.num_computed_tokens = len(seq)
    bm.register_computed_blocks(seq)
    return seq


def check_invariants(bm: BlockManager, live: list[Sequence]) -> None:
    """Reference test_block_manager.py:21-29, for every group, plus the state slots."""
    for g, pool in enumerate(bm.pools):
        refs = [0] * pool.num_blocks
        for s in live:
            for b in s.block_tables[g] if g < len(s.block_tables) else []:
                if b >= 0:
                    refs[b] += 1
        assert refs == pool.ref_counts, f"group {g}: reference counts drifted"
        assert set(pool.free_pool) == {b for b in range(pool.num_blocks) if refs[b] == 0}
        for h, b in pool.hash_to_block.items():
            assert pool.block_hash[b] == h
    if bm.slots is not None:
        held = [s.state_slot for s in live if s.state_slot >= 0]
        assert len(held) == len(set(held)), "a state slot is held twice"
        assert set(held) == bm.slots.in_use
        assert sorted(held + bm.slots.free) == list(range(bm.slots.num_slots)), "a state slot was lost"


# ------------------------------------------------------------------ the reference's own vectors
def test_hash_is_chained_and_deterministic():  # :32-35
    a = hash_block(ROOT_HASH, [1, 2, 3, 4])
    assert a == hash_block(ROOT_HASH, [1, 2, 3, 4])
    assert hash_block(a, [5, 6, 7, 8]) != hash_block(ROOT_HASH, [5, 6, 7, 8])
    assert len(a) == 16


def test_hash_is_blake2b_over_parent_then_u32le_tokens():
    import hashlib

    want = hashlib.blake2b(b"p" + (1).to_bytes(4, "little") + (258).to_bytes(4, "little"), digest_size=16).digest()
    assert hash_block(b"p", [1, 258]) == want


def test_allocate_and_free_roundtrip():  # :38-50
    bm = BlockManager(num_blocks=8, block_size=BS)
    seq = Sequence(list(range(10)))
    assert bm.try_allocate(seq, 10)
    assert len(seq.block_table) == 3 and bm.num_free_blocks == 5
    assert bm.try_allocate(seq, 12) and len(seq.block_table) == 3
    assert bm.try_allocate(seq, 13) and len(seq.block_table) == 4
    check_invariants(bm, [seq])
    bm.free(seq)
    assert seq.block_table == [] and bm.num_free_blocks == 8
    check_invariants(bm, [])


def test_allocation_is_all_or_nothing():  # :53-57
    bm = BlockManager(num_blocks=2, block_size=BS)
    seq = Sequence([1])
    assert not bm.try_allocate(seq, 9)
    assert seq.block_table == [] and bm.num_free_blocks == 2


def test_prefix_hit_shares_blocks_and_counts_refs():  # :60-71
    bm = BlockManager(num_blocks=16, block_size=BS)
    a = computed(bm, list(range(1, 11)))
    b = computed(bm, [*list(range(1, 9)), 99, 98, 97])
    assert b.block_table[:2] == a.block_table[:2] and b.block_table[2] != a.block_table[2]
    assert [bm.ref_counts[x] for x in a.block_table] == [2, 2, 1]
    check_invariants(bm, [a, b])
    bm.free(a)
    assert [bm.ref_counts[x] for x in b.block_table] == [1, 1, 1]
    check_invariants(bm, [b])


def test_full_prompt_hit_still_computes_last_token():  # :74-78
    bm = BlockManager(num_blocks=16, block_size=BS)
    computed(bm, list(range(8)))
    assert len(bm.match_prefix(list(range(8)))) == 1
    assert len(bm.match_prefix(list(range(9)))) == 2


def test_freed_blocks_stay_cached_until_evicted():  # :81-89
    bm = BlockManager(num_blocks=4, block_size=BS)
    a = computed(bm, list(range(9)))
    bm.free(a)
    assert len(bm.match_prefix(list(range(9)))) == 2
    b = computed(bm, list(range(9)))
    assert bm.ref_counts[b.block_table[0]] == 1 and bm.num_evictions == 0
    check_invariants(bm, [b])


def test_eviction_prefers_unhashed_then_lru():  # :92-106
    bm = BlockManager(num_blocks=6, block_size=BS)
    old = computed(bm, [1] * 5)
    new = computed(bm, [2] * 5)
    bm.free(old)
    bm.free(new)
    hog = Sequence([3])
    assert bm.try_allocate(hog, 4 * BS) and bm.num_evictions == 0
    assert len(bm.match_prefix([1] * 5)) == 1 and len(bm.match_prefix([2] * 5)) == 1
    assert bm.try_allocate(hog, 5 * BS) and bm.num_evictions == 1
    assert bm.match_prefix([1] * 5) == [] and len(bm.match_prefix([2] * 5)) == 1
    check_invariants(bm, [hog])


def test_reviving_cached_block_counts_against_capacity():  # :109-118
    bm = BlockManager(num_blocks=3, block_size=BS)
    a = computed(bm, list(range(9)))
    bm.free(a)
    seq = Sequence(list(range(9)) + [50] * 4)
    cached = bm.match_prefix(seq.token_ids)
    assert len(cached) == 2
    assert not bm.try_allocate(seq, len(seq), cached)
    assert seq.block_table == [] and bm.num_free_blocks == 3
    check_invariants(bm, [])


def test_duplicate_content_is_not_double_registered():  # :121-133
    bm = BlockManager(num_blocks=8, block_size=BS)
    a, b = Sequence([7] * 5), Sequence([7] * 5)
    for s in (a, b):
        assert bm.try_allocate(s, len(s))
    for s in (a, b):
        s.num_computed_tokens = len(s)
        bm.register_computed_blocks(s)
    assert a.num_block_hashes == b.num_block_hashes == 1
    assert bm.hash_to_block[hash_block(ROOT_HASH, [7] * BS)] == a.block_table[0]
    assert bm.block_hash[b.block_table[0]] is None
    bm.free(a)
    bm.free(b)
    check_invariants(bm, [])


def test_decode_tokens_get_hashed_as_blocks_fill():  # :136-144
    bm = BlockManager(num_blocks=8, block_size=BS)
    seq = computed(bm, [1, 2, 3])
    assert seq.num_block_hashes == 0
    seq.extend([4])
    seq.num_computed_tokens = 4
    bm.register_computed_blocks(seq)
    assert seq.num_block_hashes == 1
    assert bm.match_prefix([1, 2, 3, 4, 5]) == [seq.block_table[0]]


def test_prefix_caching_disabled_and_reset():  # :147-158
    bm = BlockManager(num_blocks=8, block_size=BS, enable_prefix_caching=False)
    computed(bm, list(range(9)))
    assert bm.match_prefix(list(range(9))) == [] and bm.hash_to_block == {}
    bm = BlockManager(num_blocks=8, block_size=BS)
    bm.free(computed(bm, list(range(9))))
    bm.reset_prefix_cache()
    assert bm.match_prefix(list(range(9))) == [] and all(h is None for h in bm.block_hash)


def test_double_free_is_detected():  # :161-169
    bm = BlockManager(num_blocks=4, block_size=BS)
    seq = Sequence([1])
    bm.try_allocate(seq, 1)
    (page,) = seq.block_table
    bm.free(seq)
    bm.free(seq)  # a request that holds nothing gives nothing back
    with pytest.raises(AssertionError, match="double free"):
        bm.core.release_page(0, page)  # a holder that does not exist cannot let go
    check_invariants(bm, [])


def test_cached_blocks_only_seed_an_empty_table():  # block_manager.py:90-91
    bm = BlockManager(num_blocks=8, block_size=BS)
    a = computed(bm, list(range(9)))
    with pytest.raises(ValueError):
        bm.try_allocate(a, 12, bm.match_prefix(list(range(9))))


# ------------------------------------------------------------- groups, windows and state slots
def test_groups_have_pools_and_tables_of_their_own():
    bm = BlockManager(num_blocks=6, block_size=BS, groups=(GroupSpec(), GroupSpec(window=6)))
    assert not bm.enable_prefix_caching  # a window group cannot serve prefix hits
    seq = Sequence(list(range(10)))
    assert bm.try_allocate(seq, 10)
    assert len(seq.block_tables) == 2 and len(seq.block_tables[0]) == len(seq.block_tables[1]) == 3
    assert bm.num_free_blocks == 3
    check_invariants(bm, [seq])
    bm.free(seq)
    check_invariants(bm, [])


def test_window_pages_are_given_back_once_passed_and_used_again():
    bm = BlockManager(num_blocks=3, block_size=BS, groups=(GroupSpec(window=5),))
    seq = Sequence([1] * 40)
    held_pages = set()
    for n in range(1, 41):  # token by token: 3 pages suffice for any length
        assert bm.try_allocate(seq, n), f"ran out at {n} tokens"
        seq.num_computed_tokens = n
        bm.release_passed(seq)
        table = seq.block_tables[0]
        first_needed = max(n - 5 + 1, 0)  # the next query at position n sees keys >= n - 4
        for i, page in enumerate(table):
            wholly_before = (i + 1) * BS <= first_needed
            assert (page == -1) == wholly_before, (n, i, table)
        held_pages.update(p for p in table if p >= 0)
        check_invariants(bm, [seq])
    assert held_pages <= {0, 1, 2} and len(seq.block_tables[0]) == 10  # ten table entries, pages used again
    bm.free(seq)
    check_invariants(bm, [])


def test_all_or_nothing_across_groups():
    bm = BlockManager(num_blocks=4, block_size=BS, groups=(GroupSpec(), GroupSpec(window=4, num_blocks=2)))
    seq = Sequence([1] * 12)
    assert not bm.try_allocate(seq, 12)  # group 1 has 2 pages only
    assert seq.block_tables[0] == [] and seq.block_tables[1] == []
    check_invariants(bm, [])


def test_state_slots_are_taken_and_given_back():
    bm = BlockManager(num_blocks=8, block_size=BS, num_state_slots=2, has_state=True)
    a, b, c = Sequence([1]), Sequence([2]), Sequence([3])
    assert bm.try_allocate(a, 1) and bm.try_allocate(b, 1)
    assert {a.state_slot, b.state_slot} == {0, 1}
    assert not bm.try_allocate(c, 1) and c.state_slot == -1 and c.block_table == []
    check_invariants(bm, [a, b])
    bm.free(a)
    assert a.state_slot == -1 and bm.try_allocate(c, 1) and c.state_slot in (0, 1)
    check_invariants(bm, [b, c])
    assert not bm.enable_prefix_caching  # state cannot be restored from shared pages


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("windowed", [False, True])
def test_random_orders_keep_every_page_accounted_for(seed, windowed):
    rng = random.Random(seed)
    groups = (GroupSpec(), GroupSpec(window=9)) if windowed else (GroupSpec(),)
    bm = BlockManager(num_blocks=24, block_size=BS, groups=groups, num_state_slots=5)
    live: list[Sequence] = []
    shared = [rng.randrange(50) for _ in range(12)]
    for _ in range(400):
        op = rng.random()
        if op < 0.35 and len(live) < 5:
            tokens = (shared[: rng.choice([0, 4, 8, 12])] + [rng.randrange(50) for _ in range(rng.randint(1, 14))])
            seq = Sequence(tokens)
            cached = bm.match_prefix(tokens)
            n_hit = len(cached) if not windowed else len(cached[0])
            first = rng.randint(1, len(tokens) - n_hit * BS)
            if bm.try_allocate(seq, n_hit * BS + first, cached):
                seq.num_computed_tokens = n_hit * BS + first
                live.append(seq)
                bm.register_computed_blocks(seq)
                bm.release_passed(seq)
            else:
                assert all(t == [] for t in seq.block_tables) and seq.state_slot == -1
        elif op < 0.8 and live:
            seq = rng.choice(live)
            if seq.num_computed_tokens == len(seq):
                seq.extend([rng.randrange(50)])
            n = rng.randint(1, len(seq) - seq.num_computed_tokens)
            before = [list(t) for t in seq.block_tables]
            if bm.try_allocate(seq, seq.num_computed_tokens + n):
                seq.num_computed_tokens += n
                bm.register_computed_blocks(seq)
                bm.release_passed(seq)
            else:
                assert [list(t) for t in seq.block_tables] == before
        elif live:
            seq = live.pop(rng.randrange(len(live)))
            bm.free(seq)
        check_invariants(bm, live)
    for seq in live:
        bm.free(seq)
    check_invariants(bm, [])
    assert all(len(p.free_pool) == p.num_blocks for p in bm.pools)


def test_nine_requests_live_at_once_without_state_slots():
    """A model without per-request state has no slots, so the number of live requests is bound by pages alone."""
    bm = BlockManager(num_blocks=1000, block_size=BS, num_state_slots=0)
    live = [Sequence([1, 2, 3]) for _ in range(12)]
    assert all(bm.try_allocate(s, 3) for s in live) and bm.num_free_blocks == 988
    check_invariants(bm, live)
    with_slots = BlockManager(num_blocks=1000, block_size=BS, num_state_slots=8, has_state=True)
    nine = [Sequence([1, 2, 3]) for _ in range(9)]
    got = [with_slots.try_allocate(s, 3) for s in nine]
    assert got == [True] * 8 + [False]  # the ninth lacks a slot, not a page
    del nine[0]  # a request nobody names any more gives back what it held
    assert with_slots.try_allocate(nine[-1], 3)


def test_a_window_group_refuses_what_its_pool_can_never_hold():
    """A step's portion needs the window and the portion at once in a window group's pool."""
    from mini_engine_amd.engine.core import HostCore

    core = HostCore(BS, [(8, 3)], max_num_batched_tokens=16)
    assert core.can_ever_hold(8)  # two pages
    assert not core.can_ever_hold(40)  # window 8 + portion 16 = 6 pages + 1 > 3
    roomy = HostCore(BS, [(8, 7)], max_num_batched_tokens=16)
    assert roomy.can_ever_hold(4000)
