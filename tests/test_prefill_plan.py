"""The host-side work list of the prefill attention kernel: every tile of query tokens meets exactly
the keys it may see, in one piece or in ranges that tile its keys without gap or overlap."""

import random

import numpy as np

from mini_engine_amd.ops.kernels import prefill_work_list, wide_blocks_pay


def check_plan(starts, qlens, tpb, window, nkv, slots):
    work, first, token_chunks, max_chunks = prefill_work_list(starts, qlens, tpb, window, nkv, slots,
                                                              partial_row_bytes=4096)
    offsets = np.concatenate([[0], np.cumsum(qlens)])
    assert token_chunks.shape == (offsets[-1],)
    # bundles: every entry belongs to exactly one, each ends with its only `last` mark
    assert first[0] == 0 and (np.diff(first) > 0).all() and first[-1] < work.shape[0]
    ends = set((first[1:] - 1).tolist()) | {work.shape[0] - 1}
    assert {i for i, e in enumerate(work.tolist()) if e[7] == 1} == ends
    assert len(first) <= max(slots // nkv, 1) or len(first) == work.shape[0]  # packed, or one tile per bundle
    by_tile = {}
    for item, tb, count, p_first, k0, k_last, chunk, last in work.tolist():
        assert last in (0, 1) and k0 % 64 == 0 and k0 <= k_last
        by_tile.setdefault((item, tb, count, p_first), []).append((chunk, k0, k_last))
    # every tile of every item is there, with the right tokens and positions
    want_tiles = set()
    for i, (s0, n) in enumerate(zip(starts, qlens)):
        for t in range(-(-n // tpb)):
            want_tiles.add((i, int(offsets[i]) + t * tpb, min(tpb, n - t * tpb), s0 + t * tpb))
    assert set(by_tile) == want_tiles
    for (item, tb, count, p_first), pieces in by_tile.items():
        p_last = p_first + count - 1
        lo = max(p_first - window + 1, 0) if window > 0 else 0
        pieces.sort(key=lambda p: p[1])
        if len(pieces) == 1:
            assert pieces[0][0] == -1
            assert (token_chunks[tb:tb + count] == 1).all()
        else:
            assert [p[0] for p in pieces] == list(range(len(pieces))) and len(pieces) <= max_chunks
            assert (token_chunks[tb:tb + count] == len(pieces)).all()
        assert pieces[0][1] == (lo // 64) * 64 and pieces[-1][2] == p_last
        for (_, _, last), (_, nxt, _) in zip(pieces, pieces[1:]):
            assert nxt == last + 1  # no gap, no overlap
    return work, first, max_chunks


def bundle_loads(work, first):
    bounds = first.tolist() + [work.shape[0]]
    return [sum((e[5] - e[4]) // 64 + 1 for e in work[a:b].tolist()) for a, b in zip(bounds, bounds[1:])]


def test_many_tiles_are_left_whole_longest_first():
    work, first, max_chunks = check_plan([0], [4096], 64, 0, 8, 256)
    assert max_chunks == 1 and work.shape[0] == 64 and len(first) == 64
    loads = bundle_loads(work, first)
    assert loads == sorted(loads, reverse=True)


def test_causal_prompt_with_one_tile_per_compute_unit_is_evened_out():
    work, first, max_chunks = check_plan([0], [2048], 64, 0, 8, 256)
    loads = bundle_loads(work, first)
    assert len(first) == 32 and max_chunks == 2
    assert max(loads) <= 20 < 32  # whole tiles would give 32 key tiles to the last block


def test_short_prompts_are_not_cut():
    """Cutting costs a step the partial results and the kernel that adds them up: a prompt of a few hundred tokens,
    whose longest tile walks a few key tiles, is left whole; from about a thousand tokens on it is cut."""
    for tokens in (65, 128, 256, 512):
        work, first, max_chunks = check_plan([0], [tokens], 64, 0, 8, 256)
        assert max_chunks == 1 and work.shape[0] == -(-tokens // 64)
    for tokens in (1024, 1536):
        assert check_plan([0], [tokens], 64, 0, 8, 256)[2] > 1


def test_short_portion_over_long_context_is_cut_to_fill_the_chip():
    work, first, max_chunks = check_plan([30000, 5], [64, 3], 64, 0, 8, 256)
    assert max_chunks > 8 and len(first) == 32
    assert max(bundle_loads(work, first)) <= 20


def test_random_steps():
    rng = random.Random(0)
    for _ in range(200):
        n_items = rng.randint(1, 5)
        starts = [rng.choice([0, 0, 3, 64, 1000, 5000]) for _ in range(n_items)]
        qlens = [rng.choice([1, 2, 7, 64, 65, 200, 700]) for _ in range(n_items)]
        check_plan(starts, qlens, rng.choice([8, 32, 64, 128]), rng.choice([0, 0, 37, 500]), rng.choice([1, 2, 8]),
                   rng.choice([16, 256]))


def test_wide_blocks_are_taken_for_full_steps_and_long_contexts_only():
    """128 tokens per wide block (a kv group of two heads), 8 kv heads, 256 compute units."""
    pay = lambda starts, qlens, window=0: wide_blocks_pay(starts, qlens, 128, window, 8, 256)
    assert not pay([0], [2048])            # 16 blocks per kv head: half the compute units
    assert pay([0], [4096])                # a whole block for every compute unit
    assert pay([0] * 32, [256] * 32)       # many short prompts fill the chip as well
    assert not pay([0] * 3, [1024] * 3)    # neither: few blocks, few keys
    assert pay([2048], [2048])             # few blocks, but a long walk over the keys for each
    assert pay([8192] * 2, [512] * 2)
    assert not pay([0] * 64, [64] * 64)    # wide blocks would be half empty
    assert not pay([8192] * 2, [512] * 2, window=256)  # a window takes the long walk away
