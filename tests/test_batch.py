"""Packing of a step's batch on the host, and the host-side checks that guard the kernels' indices."""

from __future__ import annotations

import numpy as np
import pytest

from mini_engine_amd.cache import GroupSpec
from mini_engine_amd.engine.batch import StepItem, pack_host, section_offsets, validate_items
from mini_engine_amd.engine.runner import batch_buckets
from mini_engine_amd.engine.sequence import Sequence


def seq_with(tables, slot=-1):
    s = Sequence([1])
    s.block_tables = [list(t) for t in tables]
    s.state_slot = slot
    return s


def test_pack_layout_of_a_mixed_batch():
    a, b = seq_with([[5, 2]], slot=1), seq_with([[7]])
    items = [StepItem(a, [11, 12, 13], 4, [0, 2]), StepItem(b, [21], 0, [0])]
    arr, t, nb, r, widths = pack_host(items, 1, spare_block=9, spare_slot=3)
    sec = section_offsets(t, nb, r, widths)
    get = lambda name: arr[sec[name][0] : sec[name][0] + sec[name][1]].tolist()
    assert (t, nb, r, widths) == (4, 2, 3, [2])
    assert get("token_ids") == [11, 12, 13, 21] and get("positions") == [4, 5, 6, 0]
    assert get("token_item") == [0, 0, 0, 1] and get("want_rows") == [0, 2, 3]
    assert get("item_start") == [0, 3, 4] and get("item_ctx") == [7, 1] and get("state_slots") == [1, 3]
    assert get("table0") == [5, 2, 7, 9]  # short tables are padded with the spare page


def test_padding_items_write_to_the_spare_page():
    a = seq_with([[4]])
    arr, t, nb, r, widths = pack_host([StepItem(a, [8], 2, [0])], 1, widths=[3], pad_items=2, spare_block=6, spare_slot=5)
    sec = section_offsets(t, nb, r, widths)
    get = lambda name: arr[sec[name][0] : sec[name][0] + sec[name][1]].tolist()
    assert (t, nb, r) == (3, 3, 3)
    assert get("positions") == [2, 0, 0] and get("item_ctx") == [3, 1, 1] and get("want_rows") == [0, 1, 2]
    assert get("table0") == [4, 6, 6, 6, 6, 6, 6, 6, 6] and get("state_slots") == [5, 5, 5]


def test_validation_catches_what_would_make_a_kernel_fault():
    g = (GroupSpec(),)
    ok = StepItem(seq_with([[0, 1]]), [1, 2, 3], 2, [2])
    validate_items([ok], 10, 4, g)
    with pytest.raises(ValueError, match="vocabulary"):
        validate_items([StepItem(seq_with([[0]]), [10], 0, [])], 10, 4, g)
    with pytest.raises(ValueError, match="vocabulary"):
        validate_items([StepItem(seq_with([[0]]), [-1], 0, [])], 10, 4, g)
    with pytest.raises(ValueError, match="pages"):
        validate_items([StepItem(seq_with([[0]]), [1, 2, 3], 2, [])], 10, 4, g)
    with pytest.raises(ValueError, match="wanted place"):
        validate_items([StepItem(seq_with([[0]]), [1], 0, [1])], 10, 4, g)
    with pytest.raises(ValueError, match="at least one"):
        validate_items([], 10, 4, g)
    with pytest.raises(ValueError, match="given back"):
        validate_items([StepItem(seq_with([[-1, 3]]), [1], 4, [])], 10, 4, g)
    # in a window group only pages the window still covers have to be there
    validate_items([StepItem(seq_with([[-1, 3]]), [1], 6, [])], 10, 4, (GroupSpec(window=3),))
    with pytest.raises(ValueError, match="given back"):
        validate_items([StepItem(seq_with([[-1, 3]]), [1], 6, [])], 10, 4, (GroupSpec(window=4),))


def test_buckets_match_the_reference():  # cuda_graphs.py:28-30, tests/test_gpu.py:47
    assert batch_buckets(5) == [1, 2, 4, 5]
    assert batch_buckets(64) == [1, 2, 4, 8, 16, 32, 48, 64]
    assert batch_buckets(1) == [1]
