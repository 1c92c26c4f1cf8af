"""Packing of a step's batch by the native host core, and its checks that guard the kernels' indices."""

from __future__ import annotations

import numpy as np
import pytest

from mini_engine_amd.engine.core import HostCore, step_layout
from mini_engine_amd.engine.runner import batch_buckets
from mini_engine_amd.engine.sequence import SamplingParams, Sequence
from mini_engine_amd.sampling.sampler import draw_key
from raw_batch import RawItem, pack_raw, raw_layout

BS = 4


def held(core: HostCore, tokens: list[int], computed: int = 0, params=None) -> Sequence:
    """A request of ``core`` with pages for all its tokens (a fresh pool hands out pages 0, 1, 2, ...)."""
    seq = Sequence(tokens, params, core=core)
    assert core.grow(seq._handle, len(tokens))
    seq.num_computed_tokens = computed
    return seq


def section(arr, lay, name, n):
    return arr[lay[name]:lay[name] + n].tolist()


def test_layout_is_the_documented_order_of_sections():
    lay = step_layout(5, 2, 3, [4, 2])
    assert lay == raw_layout(5, 2, 3, [4, 2])
    assert lay["sample_keys"] % 2 == 0 and lay["total"] == lay["tables"][1] + 2 * 2


def test_pack_layout_of_a_mixed_batch():
    core = HostCore(BS, [(0, 16)], num_state_slots=4, has_state=True, seed=11)
    a = held(core, list(range(30, 37)), computed=4, params=SamplingParams(temperature=0.5))  # pages 0, 1; slot 0
    b = held(core, [21])  # page 2; slot 1
    core.step_add(a._handle, 4, 3, [0, 2])
    core.step_add(b._handle, 0, 1, [0])
    lay = core.step_layout()
    arr = np.full(lay["total"], -7, dtype=np.int32)
    core.step_pack(arr, None, 0, spare_page=9, spare_slot=3)
    assert (lay["tokens"], lay["items"], lay["rows"], lay["widths"]) == (4, 2, 3, [2])
    assert section(arr, lay, "token_ids", 4) == [34, 35, 36, 21] and section(arr, lay, "positions", 4) == [4, 5, 6, 0]
    assert section(arr, lay, "token_item", 4) == [0, 0, 0, 1] and section(arr, lay, "want_rows", 3) == [0, 2, 3]
    assert section(arr, lay, "item_start", 3) == [0, 3, 4] and section(arr, lay, "item_ctx", 2) == [7, 1]
    assert section(arr, lay, "state_slots", 2) == [0, 1] and section(arr, lay, "live_items", 1) == [2]
    assert arr[lay["tables"][0]:lay["tables"][0] + 4].tolist() == [0, 1, 2, 9]  # short tables end in the spare page
    # the independent packer of the tests agrees on everything but the sampling inputs
    raw, raw_lay = pack_raw([RawItem([[0, 1]], [34, 35, 36], 4, [0, 2], 0), RawItem([[2]], [21], 0, [0], 1)], 1,
                            spare_block=9, spare_slot=3)
    assert raw_lay == lay
    keep = np.ones(lay["total"], dtype=bool)
    keep[lay["temperatures"]:lay["sample_keys"] + 2 * lay["rows"]] = False
    assert np.array_equal(arr[keep], raw[keep])
    # sampling inputs: only a wanted place that is its request's last token is drawn from
    temps = arr[lay["temperatures"]:lay["temperatures"] + 3].view(np.float32).tolist()
    keys = arr[lay["sample_keys"]:lay["sample_keys"] + 6].view(np.int64).tolist()
    assert temps == [0.0, 0.5, 0.0]
    assert keys == [0, draw_key(11, 0, 0), draw_key(11, 1, 0)]  # (seed, number of the request, index of the output)


def test_padding_items_write_to_the_spare_page():
    core = HostCore(BS, [(0, 16)])
    a = held(core, [5, 6, 8], computed=2)
    core.step_add(a._handle, 2, 1, [0])
    lay = core.step_layout([3], pad_items=2)
    arr = np.zeros(lay["total"], dtype=np.int32)
    core.step_pack(arr, [3], 2, spare_page=6, spare_slot=5)
    assert (lay["tokens"], lay["items"], lay["rows"]) == (3, 3, 3)
    assert section(arr, lay, "positions", 3) == [2, 0, 0] and section(arr, lay, "item_ctx", 3) == [3, 1, 1]
    assert section(arr, lay, "want_rows", 3) == [0, 1, 2] and section(arr, lay, "state_slots", 3) == [5, 5, 5]
    assert arr[lay["tables"][0]:lay["tables"][0] + 9].tolist() == [0, 6, 6, 6, 6, 6, 6, 6, 6]
    only_padding = np.zeros(step_layout(2, 2, 2, [3])["total"], dtype=np.int32)
    core.pack_padding(only_padding, [3], 2, 6, 5)
    raw, _ = pack_raw([], 1, widths=[3], pad_items=2, spare_block=6, spare_slot=5)
    assert np.array_equal(only_padding, raw)
    assert core.step_summary()[1] == 1  # the step itself is untouched by packing padding beside it


def test_checks_catch_what_would_make_a_kernel_fault():
    def check(tokens, start, count, want, pages_for=None, vocab=10, window=0, computed=None, passed=False):
        core = HostCore(BS, [(window, 32)], max_model_len=64)
        seq = Sequence(tokens, core=core)
        assert core.grow(seq._handle, len(tokens) if pages_for is None else pages_for)
        seq.num_computed_tokens = start if computed is None else computed
        if passed:
            core.drop_passed(seq._handle)
        core.step_add(seq._handle, start, count, want)
        core.step_check(vocab)

    check([1, 2, 3, 4, 5], 2, 3, [2])
    with pytest.raises(ValueError, match="vocabulary"):
        check([10], 0, 1, [])
    with pytest.raises(ValueError, match="vocabulary"):
        check([-1], 0, 1, [])
    with pytest.raises(ValueError, match="pages"):
        check([1, 2, 3, 4, 5], 2, 3, [], pages_for=4)
    with pytest.raises(ValueError, match="wanted place"):
        check([1], 0, 1, [1])
    with pytest.raises(ValueError, match="beyond its request"):
        check([1, 2], 1, 2, [])
    with pytest.raises(ValueError, match="beyond the limit"):
        check([1] * 80, 0, 80, [])
    with pytest.raises(ValueError, match="at least one"):
        HostCore(BS, [(0, 4)]).step_check(10)
    # an item that starts beyond what is computed would leave positions that nothing ever wrote under the mask
    with pytest.raises(ValueError, match="gap"):
        check([1, 2, 3, 4, 5], 2, 3, [2], computed=1)
    check([1, 2, 3, 4, 5], 2, 3, [2], computed=2)

    # in a window group only pages the window still covers have to be there: with 6 tokens computed and a
    # window of 3 the first page is given back; a step at position 6 needs keys from 4 on
    check([1] * 7, 6, 1, [], window=3, computed=6, passed=True)
    with pytest.raises(ValueError, match="given back"):  # position 4 sees keys from 2 on, which are gone
        check([1] * 7, 4, 1, [], window=3, computed=6, passed=True)


def test_a_request_may_appear_once_in_a_step():
    core = HostCore(BS, [(0, 16)])
    a, b = held(core, [1, 2, 3, 4]), held(core, [5, 6])
    core.step_add(a._handle, 0, 2, [])
    core.step_add(b._handle, 0, 2, [1])
    core.step_check(10)
    core.step_add(a._handle, 0, 2, [1])
    with pytest.raises(ValueError, match="twice"):
        core.step_check(10)
    core.step_clear()
    core.step_add(a._handle, 0, 4, [3])  # the check before left nothing behind
    core.step_check(10)


def test_refill_extends_rows_and_rewrites_what_changed():
    core = HostCore(BS, [(0, 32)], seed=3)
    a, b = held(core, [1] * 5, computed=4), held(core, [2] * 9, computed=8)
    widths, lay = [4], step_layout(2, 2, 2, [4])
    buf = np.zeros(lay["total"], dtype=np.int32)
    core.pack_padding(buf, widths, 2, 31, 0)

    def replay(seqs):
        core.step_clear()
        for s in seqs:
            core.step_add(s._handle, s.num_computed_tokens, 1, [0])
        core.step_refill(2, buf, widths, 31, 0)
        return buf[lay["tables"][0]:lay["tables"][0] + 8].reshape(2, 4).tolist()

    assert replay([a, b]) == [[0, 1, 31, 31], [2, 3, 4, 31]]
    assert section(buf, lay, "token_ids", 2) == [1, 2] and section(buf, lay, "item_ctx", 2) == [5, 9]
    buf[lay["tables"][0]] = 77  # the row of a is not rewritten while it only gains pages ...
    a.extend([1] * 4)
    assert core.grow(a._handle, 9)
    a.num_computed_tokens = 8
    assert replay([a, b])[0] == [77, 1, 5, 31]
    core.drop(a._handle)  # ... and written whole once its table was cleared
    assert core.grow(a._handle, 9)
    assert replay([a, b])[0] == a.block_table + [31]
    assert replay([b]) == [[2, 3, 4, 31], [31, 31, 31, 31]] and section(buf, lay, "live_items", 1) == [1]


def test_a_refill_that_throws_leaves_no_half_written_row_behind():
    # two groups: one keeps every key, the other a window of 3, whose passed pages are given back
    core = HostCore(BS, [(0, 32), (3, 32)], seed=3)
    a, b = held(core, [1] * 5, computed=4), held(core, [2] * 13, computed=12)
    core.drop_passed(b._handle)
    widths, lay = [4, 4], step_layout(2, 2, 2, [4, 4])
    buf = np.zeros(lay["total"], dtype=np.int32)
    core.pack_padding(buf, widths, 2, 31, 0)
    table = lambda g: buf[lay["tables"][g]:lay["tables"][g] + 8].reshape(2, 4).tolist()
    core.step_add(a._handle, 4, 1, [0])
    core.step_add(b._handle, 12, 1, [0])
    core.step_refill(2, buf, widths, 31, 0)  # a good refill first: the row remembers whose table it holds
    core.step_clear()
    core.step_add(a._handle, 4, 1, [0])
    core.step_add(b._handle, 6, 1, [0])  # position 6 would see keys from 4 on: the window group's page is gone
    with pytest.raises(ValueError, match="given back"):
        core.step_refill(2, buf, widths, 31, 0)
    assert table(0)[1] != [31] * 4  # the first group's row holds pages of b
    core.step_clear()
    core.step_add(a._handle, 4, 1, [0])  # the second row is padding now: it keeps nothing of the failed refill
    core.step_refill(2, buf, widths, 31, 0)
    assert table(0)[1] == [31] * 4 and table(1)[1] == [31] * 4
    assert table(0)[0] == a.block_tables[0] + [31, 31]


def test_buckets_match_the_reference():  # cuda_graphs.py:28-30, tests/test_gpu.py:47
    assert batch_buckets(5) == [1, 2, 4, 5]
    assert batch_buckets(64) == [1, 2, 4, 8, 16, 32, 48, 64]
    assert batch_buckets(1) == [1]
