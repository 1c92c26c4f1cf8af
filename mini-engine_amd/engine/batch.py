"""One step's batch: host lists packed into a single int32 buffer, uploaded with one copy.

An item is ``(request, its next tokens, the position of the first of them, the places among them
whose logits are wanted)``. Items are packed one after another (reference:
``src/mini_engine/engine.py:200-226``); instead of a padded mask the kernels get, per token, its
absolute position and the index of its item, and per item and cache group a row of the block table.

Sections of the buffer, in order (T tokens, B items, R wanted rows, G groups, width W_g)::

    token_ids[T] positions[T] token_item[T] want_rows[R] item_start[B+1] item_ctx[B] state_slots[B]
    block_table_0[B, W_0] ... block_table_{G-1}[B, W_{G-1}]
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any

import numpy as np
import torch


@dataclass
class StepItem:
    seq: Any  # has .block_tables (one list per group) and .state_slot
    tokens: list[int]
    start: int
    want: list[int] = field(default_factory=list)


def section_offsets(t: int, b: int, r: int, widths: list[int]) -> dict[str, tuple[int, int]]:
    off, out = 0, {}
    for name, n in (("token_ids", t), ("positions", t), ("token_item", t), ("want_rows", r),
                    ("item_start", b + 1), ("item_ctx", b), ("state_slots", b), ("live_items", 1)):
        out[name] = (off, n)
        off += n
    for g, w in enumerate(widths):
        out[f"table{g}"] = (off, b * w)
        off += b * w
    out["_total"] = (0, off)
    return out


class StepBatch:
    """Views into the packed device buffer, plus the few host-side numbers parts may need."""

    def __init__(self, buf: torch.Tensor, t: int, b: int, r: int, widths: list[int]):
        self.buf, self.num_tokens, self.num_items, self.num_rows, self.widths = buf, t, b, r, list(widths)
        self.sections = section_offsets(t, b, r, self.widths)

        def view(name):
            o, n = self.sections[name]
            return buf[o : o + n]

        self.token_ids = view("token_ids")
        self.positions = view("positions")
        self.token_item = view("token_item")
        self.want_rows = view("want_rows")
        self.item_start = view("item_start")
        self.item_ctx = view("item_ctx")
        self.state_slots = view("state_slots")
        self.live_items = view("live_items")  # how many of the items are requests; the rest is padding
        self.least_live = b  # the fewest live items a (replayed) batch of this layout will ever hold
        self._tables = [view(f"table{g}").view(b, w) for g, w in enumerate(self.widths)]
        # host-side description, filled by pack(); static graph batches keep the capture-time values
        self.starts: list[int] = []
        self.qlens: list[int] = []
        self.slots_host: list[int] = []
        self.max_qlen = 1
        self.max_ctx = 1
        self.decode_only = True
        # what parts derive from this step's items for all of their layers (work lists and the like)
        self.derived: dict = {}

    def block_table(self, group: int) -> torch.Tensor:
        return self._tables[group]


def pack_host(items: list[StepItem], num_groups: int, widths: list[int] | None = None, pad_items: int = 0,
              spare_block: int = 0, spare_slot: int = 0):
    """Flatten ``items`` into one numpy int32 array. ``pad_items`` appends one-token items that
    write to the spare page (for replaying a graph captured at a larger batch)."""
    b = len(items) + pad_items
    qlens = [len(it.tokens) for it in items] + [1] * pad_items
    t = sum(qlens)
    r = sum(len(it.want) for it in items) + pad_items
    if widths is None:
        widths = [max(1, max(len(it.seq.block_tables[g]) for it in items)) for g in range(num_groups)]
    sec = section_offsets(t, b, r, widths)
    arr = np.zeros(sec["_total"][1], dtype=np.int32)
    tok_o, pos_o, item_o = sec["token_ids"][0], sec["positions"][0], sec["token_item"][0]
    want_o, start_o, ctx_o, slot_o = sec["want_rows"][0], sec["item_start"][0], sec["item_ctx"][0], sec["state_slots"][0]
    cursor, row = 0, 0
    for i, it in enumerate(items):
        n = len(it.tokens)
        arr[tok_o + cursor : tok_o + cursor + n] = it.tokens
        arr[pos_o + cursor : pos_o + cursor + n] = np.arange(it.start, it.start + n, dtype=np.int32)
        arr[item_o + cursor : item_o + cursor + n] = i
        for w in it.want:
            arr[want_o + row] = cursor + w
            row += 1
        arr[start_o + i] = cursor
        arr[ctx_o + i] = it.start + n
        arr[slot_o + i] = it.seq.state_slot if it.seq.state_slot >= 0 else spare_slot
        for g in range(num_groups):
            table = it.seq.block_tables[g]
            o = sec[f"table{g}"][0] + i * widths[g]
            arr[o : o + widths[g]] = spare_block
            arr[o : o + len(table)] = table
        cursor += n
    for i in range(len(items), b):
        arr[item_o + cursor] = i
        arr[want_o + row] = cursor
        row += 1
        arr[start_o + i] = cursor
        arr[ctx_o + i] = 1
        arr[slot_o + i] = spare_slot
        for g in range(num_groups):
            o = sec[f"table{g}"][0] + i * widths[g]
            arr[o : o + widths[g]] = spare_block
        cursor += 1
    arr[start_o + b] = cursor
    arr[sec["live_items"][0]] = len(items)
    return arr, t, b, r, widths


def check_pages(table: list[int], first: int, need: int, group: int) -> None:
    """Entries ``first .. need - 1`` of a block table must name pages (not -1, a page given back)."""
    if first < need and min(table[first:need]) < 0:
        raise ValueError(f"group {group}: a page the step reads or writes was already given back")


def validate_items(items: list[StepItem], vocab_size: int, block_size: int, groups, max_len: int | None = None,
                   pages: bool = True) -> None:
    """Host-side checks that make every index a kernel will form a valid one. ``pages=False`` leaves
    the scan of the block tables' entries to the caller (:func:`check_pages`)."""
    if not items:
        raise ValueError("a step needs at least one item")
    for it in items:
        n = len(it.tokens)
        if n < 1:
            raise ValueError("an item needs at least one token")
        if it.start < 0:
            raise ValueError(f"item starts at negative position {it.start}")
        if max_len is not None and it.start + n > max_len:
            raise ValueError(f"item reaches position {it.start + n}, beyond the limit of {max_len}")
        lo_tok, hi_tok = min(it.tokens), max(it.tokens)
        if lo_tok < 0 or hi_tok >= vocab_size:
            raise ValueError(f"token id {lo_tok if lo_tok < 0 else hi_tok} is outside the vocabulary of {vocab_size}")
        for w in it.want:
            if not 0 <= w < n:
                raise ValueError(f"wanted place {w} is outside the item's {n} tokens")
        need = -(-(it.start + n) // block_size)
        for g, spec in enumerate(groups):
            table = it.seq.block_tables[g]
            if len(table) < need:
                raise ValueError(f"block table of group {g} has {len(table)} pages, {need} are needed")
            if pages:
                first_key = max(0, it.start - spec.window + 1) if spec.window > 0 else 0
                check_pages(table, first_key // block_size, need, g)


def make_batch(items: list[StepItem], num_groups: int, device, spare_block: int = 0, spare_slot: int = 0) -> StepBatch:
    """Pack ``items`` and upload them: the batch an eager step runs on."""
    arr, t, b, r, widths = pack_host(items, num_groups, spare_block=spare_block, spare_slot=spare_slot)
    batch = StepBatch(torch.from_numpy(arr).to(device), t, b, r, widths)
    batch.starts = [it.start for it in items]
    batch.qlens = [len(it.tokens) for it in items]
    batch.slots_host = [it.seq.state_slot for it in items]
    batch.max_qlen = max(batch.qlens)
    batch.max_ctx = max(s + q for s, q in zip(batch.starts, batch.qlens))
    batch.decode_only = batch.max_qlen == 1
    return batch
