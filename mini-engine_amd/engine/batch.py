"""One step's batch on the device: views into the packed int32 buffer that the native host core
fills (``csrc/host/step.cpp``) and that is uploaded with one copy.

An item is ``(request, its next tokens, the position of the first of them, the places among them
whose logits are wanted)``. Items are packed one after another (reference:
``src/mini_engine/engine.py:200-226``); instead of a padded mask the kernels get, per token, its
absolute position and the index of its item, and per item and cache group a row of the block table.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any

import torch


@dataclass
class StepItem:
    """``tokens`` are the request's tokens at positions ``start .. start + len(tokens) - 1`` (they
    have to be part of the request already); ``want`` are places among them."""

    seq: Any
    tokens: list[int]
    start: int
    want: list[int] = field(default_factory=list)


class StepBatch:
    """Views into the packed device buffer, plus the few host-side numbers parts may need.
    ``layout`` is what :func:`mini_engine_amd.engine.core.step_layout` returns."""

    def __init__(self, buf: torch.Tensor, layout: dict):
        self.buf, self.layout = buf, layout
        t, b, r = layout["tokens"], layout["items"], layout["rows"]
        self.num_tokens, self.num_items, self.num_rows, self.widths = t, b, r, list(layout["widths"])

        def view(name, n):
            o = layout[name]
            return buf[o : o + n]

        self.token_ids = view("token_ids", t)
        self.positions = view("positions", t)
        self.token_item = view("token_item", t)
        self.want_rows = view("want_rows", r)
        self.item_start = view("item_start", b + 1)
        self.item_ctx = view("item_ctx", b)
        self.state_slots = view("state_slots", b)
        self.live_items = view("live_items", 1)  # how many of the items are requests; the rest is padding
        self.temperatures = view("temperatures", r).view(torch.float32)  # per wanted row; 0: take the argmax
        self.sample_keys = view("sample_keys", 2 * r).view(torch.int64)  # per wanted row: the key of its draw
        self.token_source = view("token_source", t)  # -1, or the row of the fed tokens that holds the token's id
        self.least_live = b  # the fewest live items a (replayed) batch of this layout will ever hold
        self._tables = [buf[o : o + b * w].view(b, w) for o, w in zip(layout["tables"], self.widths)]
        # host-side description; static graph batches keep the capture-time values
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

    def describe(self, starts: list[int], qlens: list[int], slots: list[int]) -> "StepBatch":
        self.starts, self.qlens, self.slots_host = list(starts), list(qlens), list(slots)
        self.max_qlen = max(qlens)
        self.max_ctx = max(s + q for s, q in zip(starts, qlens))
        self.decode_only = self.max_qlen == 1
        return self
