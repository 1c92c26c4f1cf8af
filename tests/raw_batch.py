"""A packer of step batches for tests of single parts and kernels: items are plain descriptions with
page ids chosen by the test (no cache manager behind them). It is written independently of the
engine's native packer, whose output ``tests/test_batch.py`` compares with it."""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

SECTIONS = ("token_ids", "positions", "token_item", "want_rows", "item_start", "item_ctx", "state_slots", "live_items",
            "temperatures", "sample_keys")


@dataclass
class RawItem:
    tables: list[list[int]]  # one block table per cache group
    tokens: list[int]
    start: int
    want: list[int] = field(default_factory=list)
    slot: int = -1


def raw_layout(t: int, b: int, r: int, widths: list[int]) -> dict:
    sizes = (t, t, t, r, b + 1, b, b, 2, r)  # live_items: the count, then the step's flags
    lay, at = {"tokens": t, "items": b, "rows": r, "widths": list(widths)}, 0
    for name, n in zip(SECTIONS, sizes):
        lay[name] = at
        at += n
    at += at % 2  # 64-bit keys start at an even offset
    lay["sample_keys"] = at
    at += 2 * r
    lay["token_source"] = at
    at += t
    lay["tables"] = []
    for w in widths:
        lay["tables"].append(at)
        at += b * w
    lay["total"] = at
    return lay


def pack_raw(items: list[RawItem], num_groups: int, widths: list[int] | None = None, pad_items: int = 0,
             spare_block: int = 0, spare_slot: int = 0):
    b = len(items) + pad_items
    t = sum(len(it.tokens) for it in items) + pad_items
    r = sum(len(it.want) for it in items) + pad_items
    if widths is None:
        widths = [max([1] + [len(it.tables[g]) for it in items]) for g in range(num_groups)]
    lay = raw_layout(t, b, r, widths)
    arr = np.zeros(lay["total"], dtype=np.int32)
    arr[lay["token_source"]:lay["token_source"] + t] = -1  # every token's id is in token_ids
    cursor = row = 0
    for i in range(b):
        it = items[i] if i < len(items) else RawItem([[] for _ in range(num_groups)], [0], 0, [0])
        n = len(it.tokens)
        arr[lay["token_ids"] + cursor:lay["token_ids"] + cursor + n] = it.tokens
        arr[lay["positions"] + cursor:lay["positions"] + cursor + n] = range(it.start, it.start + n)
        arr[lay["token_item"] + cursor:lay["token_item"] + cursor + n] = i
        for w in it.want:
            arr[lay["want_rows"] + row] = cursor + w
            row += 1
        arr[lay["item_start"] + i] = cursor
        arr[lay["item_ctx"] + i] = it.start + n
        arr[lay["state_slots"] + i] = it.slot if it.slot >= 0 else spare_slot
        for g in range(num_groups):
            o = lay["tables"][g] + i * widths[g]
            arr[o:o + widths[g]] = spare_block
            arr[o:o + len(it.tables[g])] = it.tables[g]
        cursor += n
    arr[lay["item_start"] + b] = cursor
    arr[lay["live_items"]] = len(items)
    return arr, lay


def make_raw_batch(items: list[RawItem], num_groups: int, device, spare_block: int = 0, spare_slot: int = 0):
    """The StepBatch a part's ``forward`` takes, from raw items."""
    import torch

    from mini_engine_amd.engine.batch import StepBatch

    arr, lay = pack_raw(items, num_groups, spare_block=spare_block, spare_slot=spare_slot)
    batch = StepBatch(torch.from_numpy(arr).to(device), lay)
    return batch.describe([it.start for it in items], [len(it.tokens) for it in items], [it.slot for it in items])
