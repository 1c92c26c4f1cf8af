"""Python face of the native host core (``csrc/host``): requests, page pools, scheduler and step
packing live in C++; this module holds the ctypes declarations and turns error codes into exceptions.

One :class:`HostCore` serves one engine. The block manager, the scheduler and every
:class:`~mini_engine_amd.engine.sequence.Sequence` of that engine are views of it.
"""

from __future__ import annotations

import ctypes
import weakref

import numpy as np

from ..ops.library import lib

_vp, _i32p, _i64p, _u8p = ctypes.c_void_p, ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_uint8)
_declared = False

LAYOUT_HEAD = ("tokens", "items", "rows", "total", "token_ids", "positions", "token_item", "want_rows", "item_start",
               "item_ctx", "state_slots", "live_items", "temperatures", "sample_keys", "token_source")


def _api():
    global _declared
    L = lib()
    if not _declared:
        L.me_core_new.restype = _vp
        L.me_core_new.argtypes = [_vp, _vp, ctypes.c_int, _vp, ctypes.c_int, ctypes.c_uint64]
        L.me_core_delete.argtypes = [_vp]
        L.me_core_delete.restype = None
        L.me_core_request.restype = ctypes.c_int64
        L.me_core_request.argtypes = [_vp, _vp, ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_int]
        for name in ("me_core_release", "me_core_drop", "me_core_drop_passed", "me_core_note_computed", "me_core_enqueue"):
            getattr(L, name).argtypes = [_vp, ctypes.c_int64]
        L.me_core_request_info.argtypes = [_vp, ctypes.c_int64, _vp]
        L.me_core_request_tokens.argtypes = [_vp, ctypes.c_int64, ctypes.c_int, ctypes.c_int, _vp]
        L.me_core_request_table.argtypes = [_vp, ctypes.c_int64, ctypes.c_int, _vp, ctypes.c_int]
        L.me_core_request_extend.argtypes = [_vp, ctypes.c_int64, _vp, ctypes.c_int]
        L.me_core_request_set.argtypes = [_vp, ctypes.c_int64, ctypes.c_int, ctypes.c_int64]
        L.me_core_set_limits.argtypes = [_vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp, ctypes.c_int]
        L.me_chain_digest.argtypes = [_vp, ctypes.c_int, _vp, ctypes.c_int, _vp]
        L.me_core_match.argtypes = [_vp, _vp, ctypes.c_int, _vp, ctypes.c_int]
        L.me_core_grow.argtypes = [_vp, ctypes.c_int64, ctypes.c_int, _vp, ctypes.c_int]
        L.me_core_forget_digests.argtypes = [_vp]
        L.me_core_can_ever_hold.argtypes = [_vp, ctypes.c_int]
        L.me_core_pages_info.argtypes = [_vp, _vp]
        L.me_core_pool.argtypes = [_vp, ctypes.c_int, _vp, _vp, _vp, _vp, _vp]
        L.me_core_find_digest.argtypes = [_vp, ctypes.c_int, _vp]
        L.me_core_slots.argtypes = [_vp, _vp, ctypes.c_int]
        L.me_core_release_page.argtypes = [_vp, ctypes.c_int, ctypes.c_int]
        L.me_core_plan.argtypes = [_vp]
        L.me_core_settle.argtypes = [_vp, _vp, ctypes.c_int, _vp, ctypes.c_int]
        L.me_core_queues.argtypes = [_vp, _vp, ctypes.c_int, _vp, ctypes.c_int, _vp]
        L.me_core_counters.argtypes = [_vp, _vp]
        L.me_core_step_clear.argtypes = [_vp]
        L.me_core_step_add.argtypes = [_vp, ctypes.c_int64, ctypes.c_int, ctypes.c_int, _vp, ctypes.c_int]
        L.me_core_step_items.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_int]
        L.me_core_step_summary.argtypes = [_vp, _vp]
        L.me_core_step_check.argtypes = [_vp, ctypes.c_int, ctypes.c_int]
        L.me_step_layout.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp, ctypes.c_int, _vp]
        L.me_core_step_layout.argtypes = [_vp, _vp, ctypes.c_int, _vp]
        L.me_core_step_pack.argtypes = [_vp, _vp, ctypes.c_int, _vp, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        L.me_core_step_refill.argtypes = [_vp, ctypes.c_int, _vp, _vp, ctypes.c_int, ctypes.c_int]
        L.me_core_forget_rows.argtypes = [_vp, ctypes.c_int]
        L.me_core_pack_padding.argtypes = [_vp, _vp, ctypes.c_int, _vp, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        L.me_core_settle_rows.argtypes = [_vp, _vp, ctypes.c_int, _vp, ctypes.c_int]
        L.me_core_plan_ahead.argtypes = [_vp]
        L.me_core_settle_in_flight.argtypes = [_vp, _vp, ctypes.c_int, _vp, ctypes.c_int]
        _declared = True
    return L


_RAISES = {1: ValueError, 2: RuntimeError, 3: AssertionError}


def _raise():
    L = lib()
    raise _RAISES.get(L.me_host_error_kind(), RuntimeError)(L.me_last_error().decode())


def _ok(code: int) -> int:
    if code < 0:
        _raise()
    return code


def _ptr(a: np.ndarray | None) -> _vp:
    return _vp(None) if a is None else _vp(a.ctypes.data)


def _ints(values) -> np.ndarray:
    return np.ascontiguousarray(values, dtype=np.int32)


def chain_digest(parent: bytes, token_ids) -> bytes:
    """blake2b-128 over ``parent`` followed by every token id as four little-endian bytes."""
    tokens = _ints(list(token_ids))
    out = np.zeros(16, dtype=np.uint8)
    par = np.frombuffer(parent, dtype=np.uint8) if parent else None
    _ok(_api().me_chain_digest(_ptr(par), len(parent), _ptr(tokens), len(tokens), _ptr(out)))
    return out.tobytes()


def step_layout(tokens: int, items: int, rows: int, widths: list[int]) -> dict[str, int | list[int]]:
    """Offsets (in int32 units) of the sections of a packed step buffer, as the native packer lays them out."""
    out = np.zeros(15 + 2 * len(widths), dtype=np.int32)
    _ok(_api().me_step_layout(tokens, items, rows, _ptr(_ints(widths)), len(widths), _ptr(out)))
    return _layout_dict(out, len(widths))


def _layout_dict(out: np.ndarray, groups: int) -> dict:
    d = {k: int(v) for k, v in zip(LAYOUT_HEAD, out[:15])}
    d["widths"] = [int(out[15 + 2 * g]) for g in range(groups)]
    d["tables"] = [int(out[16 + 2 * g]) for g in range(groups)]
    return d


class HostCore:
    """Owner of the native core object. ``groups`` is a list of ``(window, num_pages)``."""

    def __init__(self, block_size: int, groups: list[tuple[int, int]], enable_prefix_caching: bool = True,
                 num_state_slots: int = 0, has_state: bool = False, max_num_seqs: int = 1 << 20,
                 max_num_batched_tokens: int = 1 << 30, max_model_len: int = 1 << 30, eos_token_ids=(), seed: int = 0):
        self._L = _api()
        self.block_size, self.num_groups = int(block_size), len(groups)
        settings = _ints([block_size, int(bool(enable_prefix_caching)), num_state_slots, int(bool(has_state)), max_num_seqs,
                          max_num_batched_tokens, max_model_len])
        flat = _ints([v for g in groups for v in g])
        eos = _ints(sorted(int(e) for e in eos_token_ids))
        self._box = self._L.me_core_new(_ptr(settings), _ptr(flat), len(groups), _ptr(eos), len(eos),
                                        ctypes.c_uint64(seed & ((1 << 64) - 1)))
        if not self._box:
            _raise()
        self._box = _vp(self._box)
        self.sequences: "weakref.WeakValueDictionary[int, object]" = weakref.WeakValueDictionary()
        self._info = np.zeros(16, dtype=np.int64)

    def __del__(self):
        box, self._box = getattr(self, "_box", None), None
        if box:
            self._L.me_core_delete(box)

    # ---- limits of the scheduler (a scheduler made for an existing block manager sets them)
    def set_limits(self, max_num_seqs: int, max_num_batched_tokens: int, max_model_len: int, eos_token_ids=()) -> None:
        eos = _ints(sorted(int(e) for e in eos_token_ids))
        _ok(self._L.me_core_set_limits(self._box, max_num_seqs, max_num_batched_tokens, max_model_len, _ptr(eos), len(eos)))

    # ---- requests
    def request(self, tokens, max_tokens: int, temperature: float, ignore_eos: bool) -> int:
        t = _ints(tokens)
        h = self._L.me_core_request(self._box, _ptr(t), len(t), max_tokens, temperature, int(ignore_eos))
        if h < 0:
            _raise()
        return h

    def release(self, handle: int) -> None:
        if self._box:
            self._L.me_core_release(self._box, handle)

    def info(self, handle: int) -> np.ndarray:
        """phase, tokens, prompt tokens, computed, cached at admission, preemptions, state slot, table epoch, digests"""
        _ok(self._L.me_core_request_info(self._box, handle, _ptr(self._info)))
        return self._info

    def tokens(self, handle: int, start: int = 0, count: int | None = None) -> list[int]:
        if count is None:
            count = int(self.info(handle)[1]) - start
        out = np.zeros(max(count, 1), dtype=np.int32)
        _ok(self._L.me_core_request_tokens(self._box, handle, start, count, _ptr(out)))
        return out[:count].tolist()

    def table(self, handle: int, group: int) -> list[int]:
        n = _ok(self._L.me_core_request_table(self._box, handle, group, None, 0))
        out = np.zeros(max(n, 1), dtype=np.int32)
        _ok(self._L.me_core_request_table(self._box, handle, group, _ptr(out), n))
        return out[:n].tolist()

    def extend(self, handle: int, tokens) -> None:
        t = _ints(tokens)
        _ok(self._L.me_core_request_extend(self._box, handle, _ptr(t), len(t)))

    def set_field(self, handle: int, what: int, value: int) -> None:
        _ok(self._L.me_core_request_set(self._box, handle, what, value))

    # ---- pages
    def match(self, tokens) -> list[list[int]]:
        t = _ints(tokens)
        cap = max(1, len(t) // self.block_size)
        out = np.zeros(cap * self.num_groups, dtype=np.int32)
        blocks = _ok(self._L.me_core_match(self._box, _ptr(t), len(t), _ptr(out), cap))
        return [out[g * blocks:(g + 1) * blocks].tolist() for g in range(self.num_groups)]

    def grow(self, handle: int, num_tokens: int, hits: list[list[int]] | None = None) -> bool:
        if hits and any(hits):
            if len(hits) != self.num_groups or len({len(h) for h in hits}) != 1:
                raise ValueError("cached pages must be given per cache group, as many for each")
            flat = _ints([p for h in hits for p in h])
            return bool(_ok(self._L.me_core_grow(self._box, handle, num_tokens, _ptr(flat), len(hits[0]))))
        return bool(_ok(self._L.me_core_grow(self._box, handle, num_tokens, None, 0)))

    def drop(self, handle: int) -> None:
        _ok(self._L.me_core_drop(self._box, handle))

    def drop_passed(self, handle: int) -> int:
        return _ok(self._L.me_core_drop_passed(self._box, handle))

    def note_computed(self, handle: int) -> None:
        _ok(self._L.me_core_note_computed(self._box, handle))

    def forget_digests(self) -> None:
        _ok(self._L.me_core_forget_digests(self._box))

    def can_ever_hold(self, tokens: int) -> bool:
        return bool(_ok(self._L.me_core_can_ever_hold(self._box, tokens)))

    def pages_info(self) -> np.ndarray:
        """groups, caching on, least free pages over the groups, evictions, state slots, free slots"""
        _ok(self._L.me_core_pages_info(self._box, _ptr(self._info)))
        return self._info

    def pool(self, group: int, num_pages: int) -> dict:
        """A pool as arrays: holders, has_digest, digests (bytes or None per page), free_order, evictions."""
        holders = np.zeros(num_pages, dtype=np.int32)
        flags = np.zeros(num_pages, dtype=np.uint8)
        digests = np.zeros(16 * num_pages, dtype=np.uint8)
        order = np.zeros(num_pages, dtype=np.int32)
        info = np.zeros(3, dtype=np.int64)
        free = _ok(self._L.me_core_pool(self._box, group, _ptr(holders), _ptr(flags), _ptr(digests), _ptr(order), _ptr(info)))
        return {"holders": holders.tolist(), "free_order": order[:free].tolist(), "evictions": int(info[2]),
                "digests": [digests[16 * p:16 * p + 16].tobytes() if flags[p] else None for p in range(num_pages)]}

    def find_digest(self, group: int, digest: bytes) -> int | None:
        """The page that serves the prefix with this digest, or None."""
        code = self._L.me_core_find_digest(self._box, group, _ptr(np.frombuffer(digest, dtype=np.uint8)))
        if code == -1:
            _raise()
        return None if code == -2 else code

    def release_page(self, group: int, page: int) -> None:
        """Drop one holder of a page by hand (diagnostics; requests give their pages back through :meth:`drop`)."""
        _ok(self._L.me_core_release_page(self._box, group, page))

    def slots_taken(self) -> list[bool]:
        n = int(self.pages_info()[4])
        flags = np.zeros(max(n, 1), dtype=np.uint8)
        _ok(self._L.me_core_slots(self._box, _ptr(flags), n))
        return [bool(f) for f in flags[:n]]

    # ---- scheduler
    def enqueue(self, handle: int) -> None:
        _ok(self._L.me_core_enqueue(self._box, handle))

    def plan(self) -> int:
        return _ok(self._L.me_core_plan(self._box))

    def settle(self, next_tokens: np.ndarray) -> list[int]:
        done = np.zeros(max(1, len(next_tokens)), dtype=np.int64)
        n = _ok(self._L.me_core_settle(self._box, _ptr(next_tokens), len(next_tokens), _ptr(done), len(done)))
        return done[:n].tolist()

    def settle_rows(self, drawn: np.ndarray) -> list[int]:
        """Settle the planned step from the tokens drawn for its wanted rows (int32, in row order)."""
        done = np.zeros(max(1, len(drawn)), dtype=np.int64)
        n = _ok(self._L.me_core_settle_rows(self._box, _ptr(drawn), len(drawn), _ptr(done), len(done)))
        return done[:n].tolist()

    def plan_ahead(self) -> int:
        """The planned step has been launched: when the step after it is known but for the token ids (every
        running request decodes one more token, nobody waits for admission), make the launched step the one
        in flight and plan that next step, whose ids the device takes from the draws in flight. Number of
        items of the new step, or 0 when nothing was changed."""
        return _ok(self._L.me_core_plan_ahead(self._box))

    def settle_in_flight(self, drawn: np.ndarray) -> list[int]:
        """The draws of the step in flight (int32, one per item in row order); the step planned ahead stays."""
        done = np.zeros(max(1, len(drawn)), dtype=np.int64)
        n = _ok(self._L.me_core_settle_in_flight(self._box, _ptr(drawn), len(drawn), _ptr(done), len(done)))
        return done[:n].tolist()

    def queues(self) -> tuple[list[int], list[int]]:
        counts = np.zeros(2, dtype=np.int32)
        _ok(self._L.me_core_queues(self._box, None, 0, None, 0, _ptr(counts)))
        w, r = np.zeros(max(1, counts[0]), dtype=np.int64), np.zeros(max(1, counts[1]), dtype=np.int64)
        _ok(self._L.me_core_queues(self._box, _ptr(w), len(w), _ptr(r), len(r), _ptr(counts)))
        return w[:counts[0]].tolist(), r[:counts[1]].tolist()

    def counters(self) -> np.ndarray:
        """preemptions, tokens served by the prefix cache, evictions, unfinished, tokens generated"""
        _ok(self._L.me_core_counters(self._box, _ptr(self._info)))
        return self._info

    # ---- the step
    def step_clear(self) -> None:
        _ok(self._L.me_core_step_clear(self._box))

    def step_add(self, handle: int, start: int, count: int, want) -> None:
        w = _ints(want)
        _ok(self._L.me_core_step_add(self._box, handle, start, count, _ptr(w), len(w)))

    def step_items(self) -> tuple[list[int], list[int], list[int], list[int], list[int]]:
        """(handles, first positions, token counts, numbers of wanted places, state slots) of the current step's items."""
        n = int(self.step_summary()[1])
        h = np.zeros(max(1, n), dtype=np.int64)
        s, c, w, sl = (np.zeros(max(1, n), dtype=np.int32) for _ in range(4))
        _ok(self._L.me_core_step_items(self._box, _ptr(h), _ptr(s), _ptr(c), _ptr(w), _ptr(sl), n))
        return h[:n].tolist(), s[:n].tolist(), c[:n].tolist(), w[:n].tolist(), sl[:n].tolist()

    def step_summary(self) -> np.ndarray:
        """tokens, items, wanted rows, longest item, longest context, decode only, last places only, any temperature"""
        out = np.zeros(8, dtype=np.int32)
        _ok(self._L.me_core_step_summary(self._box, _ptr(out)))
        return out

    def step_check(self, vocab_size: int, scan_pages: bool = True) -> None:
        _ok(self._L.me_core_step_check(self._box, vocab_size, int(scan_pages)))

    def step_layout(self, widths: list[int] | None = None, pad_items: int = 0) -> dict:
        out = np.zeros(15 + 2 * self.num_groups, dtype=np.int32)
        _ok(self._L.me_core_step_layout(self._box, _ptr(None if widths is None else _ints(widths)), pad_items, _ptr(out)))
        return _layout_dict(out, self.num_groups)

    def step_pack(self, dst: np.ndarray, widths: list[int] | None = None, pad_items: int = 0, spare_page: int = 0,
                  spare_slot: int = 0) -> int:
        return _ok(self._L.me_core_step_pack(self._box, _ptr(dst), len(dst), _ptr(None if widths is None else _ints(widths)),
                                             pad_items, spare_page, spare_slot))

    def pack_padding(self, dst: np.ndarray, widths: list[int], items: int, spare_page: int, spare_slot: int) -> int:
        return _ok(self._L.me_core_pack_padding(self._box, _ptr(dst), len(dst), _ptr(_ints(widths)), items, spare_page, spare_slot))

    def forget_rows(self, bucket: int) -> None:
        """Forget what the rows of a graph bucket's buffer hold (the buffer was made anew)."""
        _ok(self._L.me_core_forget_rows(self._box, bucket))

    def step_refill(self, bucket: int, dst: np.ndarray, widths: list[int], spare_page: int, spare_slot: int) -> None:
        _ok(self._L.me_core_step_refill(self._box, bucket, _ptr(dst), _ptr(_ints(widths)), spare_page, spare_slot))
