"""Python face of the native step program (``csrc/host/program.cpp``, ``csrc/host/runner.cpp``).

When a model is built, every part writes the operations of its forward pass into a
:class:`StepProgram` (a part's ``emit`` method; it says what the part computes, not which kernels
run). A step of the model then is one call into C++, which checks and packs the step that the
host core holds, uploads the indices, picks a kernel per operation for the step's size, launches
them all and draws the next tokens. A part that has no ``emit`` (a part defined outside the package,
with code of its own) enters the program as a *call*: the program hands its ``forward`` the step's
values as tensors when the step reaches it, so such a part, with or without state of its own, runs in
the same one pass as every other.

Values are ``[tokens, columns]`` buffers of a step; parts get them from the program and the program
hands a buffer out again once the scope that took it has ended, so a model of any depth needs the
buffers of one layer.
"""

from __future__ import annotations

import contextlib
import ctypes
import weakref

import numpy as np
import torch

from ..ops.library import lib

_vp, _i64, _i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
_declared = False

EMBED, NORM_LINEAR, NORM, LINEAR, LINEAR_DELTA, DELTA, ATTENTION, HEAD, SAMPLE, ADD, CALL, HEAD_ROWS = range(12)
_RAISES = {1: ValueError, 2: RuntimeError, 3: AssertionError}


class _RawFrame(ctypes.Structure):  # csrc/host/program.h: CallFrame
    _fields_ = [("context", _vp), ("in_", _vp), ("out", _vp), ("x", _vp), ("in_cols", _i64), ("out_cols", _i64),
                ("in_elem", _i32), ("out_elem", _i32), ("tokens", _i32), ("rows", _i32), ("stream", _vp)]


_CALL_FN = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.POINTER(_RawFrame))


class Frame:
    """What a called part sees of the step that has reached it: its input and output values and the residual
    stream as tensors (views into the step's memory, valid during the call only) and the step's batch."""

    def __init__(self, program: "StepProgram", raw: _RawFrame):
        self.program, self.tokens, self.rows = program, int(raw.tokens), int(raw.rows)
        dtype_of = {2: torch.bfloat16, 4: torch.float32}
        arena = program.current_arena
        self.input = view_in(arena, raw.in_, (self.tokens, int(raw.in_cols)), dtype_of[raw.in_elem]) if raw.in_ else None
        self.output = view_in(arena, raw.out, (self.tokens, int(raw.out_cols)), dtype_of[raw.out_elem]) if raw.out else None
        self.x = view_in(arena, raw.x, (self.tokens, program.hidden), torch.float32)

    @property
    def batch(self):
        """The step's batch (:class:`~mini_engine_amd.engine.batch.StepBatch`), made once per step."""
        return self.program.current_batch()

    def write(self, result) -> None:
        """A part's result into the output value: a tensor ``[tokens, columns]``, or partial sums over runs of k."""
        from ..ops.kernels import PartialSums

        if isinstance(result, PartialSums):
            result = result.parts.sum(dim=0)
        if tuple(result.shape) != tuple(self.output.shape):
            raise ValueError(f"a part returned {tuple(result.shape)} where the step has {tuple(self.output.shape)}")
        self.output.copy_(result)


def _api():
    global _declared
    L = lib()
    if not _declared:
        L.me_runner_new.restype = _vp
        L.me_runner_new.argtypes = [_i32, _i32, _i32]
        L.me_runner_delete.argtypes = [_vp]
        L.me_runner_delete.restype = None
        L.me_runner_value.argtypes = [_vp, _i64, _i32]
        L.me_runner_op.argtypes = [_vp, _i32, _i32, _i32, _vp, _vp, _vp]
        L.me_runner_arena_need.restype = _i64
        L.me_runner_arena_need.argtypes = [_vp, _i64, _i64, _i64, _i64]
        L.me_runner_index_need.restype = _i64
        L.me_runner_index_need.argtypes = [_vp, _i32, _i32, _i32, _vp, _i32]
        L.me_runner_memory.argtypes = [_vp, _vp, _i64, _vp, _vp, _i64, _vp, _i64, _i32, _i32]
        L.me_runner_step.argtypes = [_vp, _vp, _vp, _vp]
        L.me_runner_static.argtypes = [_vp, _vp, _i64, _vp, _i32, _vp, _i32, _i32, _i32, _vp, _i32, _vp, _vp]
        _declared = True
    return L


def _ok(code: int) -> int:
    if code < 0:
        L = lib()
        raise _RAISES.get(L.me_runner_error_kind(), RuntimeError)(L.me_last_error().decode())
    return code


class Normed:
    """The residual add and the norm that a block owes before a part, not yet written into the
    program. The part's first product takes it as its input (the program then fuses add, norm and
    product where the step is small enough); ``value()`` gives the normed activations as a value of
    their own."""

    def __init__(self, program: "StepProgram", weight: torch.Tensor, eps: float):
        self.program, self.weight, self.eps = program, weight, float(eps)
        self.used = False
        self._value: int | None = None

    def value(self) -> int:
        if self._value is None:
            p = self.program
            self._value = p.take(p.hidden, p.elem)
            p.op(NORM, out=self._value, ptrs=[self.weight], floats=[self.eps])
            p.pending_consumed()
            self.used = True
        return self._value


class CalledNorm:
    """As :class:`Normed`, for a norm that is no RMS norm: the residual add as a kernel of its own, then the norm
    part's ``forward`` on the residual stream. Parts get its value; nothing of it rides on their products."""

    def __init__(self, program: "StepProgram", norm):
        self.program, self.norm = program, norm
        self.used = False
        self._value: int | None = None

    def value(self) -> int:
        if self._value is None:
            p, norm = self.program, self.norm
            p.add()
            self._value = p.call(lambda frame: frame.output.copy_(norm.forward(frame.x)), out_cols=p.hidden)
            self.used = True
        return self._value


class StepProgram:
    def __init__(self, dtype: torch.dtype, hidden: int, vocab: int, max_positions: int):
        self._L = _api()
        self.dtype, self.hidden, self.vocab, self.max_positions = dtype, int(hidden), int(vocab), int(max_positions)
        self.elem = 4 if dtype is torch.float32 else 2
        handle = self._L.me_runner_new(0 if dtype is torch.float32 else 1, self.hidden, self.vocab)
        if not handle:
            raise RuntimeError(lib().me_last_error().decode())
        self.handle = _vp(handle)
        self._keep: list[torch.Tensor] = []  # every tensor whose address an operation holds
        self._free: dict[tuple[int, int], list[int]] = {}
        self._value_kinds: list[tuple[int, int]] = []
        self._scopes: list[list[int]] = []
        self._pending_value: int | None = None
        self.num_ops = 0
        self.draws = False
        self.last_prefill_columns = 0  # query columns of the prefill attention's blocks in the last eager step (0: none ran)
        # called parts: their C trampolines (kept alive), the memory and the batch of the step that is running,
        # and the exception a call raised (raised again once the step's call into C++ has come back)
        self._calls: list = []
        self.current_arena: torch.Tensor | None = None
        self.current_batch = lambda: None
        self.call_error: BaseException | None = None

    def __del__(self):
        handle, self.handle = getattr(self, "handle", None), None
        if handle:
            self._L.me_runner_delete(handle)

    # ------------------------------------------------------------------ values
    def take(self, cols: int, elem: int | None = None) -> int:
        """A ``[tokens, cols]`` buffer (elements of the compute dtype unless ``elem`` bytes are asked for)
        that stays the caller's until the scope it was taken in ends."""
        key = (int(cols), int(elem or self.elem))
        pool = self._free.setdefault(key, [])
        if pool:
            v = pool.pop()
        else:
            v = _ok(self._L.me_runner_value(self.handle, key[0], key[1]))
            self._value_kinds.append(key)
        if self._scopes:
            self._scopes[-1].append(v)
        return v

    @contextlib.contextmanager
    def scope(self):
        """Values taken inside are handed out again afterwards; the one that holds the pending delta of
        the residual stream only once the next norm has added it."""
        self._scopes.append([])
        try:
            yield
        finally:
            for v in self._scopes.pop():
                if v != self._pending_value:
                    self._give_back(v)

    def _give_back(self, v: int) -> None:
        self._free[self._value_kinds[v]].append(v)

    def pending_consumed(self) -> None:
        v, self._pending_value = self._pending_value, None
        if v is not None and not any(v in s for s in self._scopes):
            self._give_back(v)

    # -------------------------------------------------------------- operations
    def op(self, kind: int, in_: int = -1, out: int = -1, ptrs=(), ints=(), floats=()) -> None:
        p = (ctypes.c_void_p * 6)()
        for i, t in enumerate(ptrs):
            if t is not None:
                if not t.is_contiguous():
                    raise ValueError("a step program holds contiguous tensors only")
                self._keep.append(t)
                p[i] = t.data_ptr()
        iv = (ctypes.c_int64 * 10)(*[int(v) for v in ints])
        fv = (ctypes.c_float * 2)(*[float(v) for v in floats])
        self.num_ops = _ok(self._L.me_runner_op(self.handle, kind, in_, out, p, iv, fv))

    def embed(self, table: torch.Tensor, multiplier: float = 1.0) -> None:
        """The residual stream starts as the tokens' rows of ``table``, times ``multiplier``."""
        self._want(table, self.dtype, (self.vocab, self.hidden), "embedding table")
        self.op(EMBED, ptrs=[table], floats=[multiplier])

    def normed(self, norm) -> Normed:
        """The add-and-norm before a part, for a norm that is RMS-shaped (``norm.as_fused()`` gives its
        float32 weight and its eps)."""
        weight, eps = norm.as_fused()
        self._want(weight, torch.float32, (self.hidden,), "norm weight")
        return Normed(self, weight, eps)

    def linear(self, x, weight: torch.Tensor, gated: "bool | str" = False) -> int:
        """``x @ weight.T`` (``gated``, True or the name of an activation: ``act(gate) * up`` with the weight's
        rows being gate rows, then up rows) for a value or a :class:`Normed`; returns the value that holds
        the result."""
        from ..ops.kernels import gate_code

        gate = gate_code(gated)
        rows, k = weight.shape
        self._want(weight, self.dtype, None, "weight")
        if gated and rows % 2:
            raise ValueError("a gated product needs as many gate rows as up rows")
        out = self.take(rows // 2 if gated else rows)
        if isinstance(x, Normed) and x._value is None:
            if k != self.hidden:
                raise ValueError("a product behind the norm reads the hidden size")
            self.op(NORM_LINEAR, out=out, ptrs=[x.weight, weight], ints=[rows, k, gate], floats=[x.eps])
            x.used = True
            self.pending_consumed()
            return out
        src = x.value() if isinstance(x, (Normed, CalledNorm)) else x
        if self._value_kinds[src][0] != k:
            raise ValueError(f"the weight reads {k} columns, the value has {self._value_kinds[src][0]}")
        self.op(LINEAR, in_=src, out=out, ptrs=[None, weight], ints=[rows, k, gate])
        return out

    def linear_delta(self, x: int, weight: torch.Tensor) -> None:
        """``x @ weight.T`` as the part's result: the delta that the next norm adds to the residual stream."""
        rows, k = weight.shape
        self._want(weight, self.dtype, (self.hidden, self._value_kinds[x][0]), "weight")
        out = self.take(rows)
        self.op(LINEAR_DELTA, in_=x, out=out, ptrs=[None, weight], ints=[rows, k])
        self._pending_value = out

    def delta(self, x: int) -> None:
        """A value ``[tokens, hidden]`` in the compute dtype as the part's result."""
        if self._value_kinds[x] != (self.hidden, self.elem):
            raise ValueError("a part's result has the hidden size and the compute dtype")
        self.op(DELTA, in_=x)
        self._pending_value = x

    def attention(self, qkv: int, *, q_norm: torch.Tensor | None, k_norm: torch.Tensor | None, rope: torch.Tensor | None,
                  k_cache: torch.Tensor, v_cache: torch.Tensor, heads: int, kv_heads: int, head_dim: int, block_size: int,
                  window: int, writes: bool, group: int, eps: float, scale: float) -> int:
        """Per-head q/k norm, rotation, page write and causal attention over the request's pages for a
        value ``[tokens, (heads + 2 kv_heads) head_dim]`` (``writes`` false: ``[tokens, heads head_dim]``,
        the pages are another layer's); returns the value ``[tokens, heads head_dim]``."""
        cols = (heads + (2 * kv_heads if writes else 0)) * head_dim
        if self._value_kinds[qkv] != (cols, self.elem):
            raise ValueError(f"the attention's input has {self._value_kinds[qkv][0]} columns, not {cols}")
        rotary_dim = covers = 0
        if rope is not None:
            self._want(rope, torch.float32, None, "rotary table")
            rotary_dim, covers = 2 * rope.shape[2], rope.shape[0]
            if covers < self.max_positions:
                raise ValueError(f"the rotary table covers {covers} positions of {self.max_positions}")
        out = self.take(heads * head_dim)
        self.op(ATTENTION, in_=qkv, out=out, ptrs=[q_norm, k_norm, rope, k_cache, v_cache],
                ints=[heads, kv_heads, head_dim, rotary_dim, block_size, window, int(writes), group, covers],
                floats=[eps, scale])
        return out

    def add(self) -> None:
        """The pending delta into the residual stream, as a kernel of its own (before a norm that is not RMS-shaped)."""
        self.op(ADD)
        self.pending_consumed()

    def call(self, fn, in_: int = -1, out_cols: int | None = None, out_elem: int | None = None) -> int:
        """A part with code of its own: when a step reaches this place, ``fn(frame)`` is called with a
        :class:`Frame` (the value ``in_`` as ``frame.input``, a new value of ``out_cols`` columns as
        ``frame.output``, the residual stream as ``frame.x``, the step's batch). It launches what it has to on the
        current stream and returns nothing. Returns the output value (-1 without ``out_cols``)."""
        out = self.take(out_cols, out_elem) if out_cols else -1
        me = weakref.ref(self)  # (the program keeps the trampoline: no cycle through it)

        def trampoline(raw):
            program = me()
            try:
                fn(Frame(program, raw.contents))
                return 0
            except BaseException as e:  # an exception cannot cross the C frames in between: it is raised after the step
                program.call_error = e
                return 1

        c_fn = _CALL_FN(trampoline)
        self._calls.append(c_fn)
        p = (ctypes.c_void_p * 6)()
        p[0] = ctypes.cast(c_fn, ctypes.c_void_p).value
        iv, fv = (ctypes.c_int64 * 10)(), (ctypes.c_float * 2)()
        self.num_ops = _ok(self._L.me_runner_op(self.handle, CALL, in_, out, p, iv, fv))
        return out

    def call_part(self, part, h, extra=()) -> int:
        """A mixer or feed-forward without ``emit``: its ``forward(h, batch, *extra)`` on the normed activations, its
        result as a value ``[tokens, hidden]``."""
        src = h.value()
        return self.call(lambda frame: frame.write(part.forward(frame.input, frame.batch, *extra)), in_=src,
                         out_cols=self.hidden)

    def normed_by(self, norm) -> "CalledNorm":
        """The add-and-norm before a part, for a norm part of any shape (its ``forward`` is called)."""
        return CalledNorm(self, norm)

    def head_by(self, norm, weight: torch.Tensor, logit_scale: float = 1.0) -> None:
        """As :meth:`head`, for a final norm of any shape: the add, the norm part's ``forward`` on the wanted rows,
        the head product."""
        self._want(weight, self.dtype, (self.vocab, self.hidden), "head")
        self.add()

        def run(frame):
            if frame.rows:
                rows = frame.batch.want_rows[:frame.rows].long()
                frame.output[:frame.rows].copy_(norm.forward(frame.x.index_select(0, rows)))

        with self.scope():
            picked = self.call(run, out_cols=self.hidden)
            self.op(HEAD_ROWS, in_=picked, ptrs=[None, weight], floats=[0.0, logit_scale])

    def head(self, norm, weight: torch.Tensor, logit_scale: float = 1.0) -> None:
        """Final norm of the wanted rows, the head product, the logits times ``logit_scale``."""
        norm_weight, eps = norm.as_fused()
        self._want(weight, self.dtype, (self.vocab, self.hidden), "head")
        self.op(HEAD, ptrs=[norm_weight, weight], floats=[eps, logit_scale])
        self.pending_consumed()

    def sample(self) -> None:
        self.op(SAMPLE)
        self.draws = True

    def _want(self, t: torch.Tensor, dtype, shape, what: str) -> None:
        if t.dtype is not dtype or (shape is not None and tuple(t.shape) != tuple(shape)) or not t.is_cuda:
            raise ValueError(f"{what}: expected {dtype} {shape} on the GPU, got {t.dtype} {tuple(t.shape)} on {t.device}")

    # ------------------------------------------------------------------ memory
    def arena_need(self, tokens: int, items: int, rows: int, max_ctx: int) -> int:
        return _ok(self._L.me_runner_arena_need(self.handle, tokens, items, rows, max_ctx))

    def index_need(self, tokens: int, items: int, rows: int, widths: list[int]) -> int:
        w = np.ascontiguousarray(widths, dtype=np.int32)
        return _ok(self._L.me_runner_index_need(self.handle, tokens, items, rows, _vp(w.ctypes.data), len(w)))


class StepMemory:
    """What eager steps of a program run on: an arena for activations and workspaces, two pinned
    staging buffers and the index buffer on the device, sized for the largest step seen so far."""

    def __init__(self, program: StepProgram, device, widths: list[int], spare_page: int, spare_slot: int):
        self.program, self.device, self.widths = program, device, list(widths)
        self.spare_page, self.spare_slot = spare_page, spare_slot
        self.caps = (0, 0, 0, 0)
        self.arena = self.staging = self.index = None

    def ensure(self, tokens: int, items: int, rows: int, max_ctx: int) -> None:
        c = self.caps
        if tokens <= c[0] and items <= c[1] and rows <= c[2] and max_ctx <= c[3]:
            return
        torch.cuda.synchronize()  # nothing of the old memory is in use once the device is idle
        c = self.caps = (max(tokens, c[0]), max(items, c[1]), max(rows, c[2]), max(max_ctx, c[3]))
        p = self.program
        self.arena = torch.empty(p.arena_need(*c), dtype=torch.uint8, device=self.device)
        ints = p.index_need(c[0], c[1], c[2], self.widths)
        self.staging = [torch.empty(ints, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self.index = torch.empty(ints, dtype=torch.int32, device=self.device)
        _ok(p._L.me_runner_memory(p.handle, _vp(self.arena.data_ptr()), self.arena.numel(), _vp(self.staging[0].data_ptr()),
                                  _vp(self.staging[1].data_ptr()), ints, _vp(self.index.data_ptr()), ints, self.spare_page,
                                  self.spare_slot))


def view_in(arena: torch.Tensor, address: int, shape: tuple[int, ...], dtype: torch.dtype) -> torch.Tensor:
    """The tensor of ``shape`` that lies at ``address`` inside ``arena``."""
    offset = address - arena.data_ptr()
    count = int(np.prod(shape)) * torch.empty((), dtype=dtype).element_size()
    if offset < 0 or offset + count > arena.numel():
        raise RuntimeError("a step's result lies outside its arena")
    return arena[offset:offset + count].view(dtype).view(shape)


def _after_calls(program: StepProgram, code: int) -> None:
    """The step's call into C++ has come back: an exception that a called part raised on the way is raised now."""
    error, program.call_error = program.call_error, None
    if error is not None:
        raise error
    _ok(code)


def run_step(program: StepProgram, memory: StepMemory, core) -> tuple[torch.Tensor | None, torch.Tensor | None, int]:
    """Run the step that ``core`` holds; (logits float32 [rows, vocab], drawn int32 [rows], rows)."""
    out = np.zeros(4, dtype=np.int64)
    stream = _vp(torch.cuda.current_stream().cuda_stream)
    program.current_arena = memory.arena
    _after_calls(program, program._L.me_runner_step(program.handle, core._box, stream, _vp(out.ctypes.data)))
    rows = int(out[1])
    program.last_prefill_columns = int(out[3])
    logits = view_in(memory.arena, int(out[0]), (rows, program.vocab), torch.float32) if out[0] else None
    drawn = view_in(memory.arena, int(out[2]), (rows,), torch.int32) if out[2] else None
    return logits, drawn, rows


def run_static(program: StepProgram, arena: torch.Tensor, index: torch.Tensor, bucket: int, widths: list[int], max_ctx: int,
               least_live: int, drawn: torch.Tensor | None = None, fed: bool = False):
    """Launch a decode step of ``bucket`` one-token items whose indices are in ``index`` on the device
    (what a graph captures); (logits [bucket, vocab], drawn [bucket])."""
    out = np.zeros(4, dtype=np.int64)
    w = np.ascontiguousarray(widths, dtype=np.int32)
    stream = _vp(torch.cuda.current_stream().cuda_stream)
    program.current_arena = arena
    _after_calls(program, program._L.me_runner_static(program.handle, _vp(arena.data_ptr()), arena.numel(), _vp(index.data_ptr()),
                                                      bucket, _vp(w.ctypes.data), len(w), max_ctx, least_live,
                                                      _vp(None if drawn is None else drawn.data_ptr()), int(fed), stream,
                                                      _vp(out.ctypes.data)))
    logits = view_in(arena, int(out[0]), (bucket, program.vocab), torch.float32)
    tokens = drawn if drawn is not None else view_in(arena, int(out[2]), (bucket,), torch.int32)
    return logits, tokens
