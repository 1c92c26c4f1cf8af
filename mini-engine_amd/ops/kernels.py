"""Python entry points of the HIP kernels: each checks on the host that the operands have the
shapes, dtypes and layout the kernel and its grid assume, then launches on torch's current stream.

Tensors are torch CUDA tensors (torch is the allocator and the stream owner here); the kernels get
raw device pointers. Nothing in this module computes anything on the CPU or through a torch op,
except :func:`linear`, which hands large bfloat16 products to the GEMM library as the reference
hands every projection to one (``src/mini_engine/model.py:97-100, 125-127, 168``).
"""

from __future__ import annotations

import ctypes

import numpy as np
import torch

from .library import check, lib

_F32, _BF16 = 0, 1
_vp = ctypes.c_void_p
_i = int  # a Python int goes to a C int as it is; wrapping it in a ctypes object only costs time
_f = ctypes.c_float


def _code(dtype: torch.dtype) -> int:
    if dtype is torch.float32:
        return _F32
    if dtype is torch.bfloat16:
        return _BF16
    raise TypeError(f"kernels take float32 or bfloat16 activations, got {dtype}")


def _p(t: torch.Tensor | None) -> _vp:
    return _vp(None) if t is None else _vp(t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> _vp:
    """torch's current stream of the current device, as the handle the entry points take. An eager step
    makes a few hundred of these calls: the raw getter, where this torch has it, costs a tenth of
    building a Stream object."""
    if _raw_stream is not None:
        return _vp(_raw_stream(torch.cuda.current_device()))
    return _vp(torch.cuda.current_stream().cuda_stream)


def _want(t: torch.Tensor, name: str, dtype: torch.dtype | None = None, shape: tuple | None = None) -> None:
    """Host-side check of an operand: on the GPU, contiguous, of the wanted dtype and shape (None in the
    shape: any size). What the kernels index with is checked here, before anything is launched."""
    if not (t.is_cuda and t.is_contiguous()):
        raise ValueError(f"{name} must be a contiguous tensor on the GPU")
    if dtype is not None and t.dtype is not dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if shape is not None and t.shape != shape:  # equal tuples: the usual case, one comparison
        got = t.shape
        ok = len(got) == len(shape)
        if ok:
            for s, g in zip(shape, got):
                if s is not None and s != g:
                    ok = False
                    break
        if not ok:
            raise ValueError(f"{name} must have shape {list(shape)}, got {list(got)}")


# ------------------------------------------------------------------------------------ row-wise ops


def embed(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor | None = None, multiplier: float = 1.0) -> torch.Tensor:
    """``out[t] = float32(table[ids[t]]) * multiplier``; ids int32 [T], table [V, H]."""
    _want(ids, "ids", torch.int32)
    _want(table, "table", None, (None, None))
    t, (v, h) = ids.numel(), table.shape
    if out is None:
        out = torch.empty((t, h), dtype=torch.float32, device=table.device)
    _want(out, "out", torch.float32, (t, h))
    check(lib().me_embed(_p(out), _p(table), _p(ids), _i(t), _i(h), _i(v), _f(multiplier), _i(_code(table.dtype)), _stream()))
    return out


def probe_read(buf: torch.Tensor, out: torch.Tensor) -> None:
    """Launch the kernel that streams ``buf`` (a multiple of 16 bytes) once; ``out`` is one int32 word
    it may write. For measuring the memory rate a kernel reaches on this GPU."""
    nbytes = buf.numel() * buf.element_size()
    _want(out, "out", torch.int32)
    check(lib().me_probe_read(_p(buf), ctypes.c_longlong(nbytes), _p(out), _stream()))


def probe_mfma(blocks: int, iterations: int, out: torch.Tensor) -> float:
    """Launch the kernel that issues bfloat16 16x16x32 matrix-core products from registers; returns
    the floating-point operations of the launch. ``out`` is one float32 word it may write."""
    _want(out, "out", torch.float32)
    check(lib().me_probe_mfma(_i(blocks), _i(iterations), _p(out), _stream()))
    return blocks * 4 * 4 * iterations * 2.0 * 16 * 16 * 32


def scale_(x: torch.Tensor, factor: float) -> torch.Tensor:
    """``x *= factor`` in place, float32 of any shape."""
    _want(x, "x", torch.float32)
    check(lib().me_scale_f32(_p(x), _f(factor), ctypes.c_longlong(x.numel()), _stream()))
    return x


class PartialSums:
    """A product that still is a sum: float32 ``parts`` [S, T, D], partial products over S runs of k.
    It stands where a delta of the residual stream stands; :func:`add_rmsnorm` adds the parts up, in the
    order of the runs, as it adds the delta."""

    def __init__(self, parts: torch.Tensor):
        self.parts = parts

    @property
    def shape(self):
        return self.parts.shape[1:]

    def to_tensor(self, dtype: torch.dtype) -> torch.Tensor:
        return self.parts.sum(0).to(dtype)


def add_rmsnorm(
    x: torch.Tensor,
    delta: "torch.Tensor | PartialSums | None",
    weight: torch.Tensor,
    eps: float,
    dtype: torch.dtype,
    out: torch.Tensor | None = None,
    rows: torch.Tensor | None = None,
    write_x: bool = True,
) -> torch.Tensor:
    """Residual add then RMSNorm. ``x`` float32 [T, D] is the residual stream (updated in place when
    ``write_x``), ``delta`` [T, D] in ``dtype``, :class:`PartialSums` or None, ``weight`` float32 [D]. With ``rows`` (int32
    [R]) only those rows are read and the result is [R, D]. Returns the normed rows in ``dtype``."""
    _want(x, "x", torch.float32, (None, None))
    t, d = x.shape
    _want(weight, "weight", torch.float32, (d,))
    parts = None
    if isinstance(delta, PartialSums):
        parts, delta = delta.parts, None
        _want(parts, "partial sums", torch.float32, (None, t, d))
    elif delta is not None:
        _want(delta, "delta", dtype, (t, d))
    n = t
    if rows is not None:
        _want(rows, "rows", torch.int32)
        n = rows.numel()
    if out is None:
        out = torch.empty((n, d), dtype=dtype, device=x.device)
    _want(out, "out", dtype, (n, d))
    check(lib().me_add_rmsnorm(_p(x), _p(delta), _p(parts), _i(0 if parts is None else parts.shape[0]),
                               ctypes.c_longlong(0 if parts is None else t * d), _p(weight), _p(out), _p(rows), _i(n),
                               _i(d), _f(eps), _i(1 if write_x else 0), _i(_code(dtype)), _stream()))
    return out


def residual_add(x: torch.Tensor, delta: "torch.Tensor | PartialSums") -> torch.Tensor:
    """``x += delta`` in place for the float32 residual stream [T, D] and a delta in the compute dtype
    (or partial sums): the add alone, for a norm that runs as a part of its own."""
    _want(x, "x", torch.float32, (None, None))
    t, d = x.shape
    parts = None
    if isinstance(delta, PartialSums):
        parts, delta = delta.parts, None
        _want(parts, "partial sums", torch.float32, (None, t, d))
    else:
        if delta.dtype not in (torch.float32, torch.bfloat16):
            raise TypeError(f"delta: float32 or bfloat16 expected, got {delta.dtype}")
        _want(delta, "delta", delta.dtype, (t, d))
    check(lib().me_residual_add(_p(x), _p(delta), _p(parts), _i(0 if parts is None else parts.shape[0]),
                                ctypes.c_longlong(0 if parts is None else t * d), _i(t), _i(d),
                                _i(_code(torch.float32 if delta is None else delta.dtype)), _stream()))
    return x


def rmsnorm(inp: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor | None = None) -> torch.Tensor:
    """RMSNorm over the last dim of ``inp`` [..., D]; weight float32 [D]."""
    _want(inp, "inp")
    d = inp.shape[-1]
    _want(weight, "weight", torch.float32, (d,))
    if out is None:
        out = torch.empty_like(inp)
    _want(out, "out", inp.dtype, tuple(inp.shape))
    n = inp.numel() // d if d else 0
    check(lib().me_rmsnorm(_p(inp), _p(weight), _p(out), _i(n), _i(d), _f(eps), _i(_code(inp.dtype)), _stream()))
    return out


GATE_ACTIVATIONS = {"silu": 1, "gelu_tanh": 2}  # the codes of the kernels' `gated` arguments (MeGate in csrc/common.h)


def gate_code(gated) -> int:
    """0 for a product that is not gated; else the code of the gate's activation. ``True`` means silu."""
    if not gated:
        return 0
    if gated is True:
        return GATE_ACTIVATIONS["silu"]
    if gated not in GATE_ACTIVATIONS:
        raise ValueError(f"unknown gate activation {gated!r}; known: {sorted(GATE_ACTIVATIONS)}")
    return GATE_ACTIVATIONS[gated]


def swiglu(gate_up: torch.Tensor, out: torch.Tensor | None = None, activation: str = "silu") -> torch.Tensor:
    """``act(gate_up[:, :I]) * gate_up[:, I:]`` for gate_up [T, 2I]; ``activation`` is "silu" or "gelu_tanh"."""
    _want(gate_up, "gate_up", None, (None, None))
    t, two_i = gate_up.shape
    if two_i % 2:
        raise ValueError(f"gate_up must have an even number of columns, got {two_i}")
    inter = two_i // 2
    if out is None:
        out = torch.empty((t, inter), dtype=gate_up.dtype, device=gate_up.device)
    _want(out, "out", gate_up.dtype, (t, inter))
    check(lib().me_swiglu(_p(gate_up), _p(out), _i(t), _i(inter), _i(gate_code(activation)), _i(_code(gate_up.dtype)), _stream()))
    return out


# ------------------------------------------------------------------------------------- attention


def _check_cache(k_cache, v_cache, dtype, nkv, d, bs):
    _want(k_cache, "k_cache", dtype, (None, nkv, bs, d))
    _want(v_cache, "v_cache", dtype, (k_cache.shape[0], nkv, d, bs))


def _check_step_index(positions, token_item, block_table, t):
    _want(positions, "positions", torch.int32, (t,))
    _want(token_item, "token_item", torch.int32, (t,))
    _want(block_table, "block_table", torch.int32, (None, None))


def rope_table(inv_freq: torch.Tensor, num_positions: int) -> torch.Tensor:
    """float32 [num_positions, 2, rotary_dim / 2]: cos and sin of ``position * inv_freq[j]``."""
    _want(inv_freq, "inv_freq", torch.float32, (None,))
    half = inv_freq.numel()
    table = torch.empty((num_positions, 2, half), dtype=torch.float32, device=inv_freq.device)
    check(lib().me_rope_table(_p(table), _p(inv_freq), _i(half), _i(num_positions), _stream()))
    return table


def qk_norm_rope_scatter(
    qkv: torch.Tensor,
    q_weight: torch.Tensor | None,
    k_weight: torch.Tensor | None,
    rope: torch.Tensor | None,
    positions: torch.Tensor,
    token_item: torch.Tensor,
    block_table: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    num_heads: int,
    num_kv_heads: int,
    head_dim: int,
    eps: float,
    write_kv: bool = True,
    q_out: torch.Tensor | None = None,
    item_start: torch.Tensor | None = None,
    starts: list[int] | None = None,
    qlens: list[int] | None = None,
) -> torch.Tensor:
    """Per-head q/k RMSNorm (when weights are given), rotary encoding (when ``rope``, the table of
    :func:`rope_table`, is given; it must cover every position of the step), and the write of keys
    and values into their pages.

    qkv [T, (nh + 2 nkv) d] (or [T, nh d] with ``write_kv`` off: q only); k_cache [pages, nkv, bs, d]; v_cache [pages, nkv, d, bs];
    block_table int32 [items, width]. Returns q [T, nh, d].

    With ``item_start`` (int32 [items + 1] on the device) and the items' first positions and lengths
    on the host, steps with many tokens write the values a page segment at a time (a transposed
    tile) instead of element by element."""
    nh, nkv, d = num_heads, num_kv_heads, head_dim
    _want(qkv, "qkv", None, (None, ((nh + 2 * nkv) if write_kv else nh) * d))
    t, dtype = qkv.shape[0], qkv.dtype
    _check_step_index(positions, token_item, block_table, t)
    bs = k_cache.shape[2]
    _check_cache(k_cache, v_cache, dtype, nkv, d, bs)
    for w, name in ((q_weight, "q_weight"), (k_weight, "k_weight")):
        if w is not None:
            _want(w, name, torch.float32, (d,))
    rd = 0
    if rope is not None:
        _want(rope, "rope", torch.float32, (None, 2, None))
        rd = 2 * rope.shape[2]
    if q_out is None:
        q_out = torch.empty((t, nh, d), dtype=dtype, device=qkv.device)
    _want(q_out, "q_out", dtype, (t, nh, d))
    segments, items = 0, 0
    if write_kv and item_start is not None and starts is not None and qlens is not None and t >= 64:
        items = len(qlens)
        if sum(qlens) != t or len(starts) != items:
            raise ValueError("item lengths do not add up to the number of tokens")
        _want(item_start, "item_start", torch.int32, (items + 1,))
        segments = sum((p0 + n - 1) // 16 - p0 // 16 + 1 for p0, n in zip(starts, qlens))
    check(lib().me_qk_norm_rope_scatter(
        _p(qkv), _p(q_weight), _p(k_weight), _p(rope), _p(positions), _p(token_item), _p(block_table),
        _i(block_table.shape[1]), _p(q_out), _p(k_cache), _p(v_cache), _i(t), _i(nh), _i(nkv), _i(d), _i(rd),
        _i(bs), _f(eps), _i(1 if write_kv else 0), _i(_code(dtype)), _p(item_start if segments else None), _i(items),
        _i(segments), _stream()))
    return q_out


def attention_general(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    positions: torch.Tensor,
    token_item: torch.Tensor,
    block_table: torch.Tensor,
    scale: float,
    window: int = 0,
    out: torch.Tensor | None = None,
    shared_tiles: bool = True,
) -> torch.Tensor:
    """Causal grouped-query attention of q [T, nh, d] over the paged cache; returns [T, nh * d]. float32 steps with
    two and more tokens per row of the block table go to a kernel whose blocks share the tiles of keys and values among
    their tokens (``shared_tiles=False``: the kernel with a wave per token and head for every step; the same bits)."""
    _want(q, "q", None, (None, None, None))
    t, nh, d = q.shape
    nkv, bs = k_cache.shape[1], k_cache.shape[2]
    _check_cache(k_cache, v_cache, q.dtype, nkv, d, bs)
    _check_step_index(positions, token_item, block_table, t)
    if out is None:
        out = torch.empty((t, nh * d), dtype=q.dtype, device=q.device)
    _want(out, "out", q.dtype, (t, nh * d))
    check(lib().me_attention_general(
        _p(q), _p(k_cache), _p(v_cache), _p(positions), _p(token_item), _p(block_table), _i(block_table.shape[1]),
        _p(out), _i(t), _i(nh), _i(nkv), _i(d), _i(bs), _i(window), _f(scale), _i(_code(q.dtype)),
        _i(block_table.shape[0] if shared_tiles else 0), _stream()))
    return out


# ------------------------------------------------------------------------------ matrix products

def gemm_f32(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """float32 ``x @ weight.T`` on the matrix cores' float32 instruction (float32 operands, products and sums): an
    element's products are added two k at a time in ascending k, whatever the number of rows."""
    _want(x, "x", torch.float32, (None, None))
    m, k = x.shape
    _want(weight, "weight", torch.float32, (None, k))
    n = weight.shape[0]
    if out is None:
        out = torch.empty((m, n), dtype=torch.float32, device=x.device)
    _want(out, "out", torch.float32, (m, n))
    check(lib().me_gemm_f32(_p(x), _p(weight), _p(out), _i(m), _i(n), _i(k), _stream()))
    return out


class NormedInput:
    """``rmsnorm(x + delta) * weight`` not yet computed: what a block hands to a part that can take
    the residual add and the norm as the prologue of its first matrix product.

    ``x`` is the float32 residual stream [T, D], ``delta`` the pending addition in the compute dtype
    (or None), ``spare`` a second float32 buffer of x's shape. Whoever consumes the input performs the
    residual add; afterwards :attr:`residual` is the buffer that holds ``x + delta``."""

    def __init__(self, x: torch.Tensor, delta: torch.Tensor | None, weight: torch.Tensor, eps: float,
                 dtype: torch.dtype, spare: torch.Tensor | None):
        self.x, self.delta, self.weight, self.eps, self.dtype, self.spare = x, delta, weight, eps, dtype, spare
        self.residual: torch.Tensor | None = None
        self._tensor: torch.Tensor | None = None

    @property
    def shape(self):
        return self.x.shape

    def materialize(self) -> torch.Tensor:
        """Run the add-and-norm kernel (once) and return the normed activations."""
        if self._tensor is None:
            if self.residual is not None:  # the add already happened in a fused product
                self._tensor = add_rmsnorm(self.residual, None, self.weight, self.eps, self.dtype)
            else:
                self._tensor = add_rmsnorm(self.x, self.delta, self.weight, self.eps, self.dtype)
                self.residual = self.x
        return self._tensor

    def fusion(self, weight: torch.Tensor) -> int:
        """How add, norm and the product with ``weight`` are launched: :data:`NORM_ALONE`, :data:`NORM_IN_STREAM` (one
        launch of the weight-streaming kernel: a row or two, whatever the delta is) or :data:`NORM_IN_SMALL` (the small
        matrix-core kernel's prologue: decode-sized steps whose delta is a tensor). The rule is the native step
        program's (``csrc/host/choice.cpp``); what is asked here on top is that the add has not happened yet and that
        a sum has a second buffer to go to."""
        if (self.dtype is not torch.bfloat16 or weight.dtype is not torch.bfloat16 or self._tensor is not None
                or self.residual is not None or (self.delta is not None and self.spare is None)):
            return NORM_ALONE
        rows, k = self.x.shape
        pending = 0 if self.delta is None else 2 if isinstance(self.delta, PartialSums) else 1
        return int(lib().me_norm_fusion_choice(_i(_code(self.dtype)), _i(rows), _i(weight.shape[0]), _i(k), _i(pending),
                                               _i(compute_units(weight.device)), _i(int(weight.data_ptr() % 16 == 0))))


NORM_ALONE, NORM_IN_STREAM, NORM_IN_SMALL = 0, 1, 2  # csrc/host/choice.h: NormFusion
PRODUCT_F32, PRODUCT_SMALL, PRODUCT_STREAM, PRODUCT_TILED, PRODUCT_LIBRARY = range(5)  # csrc/host/choice.h: ProductKernel
ROLE_PLAIN, ROLE_DELTA, ROLE_HEAD, ROLE_DELTA_INTO = range(4)  # csrc/host/choice.h: ProductRole


def product_choice(dtype: torch.dtype, role: int, rows: int, rows_of_w: int, k: int, gated: bool, out_dtype: torch.dtype,
                   units: int, aligned: bool = True) -> tuple[int, int, bool, bool]:
    """Which kernel serves a product: (kernel, runs of k, the result is float32 partial sums, the gate is a kernel of
    its own behind the product). The one rule of the tree, in ``csrc/host/choice.cpp``; no GPU is touched."""
    out = (ctypes.c_int * 5)()
    lib().me_product_choice(_i(_code(dtype)), _i(role), _i(rows), _i(rows_of_w), _i(k), _i(int(bool(gated))), _i(_code(out_dtype)),
                            _i(units), _i(int(aligned)), out)
    return int(out[0]), int(out[1]), bool(out[2]), bool(out[3])


def delta_choice(rows: int, rows_of_w: int, k: int, units: int, aligned: bool = True) -> tuple[int, int, bool, bool]:
    """How the step program takes a bfloat16 product that is a delta of the float32 residual stream and may be added
    into it: (kernel, runs of k, the result is float32 partial sums, the kernel adds its product into the stream
    itself). Exactly one of the last two holds."""
    out = (ctypes.c_int * 5)()
    lib().me_product_choice(_i(_code(torch.bfloat16)), _i(ROLE_DELTA_INTO), _i(rows), _i(rows_of_w), _i(k), _i(0),
                            _i(_code(torch.bfloat16)), _i(units), _i(int(aligned)), out)
    return int(out[0]), int(out[1]), bool(out[2]), bool(out[4])


def carried_norm_choice(dtype: torch.dtype, rows: int, n: int, k: int, next_rows_of_w: int, next_gated: bool, units: int,
                        aligned: bool = True) -> bool:
    """Whether the step program lets a delta of the residual stream (``rows`` x ``n`` = hidden, over ``k``) add itself to
    the stream and leave the RMS norm behind it to the product after the norm (``next_rows_of_w`` rows of hidden): the
    rule of ``csrc/host/choice.cpp``; no GPU is touched."""
    return bool(lib().me_carried_norm_choice(_i(_code(dtype)), _i(rows), _i(n), _i(k), _i(next_rows_of_w), _i(int(bool(next_gated))),
                                             _i(units), _i(int(aligned))))


def split_sum_choice(dtype: torch.dtype, rows: int, n: int, aligned: bool = True) -> bool:
    """Whether the step program lets the output projection (``n`` = hidden columns) behind a decode attention of ``rows``
    items add up the attention's splits itself (:func:`attention_out_product_bf16`): the rule of ``csrc/host/choice.cpp``;
    no GPU is touched."""
    return bool(lib().me_split_sum_choice(_i(_code(dtype)), _i(rows), _i(n), _i(int(aligned))))


STREAM_MAX_ROWS = 256  # the weight-streaming product deals more than 64 rows to groups of blocks
SMALL_MAX_ROWS = 64  # what the small matrix-core kernel accepts


def compute_units(device=None) -> int:
    return torch.cuda.get_device_properties(device or torch.cuda.current_device()).multi_processor_count


def stream_splits(n: int, k: int, device=None, rows: int = 1, units: int | None = None) -> int:
    """Into how many runs of k :func:`gemm_bf16_stream` cuts a product of ``rows`` rows whose result may stay
    partial sums."""
    return int(lib().me_gemm_bf16_stream_splits(_i(rows), _i(n), _i(k), _i(units if units is not None else compute_units(device))))


def stream_plan(rows: int, n: int, k: int, gated: bool = False, k_splits: int = 1, device=None,
                units: int | None = None) -> tuple[int, int, int]:
    """What :func:`gemm_bf16_stream` launches for a product: (groups of 16 columns per block, runs of k, blocks along
    the columns). The columns are dealt to the blocks in fours, as evenly as they go. ``units``: plan for this many
    compute units instead of the device's (a host-side question; no GPU is touched)."""
    out = (ctypes.c_int * 3)()
    lib().me_gemm_bf16_stream_plan(_i(rows), _i(n), _i(k), _i(int(bool(gated))), _i(k_splits),
                                   _i(units if units is not None else compute_units(device)), out)
    return int(out[0]), int(out[1]), int(out[2])


def gemm_bf16_stream(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16, swiglu: bool = False,
                     out: torch.Tensor | None = None, k_splits: int = 1) -> torch.Tensor:
    """bfloat16 ``x @ weight.T`` for at most 256 rows (64 a block; more rows go to groups of blocks) and weights
    large enough that streaming them is the kernel's time: x is staged in LDS once per block of columns, the weight goes straight to the matrix
    cores. ``swiglu`` and ``k_splits`` as in :func:`gemm_bf16_small` (``k_splits`` as :func:`stream_splits`
    gives it, or 1)."""
    _want(x, "x", torch.bfloat16, (None, None))
    m, k = x.shape
    _want(weight, "weight", torch.bfloat16, (None, k))
    n = weight.shape[0]
    if swiglu:
        if n % 2:
            raise ValueError(f"a gate/up weight needs an even number of rows, got {n}")
        n //= 2
    if m > STREAM_MAX_ROWS:
        raise ValueError(f"gemm_bf16_stream takes at most {STREAM_MAX_ROWS} rows, got {m}")
    shape = (k_splits, m, n) if k_splits > 1 else (m, n)
    if out is None:
        out = torch.empty(shape, dtype=out_dtype, device=weight.device)
    _want(out, "out", out_dtype, shape)
    check(lib().me_gemm_bf16_stream(_p(x), _p(weight), _p(out), _i(m), _i(n), _i(k), _i(gate_code(swiglu)),
                                    _i(_code(out_dtype)), _i(k_splits), _i(compute_units(x.device)), _stream()))
    return out


def stream_carry_blocks(rows: int, n: int, k: int, device=None, units: int | None = None) -> int:
    """Partial sums of squares a row that :func:`gemm_bf16_stream_carry` leaves for a product of these sizes."""
    return int(lib().me_gemm_bf16_stream_carry_blocks(_i(rows), _i(n), _i(k), _i(units if units is not None else compute_units(device))))


def gemm_bf16_stream_carry(a: torch.Tensor, weight: torch.Tensor, x: torch.Tensor, norm_weight: torch.Tensor
                           ) -> tuple[torch.Tensor, torch.Tensor]:
    """A product that is a delta of the float32 residual stream, added to the stream in its epilogue:
    ``x += a @ weight.T`` in place; returns ``h = bf16(x * norm_weight)``, not yet divided by the rows' root mean
    squares, and ``ss`` float32 ``[rows, blocks]``, partial sums of squares of the rows of the new ``x``. The product
    behind the norm divides (:func:`gemm_bf16_scaled`)."""
    _want(a, "a", torch.bfloat16, (None, None))
    m, k = a.shape
    _want(weight, "weight", torch.bfloat16, (None, k))
    n = weight.shape[0]
    _want(x, "residual stream", torch.float32, (m, n))
    _want(norm_weight, "norm weight", torch.float32, (n,))
    if m > STREAM_MAX_ROWS:
        raise ValueError(f"gemm_bf16_stream_carry takes at most {STREAM_MAX_ROWS} rows, got {m}")
    blocks = stream_carry_blocks(m, n, k, a.device)
    h = torch.empty((m, n), dtype=torch.bfloat16, device=a.device)
    ss = torch.empty((m, blocks), dtype=torch.float32, device=a.device)
    check(lib().me_gemm_bf16_stream_carry(_p(a), _p(weight), _p(x), _p(h), _p(ss), _p(norm_weight), _i(m), _i(n), _i(k),
                                          _i(compute_units(a.device)), _stream()))
    return h, ss


def gemm_bf16_scaled(h: torch.Tensor, weight: torch.Tensor, ss: torch.Tensor, dim: int, eps: float, swiglu: bool = False,
                     out_dtype: torch.dtype = torch.bfloat16, kernel: str = "small") -> torch.Tensor:
    """``(h * rsqrt(ss.sum(1) / dim + eps)[:, None]) @ weight.T`` with the rows' scale applied to the product (before
    the gate): the product behind an RMS norm whose division :func:`gemm_bf16_stream_carry` left to it. ``kernel``:
    "small" (at most 64 rows) or "stream"."""
    _want(h, "h", torch.bfloat16, (None, None))
    m, k = h.shape
    _want(weight, "weight", torch.bfloat16, (None, k))
    n = weight.shape[0] // 2 if swiglu else weight.shape[0]
    _want(ss, "sums of squares", torch.float32, (m, None))
    out = torch.empty((m, n), dtype=out_dtype, device=h.device)
    if kernel == "small":
        check(lib().me_gemm_bf16_small_scaled(_p(h), _p(weight), _p(out), _i(m), _i(n), _i(k), _i(gate_code(swiglu)),
                                              _i(_code(out_dtype)), _p(ss), _i(ss.shape[1]), _i(dim), _f(eps), _stream()))
    elif kernel == "stream":
        check(lib().me_gemm_bf16_stream_scaled(_p(h), _p(weight), _p(out), _i(m), _i(n), _i(k), _i(gate_code(swiglu)),
                                               _i(_code(out_dtype)), _i(compute_units(h.device)), _p(ss), _i(ss.shape[1]),
                                               _i(dim), _f(eps), _stream()))
    else:
        raise ValueError(f"unknown kernel {kernel!r}")
    return out


def stream_norm_fits(rows: int, k: int) -> bool:
    """Whether :func:`gemm_bf16_stream_norm` takes this many rows of this length."""
    return bool(lib().me_gemm_bf16_stream_norm_fits(_i(rows), _i(k)))


def gemm_bf16_stream_norm(x: "NormedInput", weight: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16,
                          swiglu: "bool | str" = False, out: torch.Tensor | None = None) -> torch.Tensor:
    """``rmsnorm(x.x + x.delta) * x.weight @ weight.T`` for a row or a few in one launch of the weight-streaming
    kernel: every block adds and norms the rows itself while its first weights are on their way. ``x.delta`` is a
    bfloat16 tensor, :class:`PartialSums` or None; with a delta the sum goes to ``x.spare``, which becomes
    ``x.residual``."""
    m, k = x.shape
    _want(weight, "weight", torch.bfloat16, (None, k))
    n = weight.shape[0]
    if swiglu:
        if n % 2:
            raise ValueError(f"a gate/up weight needs an even number of rows, got {n}")
        n //= 2
    if not stream_norm_fits(m, k):
        raise ValueError(f"gemm_bf16_stream_norm does not take {m} rows of {k}")
    _want(x.x, "x", torch.float32, (m, k))
    _want(x.weight, "norm weight", torch.float32, (k,))
    delta = parts = None
    num_parts = stride = 0
    if isinstance(x.delta, PartialSums):
        parts = x.delta.parts
        _want(parts, "partial sums", torch.float32, (None, m, k))
        num_parts, stride = parts.shape[0], m * k
    elif x.delta is not None:
        delta = x.delta
        _want(delta, "delta", torch.bfloat16, (m, k))
    x_out = None
    if x.delta is not None:
        if x.spare is None:
            raise ValueError("the sum of the residual stream and its delta needs a second buffer")
        x_out = x.spare
        _want(x_out, "spare", torch.float32, (m, k))
        if x_out.data_ptr() == x.x.data_ptr():
            raise ValueError("the second buffer must not be the residual stream itself")
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=weight.device)
    _want(out, "out", out_dtype, (m, n))
    check(lib().me_gemm_bf16_stream_norm(_p(x.x), _p(delta), _p(parts), _i(num_parts), ctypes.c_longlong(stride), _p(x.weight),
                                         _f(x.eps), _p(x_out), _p(weight), _p(out), _i(m), _i(n), _i(k), _i(gate_code(swiglu)),
                                         _i(_code(out_dtype)), _i(compute_units(weight.device)), _stream()))
    x.residual = x_out if x_out is not None else x.x
    return out


def gemm_bf16_small(x, weight: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16, swiglu: bool = False,
                    out: torch.Tensor | None = None, k_splits: int = 1) -> torch.Tensor:
    """bfloat16 ``x @ weight.T`` for at most 64 rows on the matrix cores, float32 accumulation.

    ``x`` is a bfloat16 tensor [M, K] or a :class:`NormedInput` (then the residual add and the RMSNorm
    are the product's prologue). With ``swiglu`` the weight holds gate rows then up rows, [2N, K], and
    the result is ``silu(gate) * up`` [M, N]. With ``k_splits`` > 1 (plain float32 products) the result
    is [k_splits, M, N]: partial sums over runs of k, each by blocks of its own."""
    normed = isinstance(x, NormedInput)
    m, k = x.shape
    _want(weight, "weight", torch.bfloat16, (None, k))
    n = weight.shape[0]
    if swiglu:
        if n % 2:
            raise ValueError(f"a gate/up weight needs an even number of rows, got {n}")
        n //= 2
    if m > SMALL_MAX_ROWS:
        raise ValueError(f"gemm_bf16_small takes at most {SMALL_MAX_ROWS} rows, got {m}")
    if k_splits > 1:
        if normed or swiglu or out_dtype is not torch.float32:
            raise ValueError("partial sums over splits of k are plain float32 products")
        if out is None:
            out = torch.empty((k_splits, m, n), dtype=torch.float32, device=weight.device)
        _want(out, "out", torch.float32, (k_splits, m, n))
    else:
        if out is None:
            out = torch.empty((m, n), dtype=out_dtype, device=weight.device)
        _want(out, "out", out_dtype, (m, n))
    if normed:
        _want(x.x, "residual stream", torch.float32, (m, k))
        _want(x.weight, "norm weight", torch.float32, (k,))
        x_out = None
        if x.delta is not None:
            _want(x.delta, "delta", torch.bfloat16, (m, k))
            _want(x.spare, "spare residual buffer", torch.float32, (m, k))
            if x.spare.data_ptr() == x.x.data_ptr():
                raise ValueError("the spare residual buffer must not alias the residual stream")
            x_out = x.spare
        check(lib().me_gemm_bf16_small(_p(None), _p(x.x), _p(x.delta), _p(x.weight), _f(x.eps), _p(x_out), _p(weight),
                                       _p(out), _i(m), _i(n), _i(k), _i(1), _i(gate_code(swiglu)),
                                       _i(_code(out_dtype)), _i(1), _stream()))
        x.residual = x.x if x.delta is None else x.spare
    else:
        _want(x, "x", torch.bfloat16, (m, k))
        check(lib().me_gemm_bf16_small(_p(x), _p(None), _p(None), _p(None), _f(0.0), _p(None), _p(weight), _p(out),
                                       _i(m), _i(n), _i(k), _i(0), _i(gate_code(swiglu)), _i(_code(out_dtype)),
                                       _i(k_splits), _stream()))
    return out


def gemm_bf16_skinny(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16,
                     out: torch.Tensor | None = None) -> torch.Tensor:
    """The plain form of :func:`gemm_bf16_small` (no prologue, no epilogue)."""
    return gemm_bf16_small(x, weight, out_dtype, False, out)




def gemm_bf16_tiled(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16, swiglu: bool = False,
                    out: torch.Tensor | None = None, shape: int = 0) -> torch.Tensor:
    """bfloat16 ``x @ weight.T`` for any number of rows with LDS-tiled matrix-core blocks, float32
    accumulation; K must be a multiple of 64. With ``swiglu`` the weight holds gate rows then up rows,
    [2N, K], and the result is ``silu(gate) * up`` [M, N] in bfloat16, without the [M, 2N] product ever
    going to memory. ``shape`` names a block tile (0: the default)."""
    _want(x, "x", torch.bfloat16, (None, None))
    m, k = x.shape
    _want(weight, "weight", torch.bfloat16, (None, k))
    n = weight.shape[0]
    if swiglu:
        if n % 2:
            raise ValueError(f"a gate/up weight needs an even number of rows, got {n}")
        n //= 2
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=weight.device)
    _want(out, "out", out_dtype, (m, n))
    check(lib().me_gemm_bf16_tiled(_p(x), _p(weight), _p(out), _i(m), _i(n), _i(k), _i(gate_code(swiglu)),
                                   _i(_code(out_dtype)), _i(shape), _stream()))
    return out


def linear(x, weight: torch.Tensor, out_dtype: torch.dtype | None = None, gated: "bool | str" = False,
           as_delta: bool = False, head: bool = False):
    """``x @ weight.T`` for x [M, K], weight [N, K]; with ``gated`` (True or "silu", or "gelu_tanh") the
    weight is [2N, K] (gate rows, then up rows) and the result is ``act(gate) * up``. ``x`` may be a :class:`NormedInput`. With
    ``as_delta`` the caller says that the result only ever is the pending delta of the residual stream
    (what a mixer or a feed-forward returns): it may then come back as :class:`PartialSums`, which
    :func:`add_rmsnorm` adds up on the way. ``head``: the product gives the logits of the wanted rows.

    float32: always the deterministic float32 kernel (a true 32-bit product). bfloat16: the kernel that the native step
    program would take for the same sizes (:func:`product_choice`; the rule and its measurements are in
    ``csrc/host/choice.cpp``)."""
    activation = "silu" if gated is True else gated
    if isinstance(x, NormedInput):
        how = x.fusion(weight)
        if how == NORM_IN_STREAM:
            return gemm_bf16_stream_norm(x, weight, out_dtype or x.dtype, gated)
        if how == NORM_IN_SMALL:
            return gemm_bf16_small(x, weight, out_dtype or x.dtype, gated)
        x = x.materialize()
    out_dtype = out_dtype or x.dtype
    if x.dtype is torch.float32 and out_dtype is not torch.float32:
        raise TypeError("the float32 path keeps float32 results")
    role = ROLE_DELTA if as_delta and not gated else ROLE_HEAD if head else ROLE_PLAIN
    aligned = x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0
    kernel, runs, partial, gate_after = product_choice(x.dtype, role, x.shape[0], weight.shape[0], x.shape[1], bool(gated),
                                                       out_dtype, compute_units(x.device), aligned)
    epilogue = False if gate_after else gated
    inner = torch.float32 if partial else x.dtype if gate_after else out_dtype
    if kernel == PRODUCT_F32:
        y = gemm_f32(x, weight)
    elif kernel == PRODUCT_SMALL:
        y = gemm_bf16_small(x, weight, inner, epilogue)
    elif kernel == PRODUCT_STREAM:
        y = gemm_bf16_stream(x, weight, inner, epilogue, k_splits=runs)
    elif kernel == PRODUCT_TILED:
        y = gemm_bf16_tiled(x, weight, inner, epilogue)
    else:
        y = gemm_bf16_library(x, weight, inner)
    if partial:
        return PartialSums(y if runs > 1 else y.unsqueeze(0))
    return swiglu(y, activation=activation) if gate_after else y


def gemm_bf16_library(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16,
                      out: torch.Tensor | None = None) -> torch.Tensor:
    """bfloat16 ``x @ weight.T`` through the GEMM library with float32 accumulation, as bfloat16 or as
    float32 (logits, not rounded to bfloat16). The library is called directly (a third of the host time
    of a call through torch); where it has no algorithm for the sizes (widths that are no multiple of
    8), the kernels of this package stand in, as in the native step program."""
    _want(x, "x", torch.bfloat16, (None, None))
    m, k = x.shape
    _want(weight, "weight", torch.bfloat16, (None, k))
    n = weight.shape[0]
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    _want(out, "out", out_dtype, (m, n))
    check(lib().me_gemm_bf16_any(_p(x), _p(weight), _p(out), _i(m), _i(n), _i(k), _i(_code(out_dtype)), _stream()))
    return out


# -------------------------------------------------------------------------------------- sampling


def sample(logits: torch.Tensor, temperatures: torch.Tensor | None = None, keys: torch.Tensor | None = None,
           out: torch.Tensor | None = None) -> torch.Tensor:
    """One token per row of float32 logits [R, V]: argmax where the row's temperature is 0 (or no
    temperatures are given), else a draw from softmax(logits / temperature) keyed by ``keys``
    (int64 [R], any bit pattern)."""
    _want(logits, "logits", torch.float32, (None, None))
    r, v = logits.shape
    if temperatures is not None:
        _want(temperatures, "temperatures", torch.float32, (r,))
        if keys is None:
            raise ValueError("temperature sampling needs one key per row")
        _want(keys, "keys", torch.int64, (r,))
    if out is None:
        out = torch.empty((r,), dtype=torch.int32, device=logits.device)
    _want(out, "out", torch.int32, (r,))
    chunks = lib().me_sample_chunks(_i(v))
    workspace = torch.empty((r * chunks * 2,), dtype=torch.float32, device=logits.device)
    check(lib().me_sample(_p(logits), _i(r), _i(v), _p(temperatures), _p(keys if temperatures is not None else None),
                          _p(out), _p(workspace), _stream()))
    return out


# ------------------------------------------------------------- matrix-core attention (bfloat16)


def attention_mfma_supported(head_dim: int, block_size: int, group: int = 1) -> bool:
    """Whether the matrix-core attention kernels take this head size, page size and group size."""
    return bool(lib().me_attention_mfma_supported(_i(head_dim), _i(block_size))) and group <= 16


def decode_splits(items: int, kv_units: int, max_ctx: int, target_waves: int = 1024) -> tuple[int, int]:
    """(keys per split, number of splits) for the decode kernel: enough waves to fill the chip,
    splits of at least 64 keys, whole tiles of 16."""
    units = max(1, items * kv_units)
    splits = max(1, min(-(-target_waves // units), max(max_ctx, 64) // 64))
    split_keys = -(-max_ctx // splits)
    split_keys = -(-split_keys // 16) * 16
    return split_keys, -(-max_ctx // split_keys)


DECODE_WAVES = 1024  # waves that a decode attention launch aims at (four per compute unit of 256)


def _decode_split_plan(items: int, kv_units: int, max_ctx: int, live):
    """(split_keys, num_splits, live pointer, splits of a full step) for a decode launch. ``live`` is
    None or ``(count, least)``: a device int32 with the number of live items (the others are padding)
    and the fewest live items the launch will ever see; the grid is then laid out for ``least`` items,
    and the kernel takes as many of its splits as the live items need."""
    _, full = decode_splits(items, kv_units, max_ctx, DECODE_WAVES)
    if live is None or live[1] >= items:
        keys, splits = decode_splits(items, kv_units, max_ctx, DECODE_WAVES)
        return keys, splits, None, splits
    count, least = live
    _want(count, "live item count", torch.int32, (1,))
    keys, splits = decode_splits(max(1, least), kv_units, max_ctx, DECODE_WAVES)
    return keys, splits, count, min(full, splits)


def attention_decode_leaves_parts(items: int, num_heads: int, num_kv_heads: int, head_dim: int, num_splits: int) -> bool:
    """Whether a decode launch of these sizes leaves one partial result per split (which a second kernel, or
    :func:`attention_out_product_bf16` in its place, adds up): the launches that may be asked to ``leave_parts``."""
    return bool(lib().me_attention_decode_leaves_parts(_i(items), _i(num_heads), _i(num_kv_heads), _i(head_dim),
                                                       _i(num_splits)))


def attention_decode_bf16(q, k_cache, v_cache, item_ctx, block_table, scale: float, window: int, max_ctx: int,
                          out: torch.Tensor | None = None, live=None, step_flags: torch.Tensor | None = None,
                          leave_parts: bool = False):
    """Attention of one new token per item over its cached keys: q [items, nh, d] bfloat16,
    item_ctx int32 [items] (keys per item, the new one included, each <= max_ctx). ``live``: see
    :func:`_decode_split_plan`. ``step_flags``: None, or a device int32 whose bit 0 says that the items share
    pages (a large launch then loads keys and values with ordinary loads instead of non-temporal ones).
    ``leave_parts``: the splits are not added up; the result is ``(part_o, part_ml, num_splits)`` for
    :func:`attention_out_product_bf16` (only where :func:`attention_decode_leaves_parts` says so)."""
    _want(q, "q", torch.bfloat16, (None, None, None))
    items, nh, d = q.shape
    nkv, bs = k_cache.shape[1], k_cache.shape[2]
    _check_cache(k_cache, v_cache, torch.bfloat16, nkv, d, bs)
    _want(item_ctx, "item_ctx", torch.int32, (items,))
    _want(block_table, "block_table", torch.int32, (items, None))
    if block_table.shape[1] * bs < max_ctx:
        raise ValueError(f"block table of {block_table.shape[1]} pages cannot hold {max_ctx} keys")
    chunks = -(-(nh // nkv) // 16)
    split_keys, num_splits, live_count, full_splits = _decode_split_plan(items, nkv * chunks, max_ctx, live)
    part_o = torch.empty((items * nh * num_splits * d,), dtype=torch.float32, device=q.device)
    part_ml = torch.empty((items * nh * num_splits * 2,), dtype=torch.float32, device=q.device)
    if leave_parts:
        out = None
    else:
        if out is None:
            out = torch.empty((items, nh * d), dtype=torch.bfloat16, device=q.device)
        _want(out, "out", torch.bfloat16, (items, nh * d))
    check(lib().me_attention_decode_bf16(
        _p(q), _p(k_cache), _p(v_cache), _p(item_ctx), _p(block_table), _i(block_table.shape[1]), _p(out),
        _p(part_o), _p(part_ml), _i(items), _i(nh), _i(nkv), _i(d), _i(bs), _i(window), _f(scale), _i(split_keys),
        _i(num_splits), _i(max_ctx), _p(live_count), _i(full_splits), _i(DECODE_WAVES), _p(step_flags), _stream()))
    return (part_o, part_ml, num_splits) if leave_parts else out


def attention_decode_fused_supported(head_dim: int, block_size: int, rotary_dim: int, group: int) -> bool:
    """Whether the decode kernel can take q/k norm, rotary encoding and the page write as its prologue."""
    return bool(lib().me_attention_decode_fused_supported(_i(head_dim), _i(block_size), _i(rotary_dim), _i(group)))


def attention_decode_fused_bf16(qkv, q_weight, k_weight, rope, eps: float, write_kv: bool, k_cache, v_cache, item_ctx,
                                block_table, num_heads: int, scale: float, window: int, max_ctx: int,
                                out: torch.Tensor | None = None, live=None,
                                step_flags: torch.Tensor | None = None, leave_parts: bool = False):
    """One new token per item, from the raw q/k/v projection: what :func:`qk_norm_rope_scatter` followed
    by :func:`attention_decode_bf16` compute, in one launch. qkv [items, (nh + 2 nkv) d] bfloat16
    (or [items, nh d] with ``write_kv`` off). ``live``: see :func:`_decode_split_plan`; ``step_flags`` and
    ``leave_parts`` as in :func:`attention_decode_bf16`."""
    nkv, bs, d = k_cache.shape[1], k_cache.shape[2], k_cache.shape[3]
    nh = num_heads
    _want(qkv, "qkv", torch.bfloat16, (None, ((nh + 2 * nkv) if write_kv else nh) * d))
    items = qkv.shape[0]
    _check_cache(k_cache, v_cache, torch.bfloat16, nkv, d, bs)
    _want(item_ctx, "item_ctx", torch.int32, (items,))
    _want(block_table, "block_table", torch.int32, (items, None))
    if block_table.shape[1] * bs < max_ctx:
        raise ValueError(f"block table of {block_table.shape[1]} pages cannot hold {max_ctx} keys")
    for w, name in ((q_weight, "q_weight"), (k_weight, "k_weight")):
        if w is not None:
            _want(w, name, torch.float32, (d,))
    rd = 0
    if rope is not None:
        _want(rope, "rope", torch.float32, (None, 2, None))
        rd = 2 * rope.shape[2]
        if rope.shape[0] < max_ctx:
            raise ValueError(f"the rotary table covers {rope.shape[0]} positions, the step may reach {max_ctx}")
    chunks = -(-(nh // nkv) // 16)
    split_keys, num_splits, live_count, full_splits = _decode_split_plan(items, nkv * chunks, max_ctx, live)
    part_o = torch.empty((items * nh * num_splits * d,), dtype=torch.float32, device=qkv.device)
    part_ml = torch.empty((items * nh * num_splits * 2,), dtype=torch.float32, device=qkv.device)
    if leave_parts:
        out = None
    else:
        if out is None:
            out = torch.empty((items, nh * d), dtype=torch.bfloat16, device=qkv.device)
        _want(out, "out", torch.bfloat16, (items, nh * d))
    check(lib().me_attention_decode_fused_bf16(
        _p(qkv), _p(q_weight), _p(k_weight), _p(rope), _i(rd), _f(eps), _i(1 if write_kv else 0), _p(k_cache),
        _p(v_cache), _p(item_ctx), _p(block_table), _i(block_table.shape[1]), _p(out), _p(part_o), _p(part_ml),
        _i(items), _i(nh), _i(nkv), _i(d), _i(bs), _i(window), _f(scale), _i(split_keys), _i(num_splits), _i(max_ctx),
        _p(live_count), _i(full_splits), _i(DECODE_WAVES), _p(step_flags), _stream()))
    return (part_o, part_ml, num_splits) if leave_parts else out


def attention_out_product_supported(items: int, num_heads: int, head_dim: int, width: int, num_splits: int) -> bool:
    """Whether :func:`attention_out_product_bf16` takes these sizes."""
    return bool(lib().me_attention_out_product_supported(_i(items), _i(num_heads), _i(head_dim), _i(width), _i(num_splits)))


def attention_out_product_bf16(part_o, part_ml, num_splits: int, weight, items: int, num_heads: int) -> torch.Tensor:
    """The output projection of a decode step of very few items, from the partial results that a decode attention
    launch left (``leave_parts``): the splits are added up and rounded to bfloat16 as the second attention kernel
    does, and multiplied with weight [n, nh d]. The result is float32 [runs, items, n]: sums over runs of k that the
    next add-and-norm adds up."""
    _want(weight, "weight", torch.bfloat16, (None, None))
    n, k = weight.shape
    if k % num_heads:
        raise ValueError(f"a weight of {k} columns does not hold {num_heads} heads")
    d = k // num_heads
    _want(part_o, "part_o", torch.float32, (items * num_heads * num_splits * d,))
    _want(part_ml, "part_ml", torch.float32, (items * num_heads * num_splits * 2,))
    runs = lib().me_attention_out_product_runs(_i(num_heads))
    parts = torch.empty((runs, items, n), dtype=torch.float32, device=weight.device)
    check(lib().me_attention_out_product_bf16(_p(part_o), _p(part_ml), _i(num_splits), _p(weight), _p(parts), _i(items),
                                              _i(num_heads), _i(d), _i(n), _stream()))
    return parts


class PrefillPlan:
    """The work list of one step's prefill attention, on the device: which tile of query tokens meets
    which range of keys, and which block runs which entries. It depends on the step's items and on the
    attention's window, not on the layer, so a step builds it once."""

    def __init__(self, work: torch.Tensor, bundle_first: torch.Tensor, token_chunks: torch.Tensor | None,
                 num_bundles: int, max_chunks: int, columns: int | None = None):
        self.work, self.bundle_first, self.token_chunks = work, bundle_first, token_chunks
        self.num_bundles, self.max_chunks = num_bundles, max_chunks
        # query columns (token, head of the kv group) per block that the tiles were cut for
        self.columns = lib().me_attention_prefill_columns(0) if columns is None else columns


def prefill_work_list(starts: list[int], qlens: list[int], tpb: int, window: int, nkv: int, slots: int,
                      partial_row_bytes: int = 0):
    """Host side of :class:`PrefillPlan`: (entries int32 [n, 8], first entry of each bundle int32 [b],
    chunks per token int32 [T], max chunks), as ``csrc/host/prefill_plan.cpp`` builds it (the native
    step uses the same builder).

    A tile of ``tpb`` query tokens of an item meets the keys from its window's first (rounded down to a
    multiple of 64) to its last token's position. A bundle of entries is run by one block per kv head;
    tiles of a step with few of them are cut into key ranges whose partial results a second kernel adds
    up. An entry is (item, first token, tokens, first position, first key, last key, chunk or -1, 1 if
    its bundle ends with it)."""
    s = np.ascontiguousarray(starts, dtype=np.int32)
    q = np.ascontiguousarray(qlens, dtype=np.int32)
    total = int(q.sum())
    counts = np.zeros(3, dtype=np.int32)
    cap_entries = cap_bundles = 0
    for _ in range(2):  # the first call says how much room the lists need
        work = np.empty((cap_entries, 8), dtype=np.int32)
        first = np.empty(cap_bundles, dtype=np.int32)
        token_chunks = np.empty(total, dtype=np.int32)
        rc = lib().me_prefill_work_list(_vp(s.ctypes.data), _vp(q.ctypes.data), _i(len(q)), _i(tpb), _i(window), _i(nkv),
                                        _i(slots), ctypes.c_longlong(partial_row_bytes), _vp(work.ctypes.data), _i(cap_entries),
                                        _vp(first.ctypes.data), _i(cap_bundles), _vp(token_chunks.ctypes.data), _i(total),
                                        _vp(counts.ctypes.data))
        if rc == 0:
            return work, first, token_chunks, int(counts[2])
        cap_entries, cap_bundles = int(counts[0]), int(counts[1])
    raise RuntimeError("me_prefill_work_list: the lists do not fit the room it asked for")


_PLANS: dict = {}  # the last plans made, by what they were made from: steps of a serving loop repeat


def prefill_plan(starts: list[int], qlens: list[int], nh: int, nkv: int, d: int, window: int, device,
                 wide: bool | None = None) -> PrefillPlan:
    """``wide``: blocks of twice as many query columns or not; None lets the step's size decide."""
    key = (tuple(starts), tuple(qlens), nh, nkv, d, window, str(device), wide)
    plan = _PLANS.get(key)
    if plan is None:
        if len(_PLANS) >= 64:
            _PLANS.pop(next(iter(_PLANS)))
        plan = _PLANS[key] = _make_prefill_plan(starts, qlens, nh, nkv, d, window, device, wide)
    return plan


def wide_blocks_pay(starts: list[int], qlens: list[int], tpb: int, window: int, nkv: int, slots: int) -> bool:
    """Whether a step takes prefill attention blocks of twice as many query columns: they read each key and
    value tile once for twice the work, but a step has half as many of them (the rule and its limits live
    in ``csrc/host/prefill_plan.cpp``, which the native step uses too)."""
    s = np.ascontiguousarray(starts, dtype=np.int32)
    q = np.ascontiguousarray(qlens, dtype=np.int32)
    return bool(lib().me_prefill_wide_blocks_pay(_vp(s.ctypes.data), _vp(q.ctypes.data), _i(len(q)), _i(tpb), _i(window),
                                                 _i(nkv), _i(slots)))


def set_prefill_wide_limits(min_blocks: float, min_key_tiles: float) -> tuple[float, float]:
    """Set the two limits of :func:`wide_blocks_pay` (blocks and key tiles per compute unit from which wide
    blocks are taken) and return the old ones: for measurements and tests that want one block width
    whatever the step. Plans already made keep their width."""
    old = (ctypes.c_double * 2)()
    lib().me_prefill_wide_limits(ctypes.c_double(min_blocks), ctypes.c_double(min_key_tiles), old)
    _PLANS.clear()
    return old[0], old[1]


def _make_prefill_plan(starts: list[int], qlens: list[int], nh: int, nkv: int, d: int, window: int, device,
                       wide: bool | None = None) -> PrefillPlan:
    group = nh // nkv
    slots = torch.cuda.get_device_properties(device).multi_processor_count
    if wide is None:
        wide = wide_blocks_pay(starts, qlens, max(1, lib().me_attention_prefill_columns(1) // group), window, nkv, slots)
    columns = lib().me_attention_prefill_columns(1 if wide else 0)
    tpb = columns // group
    work, first, token_chunks, max_chunks = prefill_work_list(starts, qlens, tpb, window, nkv, slots, nh * d * 4)
    parts = [work.reshape(-1), first] + ([token_chunks] if max_chunks > 1 else [])
    both = torch.from_numpy(np.concatenate(parts)).to(device)  # one upload
    a, b = work.size, work.size + first.size
    return PrefillPlan(both[:a], both[a:b], both[b:] if max_chunks > 1 else None, first.size, max_chunks, columns)


def attention_prefill_bf16(q, k_cache, v_cache, positions, item_start, qlens: list[int], block_table, scale: float,
                           window: int = 0, out: torch.Tensor | None = None, starts: list[int] | None = None,
                           plan: PrefillPlan | None = None) -> torch.Tensor:
    """Causal attention of packed new tokens q [T, nh, d] bfloat16 over the paged cache (which already
    holds the new tokens' keys and values). item_start int32 [items + 1] are the items' offsets into
    the packed tokens, ``qlens`` the same lengths on the host and ``starts`` the position of each item's
    first token (read back from ``positions`` when not given); ``plan`` is what :func:`prefill_plan`
    makes of them, for callers that run several layers on one step."""
    _want(q, "q", torch.bfloat16, (None, None, None))
    t, nh, d = q.shape
    nkv, bs = k_cache.shape[1], k_cache.shape[2]
    _check_cache(k_cache, v_cache, torch.bfloat16, nkv, d, bs)
    items = len(qlens)
    if sum(qlens) != t:
        raise ValueError(f"item lengths sum to {sum(qlens)}, but q has {t} tokens")
    _want(positions, "positions", torch.int32, (t,))
    _want(item_start, "item_start", torch.int32, (items + 1,))
    _want(block_table, "block_table", torch.int32, (items, None))
    group = nh // nkv
    if group > 16:
        raise ValueError(f"group size {group} exceeds what the matrix-core prefill kernel takes (16)")
    if plan is None:
        if starts is None:
            firsts = np.concatenate([[0], np.cumsum(qlens)[:-1]])
            starts = positions[torch.from_numpy(firsts).to(positions.device)].tolist()
        plan = prefill_plan(starts, qlens, nh, nkv, d, window, q.device)
    if out is None:
        out = torch.empty((t, nh * d), dtype=torch.bfloat16, device=q.device)
    _want(out, "out", torch.bfloat16, (t, nh * d))
    part_o = part_ml = None
    if plan.max_chunks > 1:
        part_o = torch.empty((t * nh * plan.max_chunks * d,), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((t * nh * plan.max_chunks * 2,), dtype=torch.float32, device=q.device)
    check(lib().me_attention_prefill_bf16(
        _p(q), _p(k_cache), _p(v_cache), _i(items), _p(block_table),
        _i(block_table.shape[1]), _p(out), _p(plan.work), _p(plan.bundle_first), _i(plan.num_bundles), _p(part_o), _p(part_ml),
        _p(plan.token_chunks), _i(plan.max_chunks), _i(t), _i(nh), _i(nkv), _i(d), _i(bs), _i(window), _f(scale),
        _i(plan.columns), _stream()))
    return out

