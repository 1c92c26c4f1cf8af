"""Grouped-query attention mixer over a paged key/value cache.

Per step (reference: ``src/mini_engine/model.py:111-119`` and ``attention.py:104-175``):
one product for q, k and v (the three weights are stacked at load time), then one fused kernel for
the per-head q/k RMSNorm, the position encoding and the write of the new keys and values into their
pages, then attention of every new token over the pages of its request (causal, optionally within a
window), then the output projection.

Sizes and constants all come from the spec: head counts, head size, score scale, eps of the q/k
norm (None: no norm), window (0: none), position encoding (None: none), and ``cache_from`` (read
another layer's pages and write none).
"""

from __future__ import annotations

import torch

from ..ops import kernels as K
from ..weights.loader import TensorWant
from .base import MIXERS, POSITION_ENCODINGS, KVBinding, KVCacheNeed, Mixer

MAX_HEAD_DIM = 256


class Attention(Mixer):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        s = spec
        if not (float(s.scale) > 0.0 and float(s.scale) < float("inf")):
            raise ValueError(f"the score scale must be positive and finite, got {s.scale}: the kernels scale before they mask")
        if s.num_heads % s.num_kv_heads:
            raise ValueError(f"{s.num_heads} query heads are not a multiple of {s.num_kv_heads} key/value heads")
        if s.head_dim % 16 or not 16 <= s.head_dim <= MAX_HEAD_DIM:
            raise ValueError(f"head_dim={s.head_dim} is not supported: the attention kernels take head sizes "
                             f"from 16 to {MAX_HEAD_DIM} in steps of 16")
        if s.window < 0:
            raise ValueError(f"window={s.window} must be >= 0")
        self.nh, self.nkv, self.d = s.num_heads, s.num_kv_heads, s.head_dim
        self.position = None if s.position is None else POSITION_ENCODINGS.build(s.position, dtype, device)
        self.q_norm_w = self.k_norm_w = None
        self.w_qkv = self.w_o = None

    # ---- weights
    def weight_wants(self, prefix: str) -> dict[str, TensorWant]:
        s = self.spec
        wants = {
            f"{prefix}.q_proj.weight": TensorWant((s.num_heads * s.head_dim, s.hidden_size)),
            f"{prefix}.o_proj.weight": TensorWant((s.hidden_size, s.num_heads * s.head_dim)),
        }
        if s.cache_from is None:
            wants[f"{prefix}.k_proj.weight"] = TensorWant((s.num_kv_heads * s.head_dim, s.hidden_size))
            wants[f"{prefix}.v_proj.weight"] = TensorWant((s.num_kv_heads * s.head_dim, s.hidden_size))
        if s.qk_norm_eps is not None:
            wants[f"{prefix}.q_norm.weight"] = TensorWant((s.head_dim,), "vector")
            if s.cache_from is None:
                wants[f"{prefix}.k_norm.weight"] = TensorWant((s.head_dim,), "vector")
        return wants

    def load(self, tensors, prefix: str) -> None:
        s = self.spec
        q = tensors[f"{prefix}.q_proj.weight"]
        if s.cache_from is None:
            self.w_qkv = torch.cat((q, tensors[f"{prefix}.k_proj.weight"], tensors[f"{prefix}.v_proj.weight"]), dim=0)
        else:
            self.w_qkv = q.contiguous()
        self.w_o = tensors[f"{prefix}.o_proj.weight"]
        if s.qk_norm_eps is not None:
            self.q_norm_w = tensors[f"{prefix}.q_norm.weight"]
            self.k_norm_w = tensors.get(f"{prefix}.k_norm.weight")

    # ---- cache
    def cache_need(self):
        if self.spec.cache_from is not None:
            return None
        return KVCacheNeed(self.nkv, self.d, self.spec.window)

    def cache_source(self):
        return self.spec.cache_from

    # ---- step
    takes_normed_input = True

    def forward(self, h, batch, cache: KVBinding | None = None) -> torch.Tensor:
        s, b = self.spec, cache
        if b is None:
            raise RuntimeError("attention mixer was given no cache")
        owns = s.cache_from is None
        proj = K.linear(h, self.w_qkv)  # [T, (nh + 2 nkv) d] or [T, nh d]
        table = batch.block_table(b.group)
        rope = None if self.position is None else self.position.tables(batch.max_ctx)
        eps = 0.0 if s.qk_norm_eps is None else float(s.qk_norm_eps)
        if (self.dtype is torch.bfloat16 and batch.decode_only and K.attention_decode_fused_supported(
                self.d, b.block_size, 0 if rope is None else 2 * rope.shape[2], self.nh // self.nkv)):
            # one new token per item: norm, rotary, page write and attention in one launch
            out = K.attention_decode_fused_bf16(
                proj, self.q_norm_w, self.k_norm_w if owns else None, rope, eps, owns, b.k_cache, b.v_cache,
                batch.item_ctx, table, self.nh, float(s.scale), int(s.window), batch.max_ctx,
                live=(batch.live_items, batch.least_live))
            return K.linear(out, self.w_o, as_delta=True)
        q = K.qk_norm_rope_scatter(
            proj, self.q_norm_w, self.k_norm_w if owns else None, rope, batch.positions, batch.token_item,
            table, b.k_cache, b.v_cache, self.nh, self.nkv, self.d, eps, write_kv=owns,
            item_start=batch.item_start, starts=batch.starts, qlens=batch.qlens)
        out = self.attend(q, batch, table, b)
        return K.linear(out, self.w_o, as_delta=True)

    def emit(self, program, h, cache: KVBinding | None = None) -> None:
        s, b = self.spec, cache
        if b is None:
            raise RuntimeError("attention mixer was given no cache")
        owns = s.cache_from is None
        qkv = program.linear(h, self.w_qkv)
        out = program.attention(
            qkv, q_norm=self.q_norm_w, k_norm=self.k_norm_w if owns else None,
            rope=None if self.position is None else self.position.tables(program.max_positions),
            k_cache=b.k_cache, v_cache=b.v_cache, heads=self.nh, kv_heads=self.nkv, head_dim=self.d,
            block_size=b.block_size, window=int(s.window), writes=owns, group=b.group,
            eps=0.0 if s.qk_norm_eps is None else float(s.qk_norm_eps), scale=float(s.scale))
        program.linear_delta(out, self.w_o)

    def attend(self, q: torch.Tensor, batch, table: torch.Tensor, b: KVBinding) -> torch.Tensor:
        """bfloat16 with sizes the matrix-core kernels take: the split-context kernel when every item
        brings one token, else the tiled prefill kernel. Everything else (float32, other head or page
        sizes): the general kernel."""
        s = self.spec
        scale, window = float(s.scale), int(s.window)
        if self.dtype is torch.bfloat16 and K.attention_mfma_supported(self.d, b.block_size, self.nh // self.nkv):
            if batch.decode_only:
                return K.attention_decode_bf16(q, b.k_cache, b.v_cache, batch.item_ctx, table, scale, window,
                                               batch.max_ctx, live=(batch.live_items, batch.least_live))
            key = ("prefill_plan", self.nh, self.nkv, self.d, window)
            plan = batch.derived.get(key)
            if plan is None:  # the same for every layer of this shape: made once per step
                plan = K.prefill_plan(batch.starts, batch.qlens, self.nh, self.nkv, self.d, window, q.device)
                batch.derived[key] = plan
            return K.attention_prefill_bf16(q, b.k_cache, b.v_cache, batch.positions, batch.item_start, batch.qlens,
                                            table, scale, window, plan=plan)
        return K.attention_general(q, b.k_cache, b.v_cache, batch.positions, batch.token_item, table, scale, window)


MIXERS.register("attention", Attention)
