"""The generic decoder: embedding, a list of blocks run in the plan's order, final norm, head.

It is built from a :class:`~mini_engine_amd.config.specs.ModelPlan` alone. The forward pass takes a
packed batch of new tokens (reference: ``src/mini_engine/model.py:172-188``) and returns float32
logits for the wanted rows only; rows are selected before the final norm, as the reference does
(``model.py:186``).
"""

from __future__ import annotations

import torch

from ..config.specs import ModelPlan
from ..weights.loader import TensorWant, load_tensors
from .base import NORMS
from .block import build_block


class Decoder:
    def __init__(self, plan: ModelPlan, dtype: torch.dtype, device: torch.device | str = "cuda"):
        self.plan, self.dtype, self.device = plan, dtype, torch.device(device)
        self.blocks = [build_block(spec, dtype, self.device) for spec in plan.layers]
        self.final_norm = NORMS.build(plan.final_norm, dtype, self.device)
        self.embed_table: torch.Tensor | None = None
        self.head: torch.Tensor | None = None
        # One cache per run (position in plan.order), not per layer: a layer named twice keeps the
        # keys of each run apart. cache_owner[r] is the run whose cache run r uses: itself, or the
        # latest earlier run of the layer its mixer names as its cache source.
        self.cache_owner: list[int] = []
        for r, i in enumerate(plan.order):
            src = self.blocks[i].mixer.cache_source()
            if src is None:
                self.cache_owner.append(r)
                continue
            earlier = [q for q in range(r) if plan.order[q] == src and self.blocks[src].mixer.cache_source() is None]
            if not earlier:
                raise ValueError(f"layer {i} reads the cache of layer {src}, which has not run before it or owns none")
            self.cache_owner.append(earlier[-1])
        self.bindings: list = [None] * len(plan.order)  # filled by the cache storage

    # ---- weights
    def weight_wants(self) -> dict[str, TensorWant]:
        p = self.plan
        wants = {p.embed_name: TensorWant((p.vocab_size, p.hidden_size))}
        for blk in self.blocks:
            wants.update(blk.weight_wants())
        wants.update(self.final_norm.weight_wants(p.final_norm_name))
        if not p.tie_word_embeddings:
            wants[p.head_name] = TensorWant((p.vocab_size, p.hidden_size))
        return wants

    def load(self, source, progress=None) -> None:
        """``source`` has ``shapes()`` and ``get(name)``. A stored head is ignored when the head is
        tied to the embedding (reference: ``model.py:190-195``)."""
        p = self.plan
        ignorable = (p.head_name,) if p.tie_word_embeddings else ()
        tensors = load_tensors(source, self.weight_wants(), self.dtype, self.device, ignorable, progress)
        self.embed_table = tensors[p.embed_name]
        self.head = self.embed_table if p.tie_word_embeddings else tensors[p.head_name]
        for blk in self.blocks:
            blk.load(tensors)
        self.final_norm.load(tensors, p.final_norm_name)

    def weight_bytes(self) -> int:
        """Bytes of every distinct weight tensor a step reads (a tied head counts once)."""
        seen, total = set(), 0
        def add(t):
            nonlocal total
            if t is not None and t.data_ptr() not in seen:
                seen.add(t.data_ptr())
                total += t.numel() * t.element_size()
        add(self.head)
        parts = [self.final_norm]
        for i in set(self.plan.order):
            parts += [self.blocks[i].mixer, self.blocks[i].ffn, self.blocks[i].mixer_norm, self.blocks[i].ffn_norm]
        for obj in parts:
            for v in vars(obj).values():
                if isinstance(v, torch.Tensor):
                    add(v)
        return total

    # ---- step
    def emit(self, program) -> None:
        """Write the model's forward pass and the draw of the next tokens into a step program: what a step runs.
        The cache bindings have to be in place."""
        if self.embed_table is None:
            raise RuntimeError("weights are not loaded")
        program.embed(self.embed_table, self.plan.embedding_multiplier or 1.0)
        for r, i in enumerate(self.plan.order):
            self.blocks[i].emit(program, self.bindings[r])
        if self.final_norm.as_fused() is not None:
            program.head(self.final_norm, self.head, self.plan.logit_scale or 1.0)
        else:
            program.head_by(self.final_norm, self.head, self.plan.logit_scale or 1.0)
        program.sample()

    def graph_safe(self) -> bool:
        """Whether a decode step of this model may be captured into a graph: every part says so
        (``graph_safe`` of :class:`~mini_engine_amd.parts.base.Part`)."""
        parts = [self.final_norm]
        for i in set(self.plan.order):
            b = self.blocks[i]
            parts += [b.mixer, b.ffn, b.mixer_norm, b.ffn_norm]
        return all(getattr(p, "graph_safe", False) for p in parts)
