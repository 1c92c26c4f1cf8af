"""The model's pass launched kernel by kernel from Python, through each part's ``forward``: what the tests hold the
engine's step program against. It is no part of the product: generation, replay and the benchmark run the program
(``Decoder.emit``); this pass runs the same parts on the same cache through their Python entry points, one call per
kernel, and draws with the sampler."""

from __future__ import annotations

import numpy as np
import torch

from mini_engine_amd.engine.batch import StepBatch
from mini_engine_amd.engine.runner import ModelRunner
from mini_engine_amd.ops import kernels as K


def batch_from_core(core, device, spare_block: int = 0, spare_slot: int = 0) -> StepBatch:
    """Pack the core's current step and upload it."""
    layout = core.step_layout()
    arr = np.empty(layout["total"], dtype=np.int32)
    core.step_pack(arr, None, 0, spare_block, spare_slot)
    _, starts, counts, _, slots = core.step_items()
    return StepBatch(torch.from_numpy(arr).to(device), layout).describe(starts, counts, slots)


def run_part(part, norm, x, pending, spare, batch, extra, dtype):
    """One half of a pre-norm block: the residual add and the norm, then the part. A part whose class sets
    ``takes_normed_input`` is handed the add-and-norm unevaluated and may fuse it into its first product."""
    fused = norm.as_fused()
    if fused is None:  # any other norm: the add as a kernel of its own, then the part
        if pending is not None:
            K.residual_add(x, pending)
        return x, spare, part.forward(norm.forward(x), batch, *extra)
    h = K.NormedInput(x, pending, fused[0], fused[1], dtype, spare)
    out = part.forward(h if getattr(part, "takes_normed_input", False) else h.materialize(), batch, *extra)
    if h.residual is None:  # the part never looked at its input: the add still has to happen
        h.materialize()
    if h.residual is not x:
        x, spare = h.residual, x
    return x, spare, out


def decoder_forward(decoder, batch) -> torch.Tensor:
    """Logits float32 [R, V] for ``batch.want_rows``: embedding, every run of ``plan.order``, final norm, head."""
    plan = decoder.plan
    x = K.embed(batch.token_ids, decoder.embed_table, multiplier=plan.embedding_multiplier or 1.0)
    spare = torch.empty_like(x)  # the residual stream alternates between two buffers
    pending = None
    for r, i in enumerate(plan.order):
        blk, cache = decoder.blocks[i], decoder.bindings[r]
        x, spare, a = run_part(blk.mixer, blk.mixer_norm, x, pending, spare, batch, (cache,), decoder.dtype)
        x, spare, pending = run_part(blk.ffn, blk.ffn_norm, x, a, spare, batch, (), decoder.dtype)
    rows = batch.want_rows
    if rows.numel() == 0:
        return torch.empty((0, plan.vocab_size), dtype=torch.float32, device=decoder.device)
    fused = decoder.final_norm.as_fused()
    if fused is not None:
        h = K.add_rmsnorm(x, pending, fused[0], fused[1], decoder.dtype, rows=rows, write_x=False)
    else:
        if pending is not None:
            K.residual_add(x, pending)
        h = decoder.final_norm.forward(x.index_select(0, rows.long()))
    logits = K.linear(h, decoder.head, torch.float32, head=True)
    if plan.logit_scale not in (None, 1.0):
        K.scale_(logits, plan.logit_scale)
    return logits


class KernelByKernelRunner(ModelRunner):
    """A :class:`ModelRunner` whose steps run :func:`decoder_forward` instead of the step program: the same checks,
    cache and graphs around another pass over the same parts."""

    def _run_eager(self, tokens, items, rows, ctx):
        core = self.core
        core.step_check(self.decoder.plan.vocab_size, scan_pages=True)
        self._zero_fresh_state()
        self.batch = batch_from_core(core, self.device, self.storage.spare_block, self.storage.spare_slot)
        self._drawn = None
        return decoder_forward(self.decoder, self.batch)

    def _forward_static(self, batch, bucket):
        return decoder_forward(self.decoder, batch), None
