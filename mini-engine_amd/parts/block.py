"""Arrangements of a mixer, a feed-forward and their norms into one residual block.

``pre_norm`` (reference: ``src/mini_engine/model.py:142-151``)::

    x = x + mixer(norm1(x));  x = x + ffn(norm2(x))

The residual stream ``x`` is kept in float32 and every sum into it is a float32 sum. A block returns
its feed-forward output unadded; the next norm kernel (of the next block, or the model's final norm)
adds it while it norms, so each residual add costs no pass of its own.
"""

from __future__ import annotations

import torch

from ..ops import kernels as K
from .base import BLOCK_ARRANGEMENTS, FEED_FORWARDS, MIXERS, NORMS


class PreNormBlock:
    def __init__(self, spec, dtype: torch.dtype, device: torch.device):
        self.spec, self.dtype = spec, dtype
        self.mixer = MIXERS.build(spec.mixer, dtype, device)
        self.ffn = FEED_FORWARDS.build(spec.ffn, dtype, device)
        self.mixer_norm = NORMS.build(spec.mixer_norm, dtype, device)
        self.ffn_norm = NORMS.build(spec.ffn_norm, dtype, device)

    def weight_wants(self):
        s = self.spec
        wants = {}
        wants.update(self.mixer_norm.weight_wants(s.mixer_norm_name))
        wants.update(self.mixer.weight_wants(s.mixer_prefix))
        wants.update(self.ffn_norm.weight_wants(s.ffn_norm_name))
        wants.update(self.ffn.weight_wants(s.ffn_prefix))
        return wants

    def load(self, tensors) -> None:
        s = self.spec
        self.mixer_norm.load(tensors, s.mixer_norm_name)
        self.mixer.load(tensors, s.mixer_prefix)
        self.ffn_norm.load(tensors, s.ffn_norm_name)
        self.ffn.load(tensors, s.ffn_prefix)

    def forward(self, x: torch.Tensor, pending: torch.Tensor | None, batch, cache=None, spare: torch.Tensor | None = None):
        """``x`` float32 [T, H] is the residual stream, ``pending`` the previous block's output that
        still has to be added, ``cache`` the binding of this run of the layer, ``spare`` a second
        float32 buffer of x's shape. Returns ``(x, spare, pending)``: the buffer that now holds the
        residual stream, the other one, and this block's own pending output.

        A part whose class sets ``takes_normed_input`` is handed the add-and-norm unevaluated
        (:class:`~mini_engine_amd.ops.kernels.NormedInput`) and may fuse it into its first matrix
        product; any other part gets the normed activations."""
        x, spare, a = self._run(self.mixer, self.mixer_norm, x, pending, spare, batch, (cache,))
        return self._run(self.ffn, self.ffn_norm, x, a, spare, batch, ())

    def _run(self, part, norm, x, pending, spare, batch, extra):
        fused = norm.as_fused()
        if fused is None:  # any other norm: the add as a kernel of its own, then the part
            if pending is not None:
                K.residual_add(x, pending)
            return x, spare, part.forward(norm.forward(x), batch, *extra)
        h = K.NormedInput(x, pending, fused[0], fused[1], self.dtype, spare)
        out = part.forward(h if getattr(part, "takes_normed_input", False) else h.materialize(), batch, *extra)
        if h.residual is None:  # the part never looked at its input: the add still has to happen
            h.materialize()
        if h.residual is not x:
            x, spare = h.residual, x
        return x, spare, out


    # ---- the native step program
    def emit(self, program, cache=None) -> None:
        """Write the block into a step program. A part with ``emit`` writes its own operations; any other part, and
        any norm that is not RMS-shaped, enters as a call of its ``forward``."""
        for part, norm, extra in ((self.mixer, self.mixer_norm, (cache,)), (self.ffn, self.ffn_norm, ())):
            with program.scope():
                h = program.normed(norm) if norm.as_fused() is not None else program.normed_by(norm)
                if callable(getattr(part, "emit", None)):
                    out = part.emit(program, h, *extra)
                else:
                    out = program.call_part(part, h, extra)
                if not h.used:  # the part never looked at its input: the add still has to happen
                    h.value()
                if out is not None:
                    program.delta(out)


BLOCK_ARRANGEMENTS.register("pre_norm", PreNormBlock)


def build_block(spec, dtype, device):
    return BLOCK_ARRANGEMENTS.build(spec, dtype, device)
