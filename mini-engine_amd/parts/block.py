"""Arrangements of a mixer, a feed-forward and their norms into one residual block.

``pre_norm`` (reference: ``src/mini_engine/model.py:142-151``)::

    x = x + mixer(norm1(x));  x = x + ffn(norm2(x))

The residual stream ``x`` is kept in float32 and every sum into it is a float32 sum. A block returns
its feed-forward output unadded; the next norm kernel (of the next block, or the model's final norm)
adds it while it norms, so each residual add costs no pass of its own.
"""

from __future__ import annotations

import torch

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
