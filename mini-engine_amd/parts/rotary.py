"""Rotary position encoding part (rotate-half pairing).

``inv_freq[j] = 1 / theta ** (2j / rotary_dim)`` in float32, exactly the expression of the
reference (``src/mini_engine/model.py:75``); the angle ``position * inv_freq[j]`` and its cosine and
sine are computed in float32 (``model.py:79-90``) by a kernel, once per position, into a table
``[positions, 2, rotary_dim / 2]`` that the mixer's kernels read.
"""

from __future__ import annotations

import torch

from .base import POSITION_ENCODINGS, PositionEncoding


class Rotary(PositionEncoding):
    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        rd = int(spec.rotary_dim)
        if rd <= 0 or rd % 2:
            raise ValueError(f"rotary_dim must be a positive even number, got {rd}")
        self.rotary_dim = rd
        inv_freq = 1.0 / (float(spec.theta) ** (torch.arange(0, rd, 2, dtype=torch.float32) / rd))
        self.inv_freq = inv_freq.to(device)

        self._table: torch.Tensor | None = None
        self._retired: list[torch.Tensor] = []

    def tables(self, num_positions: int = 1) -> torch.Tensor:
        """The cos/sin table for positions ``0 .. num_positions - 1`` (grown in powers of two; never
        inside a graph capture, where the engine has sized it beforehand)."""
        if self._table is None or self._table.shape[0] < num_positions:
            from ..ops import kernels as K

            size = 256
            while size < num_positions:
                size *= 2
            if self._table is not None:
                self._retired.append(self._table)  # a captured graph may still read the smaller table
            self._table = K.rope_table(self.inv_freq, size)
        return self._table


POSITION_ENCODINGS.register("rotary", Rotary)
