"""Rotary position encoding part (rotate-half pairing).

``inv_freq[j] = 1 / theta ** (2j / rotary_dim)`` in float32, exactly the expression of the
reference (``src/mini_engine/model.py:75``); the angle ``position * inv_freq[j]`` and its cosine and
sine are computed in float32 inside the mixer's kernel (``model.py:79-90``).
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

    def tables(self) -> torch.Tensor:
        return self.inv_freq


POSITION_ENCODINGS.register("rotary", Rotary)
