"""Greedy and temperature sampling (reference: ``src/mini_engine/engine.py:282-291``).

Greedy rows take the argmax. A row with temperature ``t > 0`` draws from
``softmax(logits / max(t, 1e-5))``; the draw is made on the GPU by adding Gumbel noise to the scaled
logits and taking the argmax, which has exactly that distribution. The reference draws the whole
batch from one generator, so its samples depend on what else is in the batch; here the noise of a
draw is a function of (engine seed, number of the request within its engine, index of the output
token) alone, so a request's sampled tokens are the same under every way of batching it and in a
second engine with the same seed. The native host core derives the keys and packs them, with the
temperatures, into the step's index buffer.
"""

from __future__ import annotations

import numpy as np
import torch

from ..ops import kernels as K

_MASK = (1 << 64) - 1


def mix64(z: int) -> int:
    """The 64-bit mixer the sampling kernel uses for its noise (splitmix64's finaliser)."""
    z = (z + 0x9E3779B97F4A7C15) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def draw_key(seed: int, request_number: int, output_index: int) -> int:
    """Key of one draw as the host core derives it, as a signed 64-bit integer (the kernel reads the bits)."""
    k = mix64(mix64(mix64(seed & _MASK) ^ (request_number & _MASK)) ^ (output_index & _MASK))
    return k - (1 << 64) if k >= (1 << 63) else k


class Sampler:
    def draw(self, logits: torch.Tensor, batch, rows: int, tempered: bool) -> np.ndarray:
        """One token id per wanted row of the step (int32), read back to the host. ``batch`` is the
        step's batch: its ``temperatures`` and ``sample_keys`` sections hold what each row is drawn with."""
        if rows == 0:
            return np.zeros(0, dtype=np.int32)
        if tempered:
            out = K.sample(logits[:rows], batch.temperatures[:rows], batch.sample_keys[:rows])
        else:
            out = K.sample(logits[:rows])
        return out.cpu().numpy()
