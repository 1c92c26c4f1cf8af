"""Greedy and temperature sampling (reference: ``src/mini_engine/engine.py:282-291``).

Greedy rows take the argmax. A row with temperature ``t > 0`` draws from
``softmax(logits / max(t, 1e-5))``; the draw is made on the GPU by adding Gumbel noise to the scaled
logits and taking the argmax, which has exactly that distribution. The reference draws the whole
batch from one generator, so its samples depend on what else is in the batch; here the noise of a
draw is a function of (engine seed, request id, index of the output token) alone, so a request's
sampled tokens are the same under every way of batching it.
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


def draw_key(seed: int, request_id: int, output_index: int) -> int:
    """Key of one draw, as a signed 64-bit integer (the kernel reads the bit pattern)."""
    k = mix64(mix64(mix64(seed & _MASK) ^ (request_id & _MASK)) ^ (output_index & _MASK))
    return k - (1 << 64) if k >= (1 << 63) else k


class Sampler:
    def __init__(self, seed: int, device: torch.device):
        self.seed, self.device = seed, device

    def sample(self, logits: torch.Tensor, temperatures: list[float], request_ids: list[int],
               output_indices: list[int]) -> list[int]:
        """One token id per row of float32 ``logits`` [R, V]."""
        if logits.shape[0] == 0:
            return []
        if all(t == 0 for t in temperatures):
            return K.sample(logits).tolist()
        meta = np.zeros((2, len(temperatures)), dtype=np.int64)
        meta[0] = np.asarray(temperatures, dtype=np.float32).view(np.int32).astype(np.int64)
        meta[1] = [draw_key(self.seed, r, i) for r, i in zip(request_ids, output_indices)]
        dev = torch.from_numpy(meta).to(self.device)
        temps = dev[0].to(torch.int32).view(torch.float32).contiguous()
        return K.sample(logits, temps, dev[1].contiguous()).tolist()
