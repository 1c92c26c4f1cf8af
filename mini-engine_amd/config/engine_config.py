"""Engine options, with the reference's names and defaults (``src/mini_engine/engine.py:22-36``).

Left out on purpose: ``device`` (always the one GPU), ``speculative`` and ``attention_backend``
(one kernel set). ``cuda_graphs`` keeps its name: it switches HIP-graph replay of decode steps.
``dtype`` is ``"float32"`` or ``"bfloat16"``.
"""

from __future__ import annotations

from dataclasses import dataclass

DTYPES = ("float32", "bfloat16")


@dataclass(frozen=True)
class EngineConfig:
    block_size: int = 16
    num_blocks: int = 256
    max_num_seqs: int = 16
    max_num_batched_tokens: int = 2048
    max_model_len: int = 4096
    enable_prefix_caching: bool = True
    dtype: str = "float32"
    seed: int = 0
    cuda_graphs: bool = True
    decode_ahead: bool = True  # launch the next decode step before the host has read this step's tokens
    # None: the pool has ``num_blocks`` pages, as the reference sizes it. A fraction in (0, 1]: the pool takes what that
    # share of the GPU's memory leaves after everything already on it (the weights), and ``num_blocks`` is ignored.
    kv_memory_fraction: float | None = None

    def __post_init__(self) -> None:
        if self.dtype not in DTYPES:
            raise ValueError(f"dtype must be one of {DTYPES}, got {self.dtype!r}")
        if self.block_size < 1 or self.num_blocks < 1:
            raise ValueError("block_size and num_blocks must be positive")
        if self.kv_memory_fraction is not None and not 0.0 < self.kv_memory_fraction <= 1.0:
            raise ValueError("kv_memory_fraction must lie in (0, 1]")
        if self.max_num_seqs < 1 or self.max_num_batched_tokens < 1 or self.max_model_len < 1:
            raise ValueError("max_num_seqs, max_num_batched_tokens and max_model_len must be positive")
