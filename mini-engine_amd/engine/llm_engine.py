"""The engine loop: schedule -> step function -> sample -> postprocess
(reference: ``src/mini_engine/engine.py:59-300``, without its speculative-decoding branches)."""

from __future__ import annotations

import os
from collections.abc import Iterable
from dataclasses import dataclass, field

import torch

from .. import models as _models  # noqa: F401  (registers the architectures)
from ..config.engine_config import EngineConfig
from ..config.registry import get_architecture, plan_from_folder
from ..config.specs import ModelPlan
from ..parts.decoder import Decoder
from ..sampling.sampler import Sampler
from ..weights.loader import FolderSource
from ..weights.random_init import RandomSource
from .batch import StepItem
from .runner import TORCH_DTYPES, ModelRunner
from .scheduler import ScheduledSeq, Scheduler, SchedulerConfig
from .sequence import SamplingParams, Sequence


@dataclass
class EngineStats:
    steps: int = 0
    prompt_tokens: int = 0  # cached hits are in `scheduler.num_cached_tokens`
    computed_tokens: int = 0  # tokens actually run through the model
    generated_tokens: int = 0
    step_batch_sizes: list[int] = field(default_factory=list)


def kv_cache_bytes_per_token(plan: ModelPlan, dtype: str) -> int:
    """``2 * kv_heads * head_dim * element size`` summed over the runs of attention layers that own
    a cache (reference: ``engine.py:54-56``, where that is ``2 * layers * kv_heads * head_dim``)."""
    elem = 4 if dtype == "float32" else 2
    runs = [plan.layers[i].mixer for i in plan.order]
    return sum(2 * m.num_kv_heads * m.head_dim * elem for m in runs
               if getattr(m, "kind", "") == "attention" and m.cache_from is None)


class LLMEngine:
    def __init__(self, model: Decoder, config: EngineConfig, eos_token_ids: Iterable[int] = ()):
        if TORCH_DTYPES[config.dtype] is not model.dtype:
            raise ValueError(f"the model was built for {model.dtype}, the engine config says {config.dtype}")
        self.config = config
        self.model = model
        self.runner = ModelRunner(model, config)
        self.block_manager = self.runner.new_block_manager()
        self.scheduler = Scheduler(
            SchedulerConfig(config.max_num_seqs, config.max_num_batched_tokens, config.max_model_len),
            self.block_manager,
            set(eos_token_ids),
        )
        self.sampler = Sampler(config.seed, model.device)
        self.stats = EngineStats()

    @property
    def kv_caches(self):
        return self.runner.storage.kv

    # ----------------------------------------------------------------- loading

    @classmethod
    def from_pretrained(cls, model_id_or_path: str, config: EngineConfig | None = None, progress=None) -> "LLMEngine":
        """Load a checkpoint from a local folder: ``config.json`` names the architecture, every
        ``*.safetensors`` file holds weights. Nothing is fetched from a network."""
        config = config or EngineConfig()
        if not os.path.isdir(model_id_or_path):
            raise FileNotFoundError(f"{model_id_or_path!r} is not a folder; models are loaded from local folders only")
        arch_config, plan = plan_from_folder(model_id_or_path)
        model = Decoder(plan, TORCH_DTYPES[config.dtype], "cuda")
        model.load(FolderSource(model_id_or_path), progress)
        return cls(model, config, plan.eos_token_ids)

    @classmethod
    def from_random(cls, architecture: str, arch_config, config: EngineConfig | None = None, seed: int = 0,
                    std: float = 0.02) -> "LLMEngine":
        """Build the architecture with seeded random weights generated on the GPU (no files)."""
        config = config or EngineConfig()
        plan = get_architecture(architecture).plan_from_config(arch_config)
        model = Decoder(plan, TORCH_DTYPES[config.dtype], "cuda")
        model.load(RandomSource(model.weight_wants(), seed, std=std, device="cuda"))
        return cls(model, config, plan.eos_token_ids)

    # -------------------------------------------------------------------- API

    def add_request(self, prompt_token_ids: list[int], params: SamplingParams | None = None) -> Sequence:
        seq = Sequence(prompt_token_ids, params or SamplingParams())
        vocab = self.model.plan.vocab_size
        if min(seq.token_ids) < 0 or max(seq.token_ids) >= vocab:
            raise ValueError(f"prompt holds a token id outside the vocabulary of {vocab}")
        self.scheduler.add(seq)
        self.stats.prompt_tokens += len(seq)
        return seq

    def generate(self, prompts: list[list[int]], params: SamplingParams | None = None) -> list[list[int]]:
        """Run all prompts to completion as one continuously batched workload."""
        seqs = [self.add_request(p, params) for p in prompts]
        while self.scheduler.has_unfinished():
            self.step()
        return [s.output_token_ids for s in seqs]

    def step(self) -> list[Sequence]:
        batch = self.scheduler.schedule()
        if not batch:
            raise RuntimeError("scheduler produced an empty batch with work pending")
        items = self._prepare(batch)
        logits = self.runner.step(items)
        sampling = [item for item in batch if item.samples]
        sampled = self.sampler.sample(
            logits,
            [i.seq.params.temperature for i in sampling],
            [i.seq.seq_id for i in sampling],
            [i.seq.num_output_tokens for i in sampling],
        )
        it = iter(sampled)
        next_tokens = [next(it) if item.samples else None for item in batch]
        self._update_stats(batch)
        return self.scheduler.postprocess(batch, next_tokens)

    # ---------------------------------------------------------------- private

    @staticmethod
    def _prepare(batch: list[ScheduledSeq]) -> list[StepItem]:
        items = []
        for item in batch:
            start = item.seq.num_computed_tokens
            tokens = item.seq.token_ids[start : start + item.num_tokens]
            items.append(StepItem(item.seq, tokens, start, [item.num_tokens - 1] if item.samples else []))
        return items

    def _update_stats(self, batch: list[ScheduledSeq]) -> None:
        s = self.stats
        s.steps += 1
        s.step_batch_sizes.append(len(batch))
        for item in batch:
            s.computed_tokens += item.num_tokens
            s.generated_tokens += int(item.samples)
