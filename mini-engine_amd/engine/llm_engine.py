"""The engine: a model, its runner and the loop ``plan a step -> run it -> draw tokens -> settle``
(reference: ``src/mini_engine/engine.py:59-300``, without its speculative-decoding branches). The
planning and the settling happen in the native host core; this class wires the parts together and
keeps the reference's Python API: ``from_pretrained``, ``add_request``, ``generate``, ``step``,
``stats``.
"""

from __future__ import annotations

import os
from collections.abc import Iterable
from dataclasses import dataclass, field

import numpy as np
import torch

from .. import models as _models  # noqa: F401  (registers the architectures)
from ..config.engine_config import EngineConfig
from ..config.registry import get_architecture, plan_from_folder
from ..config.specs import ModelPlan
from ..parts.decoder import Decoder
from ..weights.loader import FolderSource
from ..weights.random_init import RandomSource
from .runner import TORCH_DTYPES, ModelRunner
from .scheduler import Scheduler, SchedulerConfig
from .sequence import SamplingParams, Sequence


@dataclass
class EngineStats:
    """Counters of the loop, under the reference's names (``engine.py:39-45``)."""

    steps: int = 0
    prompt_tokens: int = 0  # all prompt tokens submitted, whether computed or found in the prefix cache
    computed_tokens: int = 0  # tokens that went through the model
    generated_tokens: int = 0
    step_batch_sizes: list[int] = field(default_factory=list)
    # seconds spent in each phase of the steps so far
    phase_seconds: dict[str, float] = field(default_factory=lambda: {"schedule": 0.0, "forward": 0.0, "sample": 0.0,
                                                                     "postprocess": 0.0})


def kv_cache_bytes_per_token(plan: ModelPlan, dtype: str) -> int:
    """Bytes of keys and values that one token occupies over all layers of ``plan`` in ``dtype``
    (reference: ``engine.py:54-56``, where it is ``2 * layers * kv_heads * head_dim * element size``).
    Every mixer says what it keeps through its spec's ``kv_elements_per_token``; one without that
    attribute keeps no keys."""
    elem = 4 if dtype == "float32" else 2
    return elem * sum(int(getattr(plan.layers[i].mixer, "kv_elements_per_token", 0)) for i in plan.order)


def blocks_that_fit(free_bytes: int, total_bytes: int, fraction: float, plan: ModelPlan, dtype: str, block_size: int,
                    max_num_batched_tokens: int = 0) -> int:
    """How many pages a pool may have when the engine is to stay within ``fraction`` of the GPU's ``total_bytes``, of
    which ``free_bytes`` are free now (the weights are loaded): what is left after the other users of memory, and
    after the workspaces of a step of ``max_num_batched_tokens`` tokens (its float32 logits aside, a few rows of the
    hidden size per token: counted as 64 bytes per token and hidden element over the widest layer, generously),
    divided by a page's bytes over all layers. Every cache group has a pool of that many pages."""
    per_page = kv_cache_bytes_per_token(plan, dtype) * block_size
    if per_page <= 0:
        raise ValueError("this model keeps no keys or values: its pool cannot be sized by memory")
    widest = max([plan.hidden_size] + [int(getattr(layer.ffn, "intermediate_size", 0)) * 2 for layer in plan.layers])
    workspaces = 64 * max_num_batched_tokens * widest
    budget = free_bytes - int((1.0 - fraction) * total_bytes) - workspaces
    if budget < per_page:
        raise ValueError(f"{fraction:.2f} of the GPU's memory leaves no room for a page of {per_page} bytes "
                         f"({free_bytes} of {total_bytes} bytes are free)")
    return int(budget // per_page)


class LLMEngine:
    def __init__(self, model: Decoder, config: EngineConfig, eos_token_ids: Iterable[int] = ()):
        if TORCH_DTYPES[config.dtype] is not model.dtype:
            raise ValueError(f"the model was built for {model.dtype}, the engine config says {config.dtype}")
        if config.kv_memory_fraction is not None:  # the pool takes what the model left of its share of the memory
            import dataclasses
            free, total = torch.cuda.mem_get_info()
            fit = blocks_that_fit(free, total, config.kv_memory_fraction, model.plan, config.dtype, config.block_size,
                                  config.max_num_batched_tokens)
            config = dataclasses.replace(config, num_blocks=fit)
        self.config = config
        self.model = model
        eos = set(eos_token_ids)
        self.runner = ModelRunner(model, config, eos)
        self.core = self.runner.core
        self.block_manager = self.runner.new_block_manager()
        self.scheduler = Scheduler(
            SchedulerConfig(config.max_num_seqs, config.max_num_batched_tokens, config.max_model_len),
            self.block_manager, eos)
        self.sampler = self.runner.sampler
        self.stats = EngineStats()
        self.time_phases = False  # synchronise after each phase of a step and add its time to the stats
        self._launched: _Launched | None = None  # the step that was launched ahead and is not settled yet

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
        """Build the architecture with seeded random weights generated on the GPU (no files). The values come from the
        GPU's generator: they are other values than those of a model folder written for the same seed
        (``weights.random_init.write_model_folder`` draws on the CPU), with the same distribution."""
        config = config or EngineConfig()
        plan = get_architecture(architecture).plan_from_config(arch_config)
        model = Decoder(plan, TORCH_DTYPES[config.dtype], "cuda")
        model.load(RandomSource(model.weight_wants(), seed, std=std, device="cuda"))
        return cls(model, config, plan.eos_token_ids)

    # -------------------------------------------------------------------- API

    def add_request(self, prompt_token_ids: list[int], params: SamplingParams | None = None) -> Sequence:
        tokens = [int(t) for t in prompt_token_ids]
        vocab = self.model.plan.vocab_size
        if tokens and (min(tokens) < 0 or max(tokens) >= vocab):
            raise ValueError(f"prompt holds a token id outside the vocabulary of {vocab}")
        seq = Sequence(tokens, params, core=self.core)
        self.scheduler.add(seq)
        self.stats.prompt_tokens += len(tokens)
        return seq

    def generate(self, prompts: list[list[int]], params: SamplingParams | None = None) -> list[list[int]]:
        """Run all prompts to completion as one continuously batched workload; output ids per prompt."""
        requests = [self.add_request(p, params) for p in prompts]
        while self.scheduler.has_unfinished() or self._launched is not None:
            self.step()
        return [r.output_token_ids for r in requests]

    def _launch(self) -> "_Launched":
        """Launch the step the core holds; its draws are read later."""
        tokens, items, rows, *_, warm = (int(v) for v in self.core.step_summary())
        self.runner.run_planned()
        return _Launched(tokens, items, rows, bool(warm), self.runner.last_replay)

    def step(self) -> list[Sequence]:
        """One step of the loop; returns the requests that finished in it.

        With ``decode_ahead`` a decode step that was replayed from a graph is followed at once by the
        step after it, whose token ids the device takes from this step's draws, before the host reads
        those draws: scheduling, the refill of the next graph's indices and its launch overlap the
        device's work. A request that ends with an end token has then run one token too many, which is
        dropped."""
        if self.time_phases:
            return self._step_timed()
        step = self._launched
        if step is None:
            if self.core.plan() == 0:
                raise RuntimeError("scheduler produced an empty batch with work pending")
            step = self._launch()
        ahead = None
        if self.config.decode_ahead and step.replay is not None and self.core.plan_ahead() > 0:
            ahead = self._launch()
        drawn = self.runner.draw(step.rows, step.tempered, step.replay)
        before = int(self.core.counters()[4])
        finished = self.scheduler.settle_in_flight(drawn) if ahead is not None else self.scheduler.settle_rows(drawn)
        self._launched = ahead
        s = self.stats
        s.steps += 1
        s.step_batch_sizes.append(step.items)
        s.computed_tokens += step.tokens
        s.generated_tokens += int(self.core.counters()[4]) - before
        return finished

    def _step_timed(self) -> list[Sequence]:
        """A step with the device awaited after each phase, its time added to the stats (no step ahead)."""
        if self._launched is not None:  # a step launched ahead before the timing was switched on: settled untimed
            step, self._launched = self._launched, None
            finished = self.scheduler.settle_rows(self.runner.draw(step.rows, step.tempered, step.replay))
            self.stats.steps += 1
            self.stats.step_batch_sizes.append(step.items)
            self.stats.computed_tokens += step.tokens
            self.stats.generated_tokens += step.rows
            return finished
        clock = _PhaseClock(self.stats.phase_seconds)
        if self.core.plan() == 0:
            raise RuntimeError("scheduler produced an empty batch with work pending")
        tokens, items, rows, *_, warm = (int(v) for v in self.core.step_summary())
        clock.lap("schedule")
        self.runner.run_planned()
        clock.lap("forward")
        drawn = self.runner.draw(rows, bool(warm))
        clock.lap("sample")
        finished = self.scheduler.settle_rows(drawn)
        s = self.stats
        s.steps += 1
        s.step_batch_sizes.append(items)
        s.computed_tokens += tokens
        s.generated_tokens += rows
        clock.lap("postprocess")
        return finished


@dataclass
class _Launched:
    """A step that runs on the device and whose draws have not been read."""

    tokens: int
    items: int
    rows: int
    tempered: bool
    replay: int | None  # the pinned buffer its draws are copied to, when it was replayed from a graph


class _PhaseClock:
    def __init__(self, totals: dict[str, float]):
        import time

        self._now, self.totals = time.perf_counter, totals
        torch.cuda.synchronize()
        self.t = self._now()

    def lap(self, phase: str) -> None:
        torch.cuda.synchronize()
        t = self._now()
        self.totals[phase] += t - self.t
        self.t = t
