"""The step function: run a batch of (request, next tokens) through the model from the cache and
return the logits at the wanted places.

:class:`ModelRunner` owns the decoder, the cache storage and the native host core (requests, page
pools, scheduler, step packing). A step runs only the tokens it is given: portions of prompts beside
single decoded tokens, cut anywhere (reference: ``src/mini_engine/engine.py:158-226``). Steps in
which every item is one decoded token can be replayed from a HIP graph captured per batch-size
bucket (reference: ``src/mini_engine/cuda_graphs.py``): the graph reads its indices from one static
buffer whose pinned source the core refills in place before each replay.

Every model's forward pass is a native step program: a step is one call into C++ (check, pack, upload,
every kernel, the draw of the next tokens), which calls back into a part's own ``forward`` where a part
brings code of its own.
"""

from __future__ import annotations

import weakref

import torch

from ..cache.block_manager import BlockManager
from ..cache.storage import CacheStorage, plan_layout
from ..config.engine_config import EngineConfig
from ..parts.decoder import Decoder
from ..sampling.sampler import Sampler
from .batch import StepBatch, StepItem
from .core import HostCore, step_layout
from .program import StepMemory, StepProgram, run_static, run_step

TORCH_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


_capture_state_holder = None


def _ordinary_capture_state(device) -> None:
    """torch keeps the random generator's capture state in tensors that it makes at the first capture of a
    process and updates in place at every later one, for as long as any graph lives. Steps run under inference
    mode: made there, those tensors would refuse the update when someone captures a graph outside inference
    mode while an engine's graphs are alive. A first small capture outside inference mode makes them ordinary
    tensors, and its graph is kept so that they stay."""
    global _capture_state_holder
    if _capture_state_holder is None:
        with torch.inference_mode(False):
            cell = torch.zeros(1, device=device)
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                cell += 1
            torch.cuda.current_stream().wait_stream(side)
        _capture_state_holder = (graph, cell)


def batch_buckets(max_batch: int) -> list[int]:
    """Batch sizes a decode graph is captured for: 1, 2, 4, 8 below the cap, then every 16, then the
    cap itself (reference: ``cuda_graphs.py:28-30``)."""
    buckets = [b for b in (1, 2, 4, 8) if b < max_batch]
    buckets += range(16, max_batch, 16)
    return buckets + [max_batch]


class ModelRunner:
    def __init__(self, decoder: Decoder, config: EngineConfig, eos_token_ids=()):
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU is visible: this engine runs on the GPU only")
        self.decoder, self.config = decoder, config
        self.device = decoder.device
        self.dtype = decoder.dtype
        self.layout = plan_layout(decoder)
        # slots exist only for models whose layers keep per-request state
        self.num_state_slots = config.max_num_seqs if self.layout.has_state else 0
        self.storage = CacheStorage(decoder, self.layout, config.num_blocks, config.block_size,
                                    self.num_state_slots, self.dtype, self.device)
        self.num_groups = len(self.layout.groups)
        self.max_blocks_per_seq = -(-config.max_model_len // config.block_size)
        self.core = HostCore(config.block_size, [(g.window, g.num_blocks or config.num_blocks) for g in self.layout.groups],
                             config.enable_prefix_caching, self.num_state_slots, self.layout.has_state, config.max_num_seqs,
                             config.max_num_batched_tokens, config.max_model_len, eos_token_ids, config.seed)
        self.program = StepProgram(self.dtype, decoder.plan.hidden_size, decoder.plan.vocab_size, config.max_model_len)
        decoder.emit(self.program)
        batch_of_step = weakref.WeakMethod(self._batch_of_running_step)  # (no cycle: a dropped runner frees its graphs at once)
        self.program.current_batch = lambda: batch_of_step()()
        self.memory = StepMemory(self.program, self.device, [self.max_blocks_per_seq] * self.num_groups,
                                 self.storage.spare_block, self.storage.spare_slot)
        self.sampler = Sampler()
        self.graph_safe = decoder.graph_safe()  # every part can be captured: decode steps may replay graphs
        self._graphs: dict[int, tuple] = {}
        self._graph_pool = None
        self._static_arena: torch.Tensor | None = None
        self._copy_done: dict[int, torch.cuda.Event] = {}
        self.batch: StepBatch | None = None  # the running step's batch, for parts that are called (made when first asked for)
        self._logits: torch.Tensor | None = None
        self._drawn: torch.Tensor | None = None  # what the native program drew for the last step's rows
        # Replayed steps of a native program draw into one buffer on the device, from which the next replay may
        # take its token ids; every replay is followed by a copy of its draws into pinned memory (two buffers in
        # turn: a step planned ahead is launched before the draws of the step before it are read).
        self._fed = torch.zeros(max(config.max_num_seqs, 1), dtype=torch.int32, device=self.device)
        self._fed_host = [torch.zeros(max(config.max_num_seqs, 1), dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self._fed_done = [torch.cuda.Event(), torch.cuda.Event()]
        self._fed_turn = 0
        self.last_replay: int | None = None  # which pinned buffer holds the draws of the last step, if it was replayed
        self.graph_replays = 0
        self.eager_steps = 0

    def new_block_manager(self) -> BlockManager:
        c = self.config
        return BlockManager(c.num_blocks, c.block_size, c.enable_prefix_caching, self.layout.groups,
                            num_state_slots=self.num_state_slots, has_state=self.layout.has_state, core=self.core)

    # ------------------------------------------------------------------------------------ step
    def step(self, items: list[StepItem]) -> torch.Tensor:
        """Logits float32 [R, V]: for every item in order, for every place in its ``want``.

        The result lies in memory that the next step uses again: read it before the next step."""
        core = self.core
        core.step_clear()
        try:
            for it in items:
                it.seq.bind(core)
                n = len(it.tokens)
                if it.start < 0 or it.start + n > len(it.seq) or it.seq.tokens(it.start, n) != [int(t) for t in it.tokens]:
                    raise ValueError("an item's tokens must be its request's tokens at the item's positions")
                core.step_add(it.seq._handle, it.start, n, it.want)
            return self.run_planned()
        finally:
            core.step_clear()

    @torch.inference_mode()
    def run_planned(self) -> torch.Tensor:
        """Run the step that the core holds (planned by the scheduler or listed by :meth:`step`)."""
        core = self.core
        tokens, items, rows, longest, ctx, decode_only, last_only, _ = (int(v) for v in core.step_summary())
        replay = bool(self.config.cuda_graphs and self.graph_safe and decode_only and last_only
                      and 0 < items <= self.config.max_num_seqs)
        self._drawn = None
        self.last_replay = None
        if replay:
            # a replayed step checks the pages of its block tables while they are written into the graph's buffer
            core.step_check(self.decoder.plan.vocab_size, scan_pages=False)
            self._zero_fresh_state()
            return self._replay(items)
        self.eager_steps += 1
        self._logits = self._run_eager(tokens, items, rows, ctx)
        return self._logits

    def _run_eager(self, tokens: int, items: int, rows: int, ctx: int) -> torch.Tensor:
        """The step that the core holds as one call: check, pack, upload, every kernel, the draw."""
        core, c = self.core, self.config
        self.memory.ensure(max(tokens, c.max_num_batched_tokens), max(items, c.max_num_seqs), max(rows, c.max_num_seqs),
                           max(ctx, c.max_model_len))
        if self.layout.has_state:
            core.step_check(self.decoder.plan.vocab_size, scan_pages=True)  # before anything is written
            self._zero_fresh_state()
        self.batch = None
        logits, self._drawn, _ = run_step(self.program, self.memory, core)
        if logits is None:
            logits = torch.empty((0, self.decoder.plan.vocab_size), dtype=torch.float32, device=self.device)
        return logits

    def _batch_of_running_step(self) -> StepBatch:
        """What a called part gets as the step's batch: views into the index buffer that the running step uploaded
        (an eager step: made at the first call of the step) or the buffer a graph was captured on."""
        if self.batch is None:
            core, index = self.core, self.memory.index
            _, starts, counts, _, slots = core.step_items()
            self.batch = StepBatch(index, core.step_layout()).describe(starts, counts, slots)
        return self.batch

    def _zero_fresh_state(self) -> None:
        """An item that starts at position 0 starts from a zero state, whoever held its slot before."""
        if self.layout.has_state:
            _, starts, _, _, slots = self.core.step_items()
            self.storage.zero_state([s for s, p0 in zip(slots, starts) if p0 == 0 and s >= 0])

    def draw(self, rows: int, tempered: bool, replay: int | None = None):
        """One token id per wanted row of a step (int32, on the host): what the step program drew beside the
        logits (a step without a draw of its own: the sampler's draw from them). ``replay`` names the pinned buffer
        of a replayed step (``last_replay`` right after it was launched); without it the last step is meant."""
        if rows == 0:
            return self.sampler.draw(None, None, 0, False)
        if replay is None:
            replay = self.last_replay
        if replay is not None:
            self._fed_done[replay].synchronize()
            return self._fed_host[replay][:rows].numpy().copy()
        if self._drawn is not None:
            return self._drawn[:rows].cpu().numpy()
        return self.sampler.draw(self._logits, self.batch, rows, tempered)

    # ---------------------------------------------------------------------------------- graphs
    def _forward_static(self, batch: StepBatch, bucket: int):
        """The launches of one decode step on a graph's static buffers: (logits, drawn or None)."""
        self.batch = batch  # what called parts see while the launches are recorded
        return run_static(self.program, self._static_arena, batch.buf, bucket, batch.widths, batch.max_ctx, batch.least_live,
                          drawn=self._fed, fed=True)

    def _capture(self, bucket: int):
        _ordinary_capture_state(self.device)
        widths = [self.max_blocks_per_seq] * self.num_groups
        layout = step_layout(bucket, bucket, bucket, widths)
        host = torch.empty(layout["total"], dtype=torch.int32, pin_memory=True)
        self.core.pack_padding(host.numpy(), widths, bucket, self.storage.spare_block, self.storage.spare_slot)
        self.core.forget_rows(bucket)
        buf = host.to(self.device)
        batch = StepBatch(buf, layout).describe([0] * bucket, [1] * bucket, [-1] * bucket)
        batch.max_ctx = self.config.max_model_len
        smaller = [b for b in batch_buckets(self.config.max_num_seqs) if b < bucket]
        batch.least_live = smaller[-1] + 1 if smaller else 1  # fewer items replay a smaller bucket's graph
        if self._static_arena is None:
            most = self.config.max_num_seqs  # every bucket's graph works in the same memory: replays are serial
            self._static_arena = torch.empty(self.program.arena_need(most, most, most, self.config.max_model_len),
                                             dtype=torch.uint8, device=self.device)
        fed = self._fed.clone()  # the warm-up run draws too: the draws of a step in flight are put back afterwards
        stream = torch.cuda.Stream()
        stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(stream):
            self._forward_static(batch, bucket)  # warm-up outside capture: loads code objects, sets up the GEMM library
        torch.cuda.current_stream().wait_stream(stream)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, pool=self._graph_pool):
            logits, drawn = self._forward_static(batch, bucket)
        self._graph_pool = graph.pool()
        self._fed.copy_(fed)
        torch.cuda.synchronize()
        self._graphs[bucket] = (graph, batch, host, logits, drawn)
        return self._graphs[bucket]

    @torch.inference_mode()
    def capture_all(self) -> None:
        """Capture every bucket, largest first so that smaller graphs fit into its memory pool."""
        for b in reversed(batch_buckets(self.config.max_num_seqs)):
            if b not in self._graphs:
                self._capture(b)

    def _replay(self, n: int) -> torch.Tensor:
        bucket = next(b for b in batch_buckets(self.config.max_num_seqs) if b >= n)
        graph, batch, host, logits, drawn = self._graphs.get(bucket) or self._capture(bucket)
        done = self._copy_done.get(bucket)
        if done is not None:
            done.synchronize()  # the previous upload from this pinned buffer has been read
        self.core.step_refill(bucket, host.numpy(), batch.widths, self.storage.spare_block, self.storage.spare_slot)
        batch.buf.copy_(host, non_blocking=True)
        done = done or torch.cuda.Event()
        done.record()
        self._copy_done[bucket] = done
        graph.replay()
        self.graph_replays += 1
        self.batch = batch
        self._logits = logits[:n]
        self._drawn = None if drawn is None else drawn[:n]
        if drawn is not None:  # the draws leave the device behind the graph, before a later replay overwrites them
            turn = self._fed_turn = self._fed_turn ^ 1
            self._fed_host[turn][:n].copy_(drawn[:n], non_blocking=True)
            self._fed_done[turn].record()
            self.last_replay = turn
        return self._logits
