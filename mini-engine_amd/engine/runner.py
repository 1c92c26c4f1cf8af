"""The step function: run a batch of (request, next tokens) through the model from the cache and
return the logits at the wanted places.

:class:`ModelRunner` owns the decoder, the cache storage and the native host core (requests, page
pools, scheduler, step packing). A step runs only the tokens it is given: portions of prompts beside
single decoded tokens, cut anywhere (reference: ``src/mini_engine/engine.py:158-226``). Steps in
which every item is one decoded token can be replayed from a HIP graph captured per batch-size
bucket (reference: ``src/mini_engine/cuda_graphs.py``): the graph reads its indices from one static
buffer whose pinned source the core refills in place before each replay.
"""

from __future__ import annotations

import torch

from ..cache.block_manager import BlockManager
from ..cache.storage import CacheStorage, plan_layout
from ..config.engine_config import EngineConfig
from ..parts.decoder import Decoder
from .batch import StepBatch, StepItem, batch_from_core
from .core import HostCore, step_layout

TORCH_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


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
        self._graphs: dict[int, tuple[torch.cuda.CUDAGraph, StepBatch, torch.Tensor, torch.Tensor]] = {}
        self._graph_pool = None
        self._copy_done: dict[int, torch.cuda.Event] = {}
        self.batch: StepBatch | None = None  # the batch of the last step (its sampling inputs are read from it)
        self.graph_replays = 0
        self.eager_steps = 0

    def new_block_manager(self) -> BlockManager:
        c = self.config
        return BlockManager(c.num_blocks, c.block_size, c.enable_prefix_caching, self.layout.groups,
                            num_state_slots=self.num_state_slots, has_state=self.layout.has_state, core=self.core)

    # ------------------------------------------------------------------------------------ step
    def step(self, items: list[StepItem]) -> torch.Tensor:
        """Logits float32 [R, V]: for every item in order, for every place in its ``want``.

        After a replayed step the result is a view of the graph's output buffer: read it before the
        next step."""
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
        replay = bool(self.config.cuda_graphs and not self.layout.has_state and decode_only and last_only
                      and 0 < items <= self.config.max_num_seqs)
        # a replayed step checks the pages of its block tables while they are written into the graph's buffer
        core.step_check(self.decoder.plan.vocab_size, scan_pages=not replay)
        if self.layout.has_state:
            _, starts, _, _, slots = core.step_items()
            self.storage.zero_state([s for s, p0 in zip(slots, starts) if p0 == 0 and s >= 0])
        if replay:
            return self._replay(items)
        self.eager_steps += 1
        self.batch = batch_from_core(core, self.device, self.storage.spare_block, self.storage.spare_slot)
        return self.decoder.forward(self.batch)

    # ---------------------------------------------------------------------------------- graphs
    def _capture(self, bucket: int):
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
        stream = torch.cuda.Stream()
        stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(stream):
            self.decoder.forward(batch)  # warm-up outside capture: loads code objects, sets up the GEMM library
        torch.cuda.current_stream().wait_stream(stream)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, pool=self._graph_pool):
            logits = self.decoder.forward(batch)
        self._graph_pool = graph.pool()
        torch.cuda.synchronize()
        self._graphs[bucket] = (graph, batch, host, logits)
        return self._graphs[bucket]

    @torch.inference_mode()
    def capture_all(self) -> None:
        """Capture every bucket, largest first so that smaller graphs fit into its memory pool."""
        for b in reversed(batch_buckets(self.config.max_num_seqs)):
            if b not in self._graphs:
                self._capture(b)

    def _replay(self, n: int) -> torch.Tensor:
        bucket = next(b for b in batch_buckets(self.config.max_num_seqs) if b >= n)
        graph, batch, host, logits = self._graphs.get(bucket) or self._capture(bucket)
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
        return logits[:n]
