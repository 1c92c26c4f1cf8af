"""The step function: run a batch of (request, next tokens) through the model from the cache and
return the logits at the wanted places.

:class:`ModelRunner` owns the decoder, the cache storage and the geometry of the page pools. A step
runs only the tokens it is given: portions of prompts beside single decoded tokens, cut anywhere
(reference: ``src/mini_engine/engine.py:158-226``). Steps in which every item is one decoded token
can be replayed from a HIP graph captured per batch-size bucket (reference:
``src/mini_engine/cuda_graphs.py``): the graph reads its indices from one static buffer that is
refilled with a single copy before each replay.
"""

from __future__ import annotations

import torch

from ..cache.block_manager import BlockManager
from ..cache.storage import CacheStorage, plan_layout
from ..config.engine_config import EngineConfig
from ..parts.decoder import Decoder
from .batch import StepBatch, StepItem, check_pages, make_batch, pack_host, section_offsets, validate_items

TORCH_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def batch_buckets(max_batch: int) -> list[int]:
    """Batch sizes a decode graph is captured for (reference: ``cuda_graphs.py:28-30``)."""
    small = [b for b in (1, 2, 4, 8) if b < max_batch]
    return small + list(range(16, max_batch, 16)) + [max_batch]


class ModelRunner:
    def __init__(self, decoder: Decoder, config: EngineConfig):
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU is visible: this engine runs on the GPU only")
        self.decoder, self.config = decoder, config
        self.device = decoder.device
        self.dtype = decoder.dtype
        self.layout = plan_layout(decoder)
        self.storage = CacheStorage(decoder, self.layout, config.num_blocks, config.block_size,
                                    config.max_num_seqs, self.dtype, self.device)
        self.num_groups = len(self.layout.groups)
        self.max_blocks_per_seq = -(-config.max_model_len // config.block_size)
        self._graphs: dict[int, tuple[torch.cuda.CUDAGraph, StepBatch, torch.Tensor, torch.Tensor]] = {}
        self._graph_pool = None
        self._copy_done: dict[int, torch.cuda.Event] = {}
        # per bucket and row: (sequence, its table_epoch, pages written per group) of the last replay
        self._rows: dict[int, list] = {}
        self.graph_replays = 0
        self.eager_steps = 0

    def new_block_manager(self) -> BlockManager:
        c = self.config
        return BlockManager(c.num_blocks, c.block_size, c.enable_prefix_caching, self.layout.groups,
                            num_state_slots=c.max_num_seqs, has_state=self.layout.has_state)

    # ------------------------------------------------------------------------------------ step
    @torch.inference_mode()
    def step(self, items: list[StepItem]) -> torch.Tensor:
        """Logits float32 [R, V]: for every item in order, for every place in its ``want``.

        After a replayed step the result is a view of the graph's output buffer: read it before the
        next step."""
        replay = self._graph_eligible(items)
        # a replayed step checks the pages of its block tables while it writes them into the graph's buffer
        validate_items(items, self.decoder.plan.vocab_size, self.config.block_size, self.layout.groups,
                       self.config.max_model_len, pages=not replay)
        if self.layout.has_state:
            self.storage.zero_state([it.seq.state_slot for it in items if it.start == 0 and it.seq.state_slot >= 0])
        if replay:
            return self._replay(items)
        self.eager_steps += 1
        batch = make_batch(items, self.num_groups, self.device, self.storage.spare_block, self.storage.spare_slot)
        return self.decoder.forward(batch)

    # ---------------------------------------------------------------------------------- graphs
    def _graph_eligible(self, items: list[StepItem]) -> bool:
        if not self.config.cuda_graphs or self.layout.has_state or len(items) > self.config.max_num_seqs:
            return False
        for it in items:
            if len(it.tokens) != 1 or it.want != [0]:
                return False
            if any(len(tb) > self.max_blocks_per_seq for tb in it.seq.block_tables):
                return False
        return True

    def _capture(self, bucket: int):
        widths = [self.max_blocks_per_seq] * self.num_groups
        total = section_offsets(bucket, bucket, bucket, widths)["_total"][1]
        host = torch.empty(total, dtype=torch.int32, pin_memory=True)
        arr, *_ = pack_host([], self.num_groups, widths, pad_items=bucket, spare_block=self.storage.spare_block,
                            spare_slot=self.storage.spare_slot)
        host.numpy()[:] = arr
        buf = host.to(self.device)
        batch = StepBatch(buf, bucket, bucket, bucket, widths)
        batch.starts, batch.qlens, batch.slots_host = [0] * bucket, [1] * bucket, [-1] * bucket
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

    def _refill(self, bucket: int, batch: StepBatch, host: torch.Tensor, items: list[StepItem]) -> None:
        """Write this step's indices into the bucket's pinned host buffer, which still holds the last
        replay's. Token, position, length and slot of every row are written anew. A row of a block
        table is only extended by the pages its sequence has gained when the row held the same
        sequence's table last time and nothing but appended pages has changed it since
        (``Sequence.table_epoch``); tables of window groups, whose entries change as pages are given
        back, are always written whole. Rows beyond the items point at the spare page and slot."""
        a = host.numpy()
        sec, n = batch.sections, len(items)
        rows = self._rows.setdefault(bucket, [None] * bucket)
        spare_block, spare_slot = self.storage.spare_block, self.storage.spare_slot
        tok_o, pos_o, ctx_o, slot_o = (sec[k][0] for k in ("token_ids", "positions", "item_ctx", "state_slots"))
        starts = [it.start for it in items]
        pad = bucket - n
        a[tok_o : tok_o + bucket] = [it.tokens[0] for it in items] + [0] * pad
        a[pos_o : pos_o + bucket] = starts + [0] * pad
        a[ctx_o : ctx_o + bucket] = [s + 1 for s in starts] + [1] * pad
        a[slot_o : slot_o + bucket] = [it.seq.state_slot if it.seq.state_slot >= 0 else spare_slot for it in items] + [spare_slot] * pad
        a[sec["live_items"][0]] = n
        bases = [sec[f"table{g}"][0] for g in range(self.num_groups)]
        windows = [g.window for g in self.layout.groups]
        for i, it in enumerate(items):
            seq, row = it.seq, rows[i]
            same = row is not None and row[0] is seq and row[1] == seq.table_epoch
            written = row[2] if same else [0] * self.num_groups
            rows[i] = None  # until the row is complete, should a check below raise
            need = it.start // self.config.block_size + 1
            for g, table in enumerate(seq.block_tables):
                w = batch.widths[g]
                o = bases[g] + i * w
                have = written[g] if same and windows[g] == 0 else -1
                if have < 0:
                    a[o : o + w] = spare_block
                    have = 0
                # pages this step reads or writes that were not checked when an earlier step wrote them
                first_key = max(0, it.start - windows[g] + 1) if windows[g] > 0 else 0
                check_pages(table, max(have, first_key // self.config.block_size), need, g)
                if have < len(table):
                    a[o + have : o + len(table)] = table[have:]
                    written[g] = len(table)
            rows[i] = (seq, seq.table_epoch, written)
        for i in range(n, bucket):
            if rows[i] is not None:
                for g in range(self.num_groups):
                    o = bases[g] + i * batch.widths[g]
                    a[o : o + batch.widths[g]] = spare_block
                rows[i] = None

    def _replay(self, items: list[StepItem]) -> torch.Tensor:
        n = len(items)
        bucket = next(b for b in batch_buckets(self.config.max_num_seqs) if b >= n)
        entry = self._graphs.get(bucket) or self._capture(bucket)
        graph, batch, host, logits = entry
        done = self._copy_done.get(bucket)
        if done is not None:
            done.synchronize()  # the previous upload from this pinned buffer has been read
        self._refill(bucket, batch, host, items)
        batch.buf.copy_(host, non_blocking=True)
        done = done or torch.cuda.Event()
        done.record()
        self._copy_done[bucket] = done
        graph.replay()
        self.graph_replays += 1
        return logits[:n]
