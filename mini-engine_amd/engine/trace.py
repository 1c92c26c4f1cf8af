"""Trace replay: feed given token ids through the model step by step and write the logits.

It samples nothing and schedules nothing. It drives the same decoder, step function, cache manager
and kernels that generation uses: every step allocates pages for exactly the tokens it brings,
calls :meth:`ModelRunner.step`, and gives a request's pages back when the trace ends it.

Input (one JSON object a line)::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

Output: ``<out>/<step>.f32`` for every step that wants something (little-endian float32
``[wanted, vocab]``, in the order of the entries and of ``want``), and a line ``done <step>`` on
standard output after every step.
"""

from __future__ import annotations

import argparse
import json
import os
import sys

import numpy as np

PAGE_ROUNDING = 64  # a request's token count is rounded up to this for the --max-tokens bound


def build_session(model_dir: str, dtype: str, max_tokens: int, block_size: int = 16, max_live: int = 8,
                  cuda_graphs: bool = True):
    from ..config.engine_config import EngineConfig
    from ..ops.library import lib
    from .llm_engine import LLMEngine

    lib()  # compile (first call in a fresh checkout) or load the kernels before anything else
    if PAGE_ROUNDING % block_size:
        raise ValueError(f"block_size={block_size} must divide {PAGE_ROUNDING}")
    num_blocks = max(1, -(-max_tokens // block_size))
    config = EngineConfig(
        block_size=block_size,
        num_blocks=num_blocks,
        max_num_seqs=max_live,
        max_num_batched_tokens=max(max_tokens, 1),
        max_model_len=max(max_tokens, block_size),
        enable_prefix_caching=False,
        dtype=dtype,
        cuda_graphs=cuda_graphs,
    )
    return LLMEngine.from_pretrained(model_dir, config, progress=lambda m: print(f"[trace_run] {m}", file=sys.stderr, flush=True))


class TraceSession:
    def __init__(self, engine):
        from .batch import StepItem
        from .sequence import Sequence

        self._StepItem, self._Sequence = StepItem, Sequence
        self.engine = engine
        self.bm = engine.block_manager
        self.live: dict[str, object] = {}

    def run_step(self, record: dict) -> np.ndarray | None:
        """Run one step; returns the wanted logits as float32 [wanted, vocab], or None."""
        items = []
        touched = []
        for entry in record.get("entries", []):
            rid, tokens = str(entry["id"]), [int(t) for t in entry["tokens"]]
            want = [int(w) for w in entry.get("want", [])]
            if not tokens:
                raise ValueError(f"step {record.get('step')}: request {rid!r} brings no tokens")
            seq = self.live.get(rid)
            if seq is None:
                seq = self._Sequence(tokens)
                seq.token_ids = []
                self.live[rid] = seq
            start = seq.num_computed_tokens
            seq.token_ids.extend(tokens)
            if not self.bm.try_allocate(seq, start + len(tokens)):
                raise RuntimeError(
                    f"step {record.get('step')}: out of cache pages for request {rid!r} "
                    f"({self.bm.num_free_blocks} pages of {self.bm.block_size} tokens free); --max-tokens is too small")
            items.append(self._StepItem(seq, tokens, start, want))
            touched.append((seq, len(tokens)))
        out = None
        if items:
            logits = self.engine.runner.step(items)
            if logits.shape[0]:
                out = logits.float().cpu().numpy()
            for seq, n in touched:
                seq.num_computed_tokens += n
                self.bm.release_passed(seq)
        for rid in record.get("end", []):
            seq = self.live.pop(str(rid), None)
            if seq is not None:
                self.bm.free(seq)
        return out


def main(argv: list[str] | None = None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder the logits files are written to")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64); sizes the cache pool")
    args = ap.parse_args(argv)
    os.makedirs(args.out, exist_ok=True)
    print("[trace_run] loading kernels and model", file=sys.stderr, flush=True)
    session = TraceSession(build_session(args.model, args.dtype, args.max_tokens))
    print("[trace_run] ready", file=sys.stderr, flush=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step = record["step"]
        out = session.run_step(record)
        if out is not None:
            out.astype("<f4", copy=False).tofile(os.path.join(args.out, f"{step}.f32"))
        print(f"done {step}", flush=True)
    return 0
