"""The layer sizes of the benchmark's model (hidden 1024, 16 query and 8 kv heads of 128, feed-forward
3072) with two layers and a small vocabulary, in bfloat16, against the plain implementation: the paths
that only such sizes reach. A 700-token prompt in one step (the tiled matrix-core GEMM with the SwiGLU
epilogue, prefill attention over whole tiles of different lengths), a 130-token prompt in a step of its own (the
gated product in the weight-streaming kernel, three groups of rows), 24 short prompts in one step, then
all 26 requests decoding side by side (17 to 64 rows: the weight-streaming products, projections as partial
sums over runs of k, the fused decode attention with its keys dealt to the splits), eagerly and as a
replayed graph."""

from __future__ import annotations

import pytest
import torch

import trace_helpers as th
from conftest import random_prompt, write_tiny

pytestmark = pytest.mark.gpu

EXTRA = 6  # tokens each request is fed one by one after its prompt


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    from mini_engine_amd.models.qwen3 import Qwen3Config

    cfg = Qwen3Config(vocab_size=512, hidden_size=1024, intermediate_size=3072, num_hidden_layers=2,
                      num_attention_heads=16, num_key_value_heads=8, head_dim=128, rms_norm_eps=1e-6,
                      rope_theta=1e6, max_position_embeddings=4096, tie_word_embeddings=True)
    folder = write_tiny(str(tmp_path_factory.mktemp("model_shape")), cfg, seed=5, std=0.03)
    reqs = {"long": random_prompt(700 + EXTRA, cfg.vocab_size, seed=1), "mid": random_prompt(130 + EXTRA, cfg.vocab_size, seed=2)}
    for i in range(24):
        reqs[f"s{i}"] = random_prompt(20 + (7 * i) % 41 + EXTRA, cfg.vocab_size, seed=10 + i)
    return folder, reqs, th.plain_logits(folder, reqs)


def steps_for(reqs):
    def entry(rid, lo, hi):
        return {"id": rid, "tokens": reqs[rid][lo:hi], "want": list(range(hi - lo))}

    steps = [{"step": 0, "entries": [entry("long", 0, len(reqs["long"]) - EXTRA)], "end": []},
             {"step": 1, "entries": [entry("mid", 0, len(reqs["mid"]) - EXTRA)], "end": []},
             {"step": 2, "entries": [entry(r, 0, len(t) - EXTRA) for r, t in reqs.items() if r not in ("long", "mid")], "end": []}]
    for j in range(EXTRA):
        steps.append({"step": 3 + j, "entries": [entry(r, len(t) - EXTRA + j, len(t) - EXTRA + j + 1) for r, t in reqs.items()],
                      "end": list(reqs) if j == EXTRA - 1 else []})
    return steps


@pytest.mark.parametrize("path", ["replayed", "eager", "per kernel"])
def test_benchmark_layer_sizes_against_plain(model, path):
    """The step program, replayed and eager, and the same parts launched kernel by kernel from Python."""
    from types import SimpleNamespace

    from kernel_by_kernel import KernelByKernelRunner
    from mini_engine_amd.engine.trace import TraceSession, build_session

    folder, reqs, want = model
    steps = steps_for(reqs)
    engine = build_session(folder, "bfloat16", 4096, block_size=16, max_live=32, cuda_graphs=path == "replayed")
    if path == "per kernel":
        runner = KernelByKernelRunner(engine.model, engine.config)
        engine = SimpleNamespace(runner=runner, core=runner.core, block_manager=runner.new_block_manager())
    session = TraceSession(engine)
    got = th.collect(steps, th.replay_in_process(session, steps))
    for rid in reqs:
        th.assert_logits_close(got[rid], want[rid], "bfloat16", f"{path}: request {rid}")
    assert (engine.runner.graph_replays > 0) == (path == "replayed")
    assert all(len(p.free_pool) == p.num_blocks for p in session.bm.pools)


def test_long_prompt_runs_wide_attention_blocks_and_agrees_with_narrow_ones(model):
    """A 4,200-token prompt gives every compute unit a block of 256 query columns, so the step takes
    the wide prefill attention blocks; its logits agree with those of the narrow blocks (which the
    test above holds against the plain implementation), and so does a later portion of 100 tokens
    whose tiles are cut into key ranges."""
    from mini_engine_amd.engine.trace import TraceSession, build_session
    from mini_engine_amd.ops import kernels as K

    folder, _, _ = model
    tokens = random_prompt(4300, 512, seed=77)
    steps = [{"step": 0, "entries": [{"id": "p", "tokens": tokens[:4200], "want": list(range(4190, 4200))}], "end": []},
             {"step": 1, "entries": [{"id": "p", "tokens": tokens[4200:], "want": list(range(90, 100))}], "end": ["p"]}]
    outs = {}
    chosen_limits = K.set_prefill_wide_limits(1e9, 1e9)
    try:
        for name, limits in {"narrow": (1e9, 1e9), "chosen": chosen_limits}.items():
            K.set_prefill_wide_limits(*limits)
            session = TraceSession(build_session(folder, "bfloat16", 4352, block_size=16, max_live=2, cuda_graphs=False))
            program = session.engine.runner.program
            assert program is not None
            outs[name], columns = [], []
            for step in steps:
                outs[name].append(torch.from_numpy(session.run_step(step).copy()))
                columns.append(program.last_prefill_columns)
            assert not session.live
            assert columns == ([256, 128] if name == "chosen" else [128, 128]), (name, columns)
    finally:
        K.set_prefill_wide_limits(*chosen_limits)
    for step in (0, 1):
        a, b = outs["chosen"][step], outs["narrow"][step]
        assert len({int(t) for t in a.argmax(-1)}) > 1
        th.assert_logits_close(a, b, "bfloat16", f"step {step}")
