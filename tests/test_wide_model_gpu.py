"""One layer as wide as a large model's (hidden 5120 with 16 query heads, or hidden 4096 with 32; feed-forward 12288, 8 kv
heads of 128, 2,048 tokens in the vocabulary), in bfloat16, against the plain implementation: every projection's weight
has 16 MiB and more, which sends its products down other paths than the small layers of the other tests take. 40 short
prompts in one step (the GEMM library), then the requests decode side by side while most of them end: 40 rows (qkv and
gate/up in the library, o and down as partial sums of the weight-streaming kernel, down in blocks of 128 columns at hidden
5120; the head in the library), 24 rows (at hidden 4096, whose weights' rows lie a multiple of 4 KiB apart and whose
products fill whole rounds of blocks, qkv and gate/up in the weight-streaming kernel too), 10 rows (everything in that
kernel, the head too), 2 rows and 1 (the add-and-norm as that kernel's prologue)."""

from __future__ import annotations

import pytest

import trace_helpers as th
from conftest import random_prompt, write_tiny

pytestmark = pytest.mark.gpu

LIVE = [40, 40, 24, 24, 10, 10, 2, 2, 1]  # requests that decode in each step after the prompts


@pytest.fixture(scope="module", params=[(5120, 16), (4096, 32)], ids=["hidden5120", "hidden4096"])
def model(request, tmp_path_factory):
    from mini_engine_amd.models.qwen3 import Qwen3Config

    hidden, heads = request.param
    cfg = Qwen3Config(vocab_size=2048, hidden_size=hidden, intermediate_size=12288, num_hidden_layers=1,
                      num_attention_heads=heads, num_key_value_heads=8, head_dim=128, rms_norm_eps=1e-6,
                      rope_theta=1e6, max_position_embeddings=4096, tie_word_embeddings=True)
    folder = write_tiny(str(tmp_path_factory.mktemp("wide_model")), cfg, seed=7, std=0.02)
    reqs = {f"r{i:02d}": random_prompt(5 + (3 * i) % 8 + sum(1 for n in LIVE if n > i), cfg.vocab_size, seed=40 + i) for i in range(40)}
    return folder, reqs, th.plain_logits(folder, reqs), hidden


def steps_for(reqs):
    def entry(rid, lo, hi):
        return {"id": rid, "tokens": reqs[rid][lo:hi], "want": list(range(hi - lo))}

    fed = {rid: len(t) - sum(1 for n in LIVE if n > i) for i, (rid, t) in enumerate(reqs.items())}
    steps = [{"step": 0, "entries": [entry(rid, 0, fed[rid]) for rid in reqs], "end": []}]
    for j, n in enumerate(LIVE):
        live = list(reqs)[:n]
        entries = [entry(rid, fed[rid], fed[rid] + 1) for rid in live]
        for rid in live:
            fed[rid] += 1
        steps.append({"step": 1 + j, "entries": entries, "end": [rid for rid in live if fed[rid] == len(reqs[rid])]})
    assert all(fed[rid] == len(reqs[rid]) for rid in reqs)
    return steps


@pytest.mark.parametrize("path", ["replayed", "eager", "per kernel"])
def test_wide_layers_against_plain(model, path):
    """The step program, replayed and eager, and the same parts launched kernel by kernel from Python, whose products
    (``ops/kernels.py::linear``) ask the same rule for their kernel."""
    from types import SimpleNamespace

    from kernel_by_kernel import KernelByKernelRunner
    from mini_engine_amd.engine.trace import TraceSession, build_session
    from mini_engine_amd.ops import kernels as K

    folder, reqs, want, hidden = model
    # the paths this test is for: weights that count as bound by their streaming; at hidden 4096 the products of 24 rows that
    # the weight-streaming kernel takes from the library
    import torch

    units, bf16 = K.compute_units(), torch.bfloat16
    choice = lambda rows, rows_of_w, k, gated: K.product_choice(bf16, K.ROLE_PLAIN, rows, rows_of_w, k, gated, bf16, units)[0]
    assert choice(8, 2 * 12288, hidden, True) == K.PRODUCT_STREAM and choice(8, 2048, hidden, False) == K.PRODUCT_STREAM
    assert (choice(24, 2 * 12288, hidden, True) == K.PRODUCT_STREAM) == (hidden == 4096)
    assert choice(24, 6144, 4096, False) == K.PRODUCT_STREAM and choice(24, 5120, 4096, False) == K.PRODUCT_LIBRARY
    steps = steps_for(reqs)
    engine = build_session(folder, "bfloat16", 64 * 40, block_size=16, max_live=40, cuda_graphs=path == "replayed")
    if path == "per kernel":
        runner = KernelByKernelRunner(engine.model, engine.config)
        engine = SimpleNamespace(runner=runner, core=runner.core, block_manager=runner.new_block_manager())
    else:
        assert engine.runner.program is not None
    session = TraceSession(engine)
    got = th.collect(steps, th.replay_in_process(session, steps))
    for rid in reqs:
        th.assert_logits_close(got[rid], want[rid], "bfloat16", f"{path}: request {rid}")
    assert (engine.runner.graph_replays > 0) == (path == "replayed")
