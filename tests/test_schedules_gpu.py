"""Schedules and sizes that the other files do not reach: the true 32-bit path at the layer sizes
and the vocabulary of the benchmark's model; a decode step of 80 live requests (more rows than the
small matrix-core product and the fused norm take); and bfloat16 generation with prefix-cache hits
and under preemption on the configurations whose attention runs on the matrix cores."""

from __future__ import annotations

import pytest
import torch

import plain_qwen3 as plain
import trace_helpers as th
from conftest import BLOCK_SIZES, random_prompt, tiny_configs, write_tiny

pytestmark = pytest.mark.gpu


def test_float32_at_the_benchmark_layer_sizes_and_vocabulary(tmp_path):
    """Hidden 1024, feed-forward 3072, 16/8 heads of 128, a vocabulary of 151,936, two layers, in
    float32: whole, and most in one step with the last 32 tokens one by one, against plain."""
    from mini_engine_amd.engine.trace import TraceSession, build_session
    from mini_engine_amd.models.qwen3 import Qwen3Config

    cfg = Qwen3Config(vocab_size=151936, hidden_size=1024, intermediate_size=3072, num_hidden_layers=2,
                      num_attention_heads=16, num_key_value_heads=8, head_dim=128, rms_norm_eps=1e-6,
                      rope_theta=1e6, max_position_embeddings=40960, tie_word_embeddings=True)
    folder = write_tiny(str(tmp_path / "model"), cfg, seed=21, std=0.03)
    reqs = {"a": random_prompt(75, cfg.vocab_size, seed=5)}
    want = th.plain_logits(folder, reqs)
    session = TraceSession(build_session(folder, "float32", 128, block_size=16, max_live=2))
    for build in (th.whole, th.tail_one_by_one):
        steps = build(reqs)
        got = th.collect(steps, th.replay_in_process(session, steps))
        th.assert_logits_close(got["a"], want["a"], "float32", f"float32 at the benchmark sizes, {build.__name__}")
    assert len({int(t) for t in want["a"].argmax(-1)}) > 10


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["C", "D"])
def test_eighty_requests_decode_side_by_side(tiny_folders, name, dtype):
    """80 prompts in one step, then five steps in which all 80 bring one token, replayed from a
    graph and run eagerly."""
    from mini_engine_amd.engine.trace import TraceSession, build_session

    vocab, extra = tiny_configs()[name].vocab_size, 5
    reqs = {f"q{i}": random_prompt(3 + (5 * i) % 23 + extra, vocab, seed=900 + i) for i in range(80)}
    want = th.plain_logits(tiny_folders[name], reqs)

    def entry(rid, lo, hi):
        return {"id": rid, "tokens": reqs[rid][lo:hi], "want": list(range(hi - lo))}

    steps = [{"step": 0, "entries": [entry(r, 0, len(t) - extra) for r, t in reqs.items()], "end": []}]
    for j in range(extra):
        steps.append({"step": 1 + j, "entries": [entry(r, len(t) - extra + j, len(t) - extra + j + 1) for r, t in reqs.items()],
                      "end": list(reqs) if j == extra - 1 else []})
    for graphs in (True, False):
        session = TraceSession(build_session(tiny_folders[name], dtype, 80 * 64, block_size=BLOCK_SIZES[name], max_live=80,
                                             cuda_graphs=graphs))
        got = th.collect(steps, th.replay_in_process(session, steps))
        for rid in reqs:
            th.assert_logits_close(got[rid], want[rid], dtype, f"{name} {dtype} graphs={graphs} request {rid}")
        assert (session.engine.runner.graph_replays == extra) == graphs


@pytest.fixture(scope="module")
def peaked(tmp_path_factory):
    """C and D with a wide init, so that logits are peaked (as tests/test_engine_gpu.py does)."""
    out = {}
    for name in ("C", "D"):
        cfg = tiny_configs()[name]
        folder = write_tiny(str(tmp_path_factory.mktemp(f"peaked16_{name}")), cfg, seed=4, std=0.2)
        out[name] = (folder, plain.read_config(folder), plain.read_weights(folder))
    return out


def assert_tokens_rank_first_beyond_rounding(weights, pcfg, prompt, output, what):
    """Every generated token is the plain logits' best one, or within bfloat16's rounding of it (2% of
    the row's largest logit): equal tokens cannot be promised where two logits nearly tie."""
    logits = plain.forward_logits(weights, pcfg, prompt + output)[len(prompt) - 1:-1]
    chosen = logits.gather(1, torch.tensor(output)[:, None])[:, 0]
    gap = logits.max(-1).values - chosen
    assert (gap <= 0.02 * logits.abs().max(-1).values).all(), (what, gap.max().item())


@pytest.mark.parametrize("name", ["C", "D"])
def test_bfloat16_generation_with_prefix_hits_and_preemption(peaked, name):
    """The same bfloat16 engine configuration runs every prompt alone (no prefix cache), then all
    of them with a shared prefix found in the cache, then in a pool so small that requests are
    preempted and recomputed. Every run's tokens rank first in the plain logits beyond rounding."""
    from mini_engine_amd import EngineConfig, LLMEngine, SamplingParams

    folder, pcfg, w = peaked[name]
    vocab = tiny_configs()[name].vocab_size
    system = random_prompt(37, vocab, seed=70)
    prompts = [system + random_prompt(2 + 3 * i, vocab, seed=71 + i) for i in range(6)] + [random_prompt(29, vocab, seed=80)]
    params = SamplingParams(max_tokens=12)

    def make(**over):
        return LLMEngine.from_pretrained(folder, EngineConfig(**{"block_size": 16, "num_blocks": 128, "dtype": "bfloat16",
                                                                 "max_num_seqs": 8, **over}))

    alone_engine = make(enable_prefix_caching=False)
    alone = [alone_engine.generate([p], params)[0] for p in prompts]
    cached_engine = make()
    cached = cached_engine.generate(prompts[:1], params) + cached_engine.generate(prompts[1:], params)
    assert cached_engine.scheduler.num_cached_tokens == 5 * 32  # two full pages of the shared prefix, five times
    squeezed_engine = make(num_blocks=14, enable_prefix_caching=False)
    squeezed = squeezed_engine.generate(prompts, params)
    assert squeezed_engine.scheduler.num_preemptions > 0
    assert all(len(pool.free_pool) == pool.num_blocks for pool in squeezed_engine.block_manager.pools)
    for p, a, c, s in zip(prompts, alone, cached, squeezed):
        # where two runs part, both tokens are within rounding of the best one at that place (the rows
        # of a prompt and of a decoded token round differently); from there on each follows its own text
        for run, out in (("alone", a), ("prefix hits", c), ("preempted", s)):
            assert len(out) == 12
            assert_tokens_rank_first_beyond_rounding(w, pcfg, p, out, f"{name} {run}")
    assert sum(a == c for a, c in zip(alone, cached)) + sum(a == s for a, s in zip(alone, squeezed)) >= 7  # most runs never meet a near-tie
