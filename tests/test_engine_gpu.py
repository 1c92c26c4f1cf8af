"""Generation through the entry point (LLMEngine.generate) against the plain implementation: each
request alone, batched, with prefix-cache hits, under preemption, with a 7-token budget, with EOS,
long decoding through replayed graphs, temperature sampling, and the command line. The shapes of
these tests follow the reference's tests/test_parity.py (cited per test)."""

from __future__ import annotations

import os
import subprocess
import sys

import pytest
import torch

import plain_qwen3 as plain
from conftest import BLOCK_SIZES, ROOT, random_prompt, tiny_configs, write_tiny

pytestmark = pytest.mark.gpu

MAX_NEW = 16


@pytest.fixture(scope="module")
def peaked(tmp_path_factory):
    """The tiny configurations with a wide init (std 0.2), so that logits are peaked and float32
    rounding cannot flip an argmax (the reference's precaution, tests/conftest.py:25-27)."""
    out = {}
    for name, cfg in tiny_configs().items():
        folder = write_tiny(str(tmp_path_factory.mktemp(f"peaked_{name}")), cfg, seed=3, std=0.2, dtype=torch.float32)
        out[name] = (folder, plain.read_config(folder), plain.read_weights(folder))
    return out


def prompts_for(name: str, n: int = 8, lo: int = 1, hi: int = 45, seed: int = 1) -> list[list[int]]:
    g = torch.Generator().manual_seed(seed)
    lens = torch.randint(lo, hi + 1, (n,), generator=g).tolist()
    vocab = tiny_configs()[name].vocab_size
    return [torch.randint(1, vocab, (k,), generator=g).tolist() for k in lens]


def engine(folder, name, **over):
    from mini_engine_amd import EngineConfig, LLMEngine

    cfg = {"block_size": 4 if name == "A" else 8, "num_blocks": 256, "dtype": "float32", **over}
    return LLMEngine.from_pretrained(folder, EngineConfig(**cfg))


_reference = {}


def reference(peaked, name):
    if name not in _reference:
        folder, pcfg, w = peaked[name]
        _reference[name] = [plain.greedy_generate(w, pcfg, p, MAX_NEW) for p in prompts_for(name)]
    return _reference[name]


@pytest.mark.parametrize("name", ["A", "B"])
def test_unbatched_and_batched(peaked, name):  # test_parity.py:80-89
    from mini_engine_amd import SamplingParams

    want = reference(peaked, name)
    eng = engine(peaked[name][0], name, enable_prefix_caching=False)
    assert [eng.generate([p], SamplingParams(max_tokens=MAX_NEW))[0] for p in prompts_for(name)] == want
    eng = engine(peaked[name][0], name)
    assert eng.generate(prompts_for(name), SamplingParams(max_tokens=MAX_NEW)) == want
    assert max(eng.stats.step_batch_sizes) == 8
    assert eng.stats.generated_tokens == 8 * MAX_NEW and eng.runner.graph_replays > 0
    assert all(rc == 0 for rc in eng.block_manager.ref_counts)


@pytest.mark.parametrize("name", ["A", "B"])
def test_prefix_cache_hits_keep_parity(peaked, name):  # test_parity.py:92-104
    from mini_engine_amd import SamplingParams

    folder, pcfg, w = peaked[name]
    bs = 4 if name == "A" else 8
    system = prompts_for(name, 1, 23, 23, seed=7)[0]
    tails = prompts_for(name, 5, 1, 12, seed=8)
    prompts = [system + t for t in tails] + [system]
    want = [plain.greedy_generate(w, pcfg, p, MAX_NEW) for p in prompts]
    eng = engine(folder, name)
    first = eng.generate(prompts[:1], SamplingParams(max_tokens=MAX_NEW))
    rest = eng.generate(prompts[1:], SamplingParams(max_tokens=MAX_NEW))
    assert first + rest == want
    # every later prompt reuses the full blocks of the shared prefix; the bare system prompt too,
    # because its last token is the one that is recomputed
    assert eng.scheduler.num_cached_tokens == 5 * bs * ((23 - 1) // bs)


@pytest.mark.parametrize("name", ["A", "B"])
def test_preemption_keeps_parity(peaked, name):  # test_parity.py:107-112
    from mini_engine_amd import SamplingParams

    eng = engine(peaked[name][0], name, num_blocks=20 if name == "A" else 12)
    assert eng.generate(prompts_for(name), SamplingParams(max_tokens=MAX_NEW)) == reference(peaked, name)
    assert eng.scheduler.num_preemptions > 0
    assert all(rc == 0 for rc in eng.block_manager.ref_counts)


@pytest.mark.parametrize("name", ["A", "B"])
def test_chunked_prefill_keeps_parity(peaked, name):  # test_parity.py:115-119
    from mini_engine_amd import SamplingParams

    eng = engine(peaked[name][0], name, max_num_batched_tokens=7)
    assert eng.generate(prompts_for(name), SamplingParams(max_tokens=MAX_NEW)) == reference(peaked, name)
    assert eng.stats.steps > 30


def test_engine_stops_at_eos(peaked):  # test_parity.py:122-129
    from mini_engine_amd import SamplingParams

    name = "A"
    want = reference(peaked, name)
    eos = want[0][3]
    eng = engine(peaked[name][0], name, num_blocks=64)
    eng.scheduler.eos_token_ids = {eos}
    out = eng.generate([prompts_for(name)[0]], SamplingParams(max_tokens=MAX_NEW))[0]
    assert out == want[0][: want[0].index(eos) + 1]
    out = eng.generate([prompts_for(name)[0]], SamplingParams(max_tokens=MAX_NEW, ignore_eos=True))[0]
    assert out == want[0]


@pytest.mark.parametrize("graphs", [True, False])
def test_long_decoding(peaked, graphs):
    """300 tokens from a short prompt: many pages, several 64-key tiles, every step a replay."""
    from mini_engine_amd import SamplingParams

    name = "B"
    folder, pcfg, w = peaked[name]
    prompt = prompts_for(name)[2][:5]
    want = plain.greedy_generate(w, pcfg, prompt, 300)
    eng = engine(folder, name, cuda_graphs=graphs, max_model_len=512)
    got = eng.generate([prompt], SamplingParams(max_tokens=300))[0]
    assert got == want
    assert (eng.runner.graph_replays > 250) == graphs


@pytest.mark.parametrize("name", ["A", "C"])
def test_random_workload_is_the_same_replayed_and_eager(peaked, name):
    """Sixty requests of random lengths, some with a common prefix, through so few pages that requests
    are preempted and re-admitted, eight at a time: the float32 outputs of an engine that replays its
    decode steps from graphs (index buffer refilled in place, block-table rows extended or rewritten as
    sequences come, go and come back) equal those of an engine that runs every step eagerly, token by
    token, and every page is back in its pool at the end."""
    import random

    from mini_engine_amd import SamplingParams

    folder, pcfg, _ = peaked[name]
    rng = random.Random(5)
    shared = [rng.randrange(1, pcfg.vocab_size) for _ in range(48)]
    work = []
    for _ in range(60):
        p = [rng.randrange(1, pcfg.vocab_size) for _ in range(rng.choice([1, 2, 5, 17, 33, 64, 100]))]
        if rng.random() < 0.4:
            p = shared[: rng.choice([16, 32, 48])] + p
        work.append((p, rng.choice([1, 3, 8, 20, 45])))
    outs = {}
    for graphs in (True, False):
        eng = engine(folder, name, block_size=16, num_blocks=24, max_num_seqs=8, max_num_batched_tokens=96,
                     max_model_len=256, cuda_graphs=graphs)
        seqs = [eng.add_request(p, SamplingParams(max_tokens=m, temperature=0.0, ignore_eos=True)) for p, m in work]
        while eng.scheduler.has_unfinished():
            eng.step()
        outs[graphs] = [s.output_token_ids for s in seqs]
        assert all(len(o) == m for o, (_, m) in zip(outs[graphs], work))
        assert eng.scheduler.num_preemptions > 0 and eng.scheduler.num_cached_tokens > 0
        assert (eng.runner.graph_replays > 50) == graphs
        assert all(len(pool.free_pool) == pool.num_blocks for pool in eng.block_manager.pools)
    assert outs[True] == outs[False]


@pytest.mark.parametrize("name", ["C", "D"])
def test_arrivals_temperatures_and_end_tokens_in_every_mode(peaked, name):
    """Three hundred requests that arrive a few per step while others run, greedy and with two temperatures, half of
    them ending at an end token: an engine with graphs and steps launched ahead, one with neither, and one with so
    few pages and seats that it preempts all the time give every request the same tokens in float32 (a draw is
    keyed on seed, request and position, so temperature requests too)."""
    import random

    from mini_engine_amd import SamplingParams

    folder, pcfg, _ = peaked[name]
    rng = random.Random(17)
    shared = [rng.randrange(1, pcfg.vocab_size) for _ in range(64)]
    work = []
    for _ in range(300):
        p = [rng.randrange(1, pcfg.vocab_size) for _ in range(rng.choice([1, 2, 5, 17, 33, 64, 100, 130]))]
        if rng.random() < 0.4:
            p = shared[: rng.choice([16, 32, 48, 64])] + p
        work.append((p, rng.choice([1, 2, 3, 8, 20, 45, 60]), rng.choice([0.0, 0.0, 0.7, 1.3]), rng.random() < 0.5))
    outs = {}
    for mode, (graphs, ahead, seats, blocks) in {"fast": (True, True, 12, 40), "plain": (False, False, 12, 40),
                                                 "tight": (True, True, 5, 22)}.items():
        eng = engine(folder, name, block_size=16, num_blocks=blocks, max_num_seqs=seats, max_num_batched_tokens=112,
                     max_model_len=320, cuda_graphs=graphs, decode_ahead=ahead, seed=11)
        eng.scheduler.eos_token_ids = set(range(1, pcfg.vocab_size, 13))  # one id in thirteen ends a request
        arrivals = random.Random(3)
        seqs, pending = [], list(work)
        while pending or eng.scheduler.has_unfinished() or eng._launched:
            for _ in range(arrivals.choice([0, 1, 1, 2, 4])):
                if pending:
                    p, m, temp, ignore = pending.pop(0)
                    seqs.append(eng.add_request(p, SamplingParams(max_tokens=m, temperature=temp, ignore_eos=ignore)))
            if eng.scheduler.has_unfinished() or eng._launched:
                eng.step()
        outs[mode] = [list(s.output_token_ids) for s in seqs]
        assert all(len(pool.free_pool) == pool.num_blocks for pool in eng.block_manager.pools)
        assert eng.scheduler.num_preemptions > 0 and eng.scheduler.num_cached_tokens > 0
        assert (eng.runner.graph_replays > 100) == graphs
    assert outs["fast"] == outs["plain"] == outs["tight"]
    assert any(len(o) < m for o, (_, m, _, ignore) in zip(outs["fast"], work) if not ignore)  # some did end at an end token


def test_bfloat16_generation_stays_close(peaked):
    """bfloat16 cannot promise equal tokens (near-ties flip, reference DECISIONS.md:80-82): the first
    tokens agree, and each engine token is one the plain logits rank near the top."""
    from mini_engine_amd import SamplingParams

    for name in ("A", "B", "C", "D"):  # C, D: heads of 64 and 128, the matrix-core attention kernels
        folder, pcfg, w = peaked[name]
        eng = engine(folder, name, dtype="bfloat16", block_size=16)
        prompts = prompts_for(name)
        got = eng.generate(prompts, SamplingParams(max_tokens=MAX_NEW))
        want = reference(peaked, name)
        assert sum(g[0] == e[0] for g, e in zip(got, want)) >= 7
        for p, g in zip(prompts, got):
            logits = plain.forward_logits(w, pcfg, p + g)[len(p) - 1 : -1]
            chosen = logits.gather(1, torch.tensor(g)[:, None])[:, 0]
            assert ((logits.max(-1).values - chosen) <= 0.02 * logits.abs().max(-1).values).all()


def test_tiny_b_workload_with_temperature_and_shared_prefix(peaked):
    """Prompt lengths 1/9/16/31/50, two sharing a 16-token prefix (staged so that the second hits
    it), 12 tokens at temperature 0.8 from a fixed seed. A request's samples are keyed on (seed,
    request, token index), so the same tokens come out alone, batched, chunked and preempted."""
    from mini_engine_amd import EngineConfig, LLMEngine, SamplingParams
    from mini_engine_amd.engine.sequence import Sequence

    name = "B"
    folder, pcfg, w = peaked[name]
    vocab = tiny_configs()[name].vocab_size
    shared = random_prompt(16, vocab, 50)
    prompts = [random_prompt(1, vocab, 51), random_prompt(9, vocab, 52), shared,
               shared + random_prompt(15, vocab, 53), random_prompt(50, vocab, 54)]
    params = SamplingParams(max_tokens=12, temperature=0.8)

    def run(stage, **over):
        eng = LLMEngine.from_pretrained(folder, EngineConfig(**{"block_size": 8, "dtype": "float32", "seed": 5, **over}))
        outs = []
        for group in stage:
            outs += eng.generate([prompts[i] for i in group], params)
        return eng, [outs[sum(stage, []).index(i)] for i in range(5)]

    eng, base = run([[0, 1, 2], [3, 4]], num_blocks=64)
    assert all(len(o) == 12 for o in base)  # a sampled request yields exactly max_tokens tokens
    assert eng.scheduler.num_cached_tokens == 16  # request 3 hit the two full pages of request 2
    assert base != [plain.greedy_generate(w, pcfg, p, 12) for p in prompts]  # it does sample
    for p, o in zip(prompts, base):  # every sampled token is plausible under the plain distribution
        probs = plain.temperature_probs(plain.forward_logits(w, pcfg, p + o)[len(p) - 1 : -1], 0.8)
        assert (probs.gather(1, torch.tensor(o)[:, None]) > 1e-4).all()
    _, again = run([[0, 1, 2], [3, 4]], num_blocks=64)
    assert again == base  # fixed seed: repeatable
    _, chunked = run([[0, 1, 2], [3, 4]], num_blocks=64, max_num_batched_tokens=7)
    assert chunked == base
    eng, squeezed = run([[0, 1, 2], [3, 4]], num_blocks=11, max_num_batched_tokens=24)
    assert squeezed == base and eng.scheduler.num_preemptions > 0
    _, other_seed = run([[0, 1, 2], [3, 4]], num_blocks=64, seed=6)
    assert other_seed != base
    greedy = LLMEngine.from_pretrained(folder, EngineConfig(block_size=8, dtype="float32", num_blocks=64))
    assert greedy.generate(prompts, SamplingParams(max_tokens=12)) == [plain.greedy_generate(w, pcfg, p, 12) for p in prompts]


def test_tiny_a_workload(peaked):
    """Prompts 5/17/33, 8 greedy tokens; whole, token by token, in 7-token portions, mixed."""
    from mini_engine_amd import SamplingParams

    name = "A"
    folder, pcfg, w = peaked[name]
    vocab = tiny_configs()[name].vocab_size
    prompts = [random_prompt(n, vocab, 60 + n) for n in (5, 17, 33)]
    want = [plain.greedy_generate(w, pcfg, p, 8) for p in prompts]
    for over in ({}, {"max_num_batched_tokens": 1}, {"max_num_batched_tokens": 7}, {"max_num_seqs": 2}):
        eng = engine(folder, name, block_size=16, **over)
        assert eng.generate(prompts, SamplingParams(max_tokens=8)) == want, over


def test_pool_sized_by_a_share_of_the_memory(peaked):
    """``kv_memory_fraction`` instead of ``num_blocks``: the pool has the pages that fit into that share of the GPU's
    memory beside what is already on it, and generation is what it is with a pool of a given size."""
    from mini_engine_amd import SamplingParams
    from mini_engine_amd.engine.llm_engine import kv_cache_bytes_per_token

    free, total = torch.cuda.mem_get_info()
    share = (total - free + (64 << 20) + (1 << 30)) / total  # what is in use now, a step's workspaces and a gigabyte of pages
    eng = engine(peaked["A"][0], "A", kv_memory_fraction=share, num_blocks=1)
    page = kv_cache_bytes_per_token(eng.model.plan, "float32") * 4
    assert (1 << 29) // page <= eng.config.num_blocks <= (3 << 29) // page  # about a gigabyte of pages, whatever num_blocks said
    assert eng.block_manager.num_free_blocks == eng.config.num_blocks
    assert eng.generate(prompts_for("A"), SamplingParams(max_tokens=MAX_NEW)) == reference(peaked, "A")
    with pytest.raises(ValueError, match="no room"):
        engine(peaked["A"][0], "A", kv_memory_fraction=1e-6)


def test_requests_that_cannot_fit_are_refused(peaked):
    from mini_engine_amd import SamplingParams

    eng = engine(peaked["A"][0], "A", num_blocks=4, max_model_len=64)
    with pytest.raises(ValueError, match="KV blocks"):
        eng.add_request([1] * 14, SamplingParams(max_tokens=8))
    with pytest.raises(ValueError, match="max_model_len"):
        eng.add_request([1] * 60, SamplingParams(max_tokens=8))
    with pytest.raises(ValueError, match="vocabulary"):
        eng.add_request([1, 100000], SamplingParams(max_tokens=2))


def test_missing_library_fails_loudly(monkeypatch):
    """No fallback: when the kernels can be neither found nor built, the first op raises."""
    import mini_engine_amd.ops.library as library

    monkeypatch.setattr(library, "_lib", None)

    def broken():
        class M:
            LIB_NAME = "x.so"

            @staticmethod
            def default_lib_path():
                return "/nonexistent/libmini_engine_hip.so"

            @staticmethod
            def is_current(p):
                return False

            @staticmethod
            def build():
                raise RuntimeError("hipcc not found: the HIP kernels cannot be compiled")

        return M

    monkeypatch.setattr(library, "_build_module", broken)
    with pytest.raises(RuntimeError, match="cannot be compiled"):
        library.lib()


def test_command_line(peaked):
    folder = peaked["A"][0]
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "examples", "generate.py"), "--model", folder,
                           "--max-tokens", "6", "--dtype", "float32", "--prompt-ids", "5,6,7,8,9", "--prompt-ids", "5,6,7,8,9,10,11"],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    _, pcfg, w = peaked["A"]
    lines = [l for l in proc.stdout.splitlines() if l.startswith("A: ")]
    assert lines[0] == "A: " + " ".join(map(str, plain.greedy_generate(w, pcfg, [5, 6, 7, 8, 9], 6)))
    assert "tokens in" in proc.stdout and "served from prefix cache" in proc.stdout


def test_command_line_with_a_random_shape_and_random_prompts():
    """``--random ARCH:keys --seed`` stands for a model folder and ``--random-prompts NxLEN`` for prompts:
    the same seed gives the same text twice, another seed another, and the shared half of the prompts
    is served from the prefix cache."""
    shape = ("Qwen3ForCausalLM:vocab_size=211,hidden_size=48,intermediate_size=80,num_hidden_layers=2,num_attention_heads=3,"
             "num_key_value_heads=1,head_dim=16,rms_norm_eps=1e-6,rope_theta=10000.0,max_position_embeddings=256,"
             "tie_word_embeddings=true")

    def run(seed):
        proc = subprocess.run([sys.executable, os.path.join(ROOT, "examples", "generate.py"), "--random", shape, "--seed", str(seed),
                               "--random-prompts", "4x40", "--max-tokens", "5", "--dtype", "float32", "--block-size", "8"],
                              capture_output=True, text=True, timeout=300)
        assert proc.returncode == 0, proc.stderr[-2000:]
        return proc.stdout

    first = run(3)
    answers = [l for l in first.splitlines() if l.startswith("A: ")]
    assert len(answers) == 4 and all(len(a.split()) == 6 for a in answers)
    assert "served from prefix cache 48" in first  # 20 shared ids: two full pages of 8, three times
    assert [l for l in run(3).splitlines() if l.startswith("A: ")] == answers
    assert [l for l in run(4).splitlines() if l.startswith("A: ")] != answers


@pytest.mark.parametrize("name", ["A", "C"])
def test_steps_launched_ahead_change_no_token(peaked, name):
    """With ``decode_ahead`` the next decode step is launched before this step's tokens are read, its token
    ids fed on the device. Greedy and sampled generation, end tokens (a request that ends has run one token
    for nothing), a pool so small that requests are preempted, and graphs captured while a step is in
    flight (buckets shrink as requests end): the same tokens as with every step settled before the next."""
    from mini_engine_amd import EngineConfig, LLMEngine, SamplingParams

    folder, pcfg, w = peaked[name]
    prompts = prompts_for(name, n=11, hi=30, seed=5)
    want = [plain.greedy_generate(w, pcfg, p, 24) for p in prompts]
    eos = want[2][5]  # ends some requests early, others not at all
    outs = {}
    for ahead in (True, False):
        for kind, over, params in (("greedy", {}, SamplingParams(max_tokens=24)),
                                   ("sampled", {"seed": 3}, SamplingParams(max_tokens=17, temperature=0.9)),
                                   ("squeezed", {"num_blocks": 12}, SamplingParams(max_tokens=24))):
            eng = LLMEngine.from_pretrained(folder, EngineConfig(**{"block_size": 8, "num_blocks": 128, "dtype": "float32",
                                                                    "max_num_seqs": 16, "decode_ahead": ahead, **over}))
            eng.scheduler.eos_token_ids = {eos}
            outs[ahead, kind] = eng.generate(prompts, params)
            assert eng.runner.graph_replays > 0 and eng._launched is None
            assert eng.stats.generated_tokens == sum(len(o) for o in outs[ahead, kind])
            assert all(len(pool.free_pool) == pool.num_blocks for pool in eng.block_manager.pools)
            if kind == "squeezed":
                assert eng.scheduler.num_preemptions > 0
    cut = [o[: o.index(eos) + 1] if eos in o else o for o in want]
    assert outs[True, "greedy"] == outs[False, "greedy"] == cut
    assert outs[True, "squeezed"] == outs[False, "squeezed"] == cut
    assert outs[True, "sampled"] == outs[False, "sampled"] and outs[True, "sampled"] != [o[:17] for o in cut]
    assert any(eos in o for o in cut) and any(eos not in o for o in cut)


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "float32"), ("D", "bfloat16")])
def test_from_random_fills_every_tensor(tmp_path, name, dtype):
    """``LLMEngine.from_random`` (engine.py:136-141 there; the loader of every benchmark number here) draws its weights on
    the GPU, so they are other values than a model folder written for the same seed holds. The same source, asked
    tensor by tensor, gives the tensors to write a folder from; the plain implementation on that folder must agree
    with the engine: every wanted tensor was filled, the norm weights lie around 1, a tied head is the embedding."""
    import trace_helpers as th
    from mini_engine_amd import EngineConfig, LLMEngine, SamplingParams
    from mini_engine_amd.engine.batch import StepItem
    from mini_engine_amd.engine.sequence import Sequence
    from mini_engine_amd.weights import RandomSource
    from mini_engine_amd.weights.safetensors_io import write_file
    import json

    cfg = tiny_configs()[name]
    torch_dtype = torch.float32 if dtype == "float32" else torch.bfloat16
    eng = LLMEngine.from_random("Qwen3ForCausalLM", cfg, EngineConfig(block_size=BLOCK_SIZES[name], num_blocks=64, dtype=dtype,
                                                                      max_model_len=256), seed=5, std=0.2 if dtype == "float32" else 0.05)
    wants = eng.model.weight_wants()
    src = RandomSource(wants, 5, std=0.2 if dtype == "float32" else 0.05, device="cuda")
    tensors = {n: src.get(n).to(torch.float32 if wants[n].role == "vector" else torch_dtype).cpu() for n in wants}
    assert ("lm_head.weight" in tensors) == (not cfg.tie_word_embeddings)
    norms = [t for n, t in tensors.items() if wants[n].role == "vector"]
    assert norms and all(abs(t.mean().item() - 1) < 0.05 and 0 < t.std().item() < 0.05 for t in norms)
    folder = str(tmp_path)
    write_file(os.path.join(folder, "model.safetensors"), tensors, {"format": "pt"})
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg.to_config_json(), f)
    pcfg, w = plain.read_config(folder), plain.read_weights(folder)
    tokens = random_prompt(40, cfg.vocab_size, seed=2)
    want = plain.forward_logits(w, pcfg, tokens)
    seq = Sequence(tokens, core=eng.core)
    assert eng.block_manager.try_allocate(seq, len(tokens))
    got = eng.runner.step([StepItem(seq, tokens, 0, list(range(len(tokens))))]).float().cpu()
    eng.block_manager.free(seq)
    th.assert_logits_close(got, want, dtype, f"from_random {name} {dtype}")
    if dtype == "float32":
        assert eng.generate([tokens[:9]], SamplingParams(max_tokens=6))[0] == plain.greedy_generate(w, pcfg, tokens[:9], 6)


def test_someone_elses_graph_capture_beside_a_live_engine(peaked):
    """An engine captures its decode graphs under inference mode; a capture that other code starts outside
    inference mode while those graphs live must still work (torch updates the generator's capture state in place)."""
    from mini_engine_amd import SamplingParams

    eng = engine(peaked["A"][0], "A")
    eng.generate(prompts_for("A", 3), SamplingParams(max_tokens=4))
    assert eng.runner.graph_replays > 0
    x = torch.zeros(4, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        x += 1
    graph.replay()
    torch.cuda.synchronize()
    assert x.tolist() == [1.0] * 4  # (a capture records, it does not run)
    assert eng.generate(prompts_for("A", 2), SamplingParams(max_tokens=3)) is not None
