"""Replay of the same requests under every way of cutting them, in float32 and bfloat16, on the
tiny configurations (C and D reach the matrix-core attention kernels in bfloat16, D with the head, group
and page sizes of the benchmark's model), compared with the plain implementation position by position:
whole; most in one step and the last 32 tokens one by one; portions of changing size down to two
tokens; mixed with other requests in a pool so small that pages are used again."""

from __future__ import annotations

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import trace_helpers as th
from conftest import BLOCK_SIZES, ROOT, random_prompt, tiny_configs

pytestmark = pytest.mark.gpu

LENGTHS = [5, 17, 33, 70, 150, 64, 2, 41]


def requests_for(name: str) -> dict[str, list[int]]:
    vocab = tiny_configs()[name].vocab_size
    return {f"r{i}": random_prompt(n, vocab, seed=100 * i + len(name)) for i, n in enumerate(LENGTHS)}


_sessions = {}


def session_for(folders, name: str, dtype: str, max_tokens: int):
    from mini_engine_amd.engine.trace import TraceSession, build_session

    key = (name, dtype, max_tokens)
    if key not in _sessions:
        _sessions[key] = TraceSession(build_session(folders[name], dtype, max_tokens, block_size=BLOCK_SIZES[name]))
    return _sessions[key]


_plain = {}
_rounded = {}


def plain_for(folders, name):
    if name not in _plain:
        _plain[name] = th.plain_logits(folders[name], requests_for(name))
    return _plain[name]


def rounded_for(folders, name):
    """The plain implementation with operands rounded where a bfloat16 engine rounds them."""
    import plain_qwen3 as plain

    if name not in _rounded:
        cfg, w = plain.read_config(folders[name]), plain.read_weights(folders[name])
        _rounded[name] = {rid: plain.forward_logits_rounded(w, cfg, toks) for rid, toks in requests_for(name).items()}
    return _rounded[name]


def worst_row(got: dict, want: dict) -> float:
    """The largest error of any row, as a share of that row's largest logit in ``want``."""
    return max(((got[r] - want[r]).abs().amax(-1) / want[r].abs().amax(-1)).max().item() for r in want)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E", "F"])
@pytest.mark.parametrize("mode", ["whole", "tail", "portions", "mixed"])
def test_replay_matches_plain(tiny_folders, name, dtype, mode):
    reqs = requests_for(name)
    max_tokens = 320  # 150 -> 192, plus two more 64s: a few requests live, pages used again and again
    steps = {"whole": th.whole, "tail": th.tail_one_by_one, "portions": th.portions,
             "mixed": lambda r: th.mixed(r, max_tokens, seed=7)}[mode](reqs)
    if mode == "mixed":
        assert max(len(s["entries"]) for s in steps) >= 3
        assert any(len(e["tokens"]) == 1 for s in steps for e in s["entries"]) and any(
            len(e["tokens"]) > 1 for s in steps if len(s["entries"]) > 1 for e in s["entries"])
    session = session_for(tiny_folders, name, dtype, max_tokens)
    got = th.collect(steps, th.replay_in_process(session, steps))
    want = plain_for(tiny_folders, name)
    for rid in reqs:
        th.assert_logits_close(got[rid], want[rid], dtype, f"{name} {dtype} {mode} request {rid}")
    if dtype == "bfloat16":
        # What bfloat16 itself costs on these weights and requests: the plain implementation with its operands rounded
        # where an engine holds them in bfloat16 (float32 sums). The engine may be that far from the true result and
        # little further. (It is as far from the rounded computation as that is from the true one, 0.6-1.4% of a row's
        # largest logit: a sum taken in another order flips roundings, which spread like the roundings themselves. So
        # the rounded computation bounds the engine's error by its size, not row by row. Measured excess: at most 0.15%.)
        rounded = rounded_for(tiny_folders, name)
        budget = worst_row({r: rounded[r] for r in reqs}, want)
        assert 0.004 < budget < 0.02, budget
        assert worst_row(got, {r: want[r] for r in reqs}) <= budget + 0.003, (name, mode, worst_row(got, want), budget)
    bm = session.bm
    assert all(len(p.free_pool) == p.num_blocks for p in bm.pools), "every page must be back in the pool"
    assert session.engine.runner.graph_replays > 0 or mode in ("whole", "portions")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E", "F"])
def test_modes_agree_with_each_other_beyond_rounding(tiny_folders, name, dtype):
    """The logits at a position do not depend on the cut: compare the modes directly, row by row
    (float32: the same sums in the same order, so nearly the same bits; bfloat16: the kernels of
    prompts and of decoded tokens round at different places, measured 1.1-1.8% of a row's largest
    logit)."""
    reqs = requests_for(name)
    session = session_for(tiny_folders, name, dtype, 320)
    results = []
    for build in (th.whole, th.tail_one_by_one, th.portions, lambda r: th.mixed(r, 320, seed=3)):
        steps = build(reqs)
        results.append(th.collect(steps, th.replay_in_process(session, steps)))
    tol = 2e-5 if dtype == "float32" else 0.02
    for other in results[1:]:
        for rid in reqs:
            err = (other[rid] - results[0][rid]).abs().max(dim=-1).values
            scale = results[0][rid].abs().max(dim=-1).values
            assert (err <= tol * scale).all(), (name, rid, (err / scale).max().item())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["C", "D"])
def test_long_contexts_in_portions_and_decoded(tiny_folders, name, dtype):
    """Thousands of keys: a 3,000-token request in portions of 512 (from the second on a short run of queries behind a
    long context: the prefill attention cuts its tiles into key ranges and a second kernel adds them up; in float32 a
    run's tiles of keys are shared in LDS over a dozen chunks of 256), a 1,500-token request that joins it in portions
    of 700, and the last eight tokens of both decoded one by one, side by side (many splits of a long context per
    item; in float32 eight waves that take a token's chunks in turns). Logits are taken at the end of every portion, at a
    few places inside, and at every decoded token."""
    vocab = tiny_configs()[name].vocab_size
    reqs = {"long": random_prompt(3000, vocab, seed=31), "mid": random_prompt(1500, vocab, seed=32)}
    cuts = {"long": [512] * 5 + [432] + [1] * 8, "mid": [0, 0, 700, 700, 92] + [0] + [1] * 8}
    steps, done = [], {"long": 0, "mid": 0}
    for i in range(len(cuts["long"])):
        entries = []
        for rid in ("long", "mid"):
            n = cuts[rid][i]
            if n:
                want = sorted({0, n // 3, n - 1})
                entries.append({"id": rid, "tokens": reqs[rid][done[rid]:done[rid] + n], "want": want, "at": [done[rid] + j for j in want]})
                done[rid] += n
        steps.append({"step": i, "entries": entries, "end": [rid for rid in reqs if done[rid] == len(reqs[rid]) and cuts[rid][i]]})
    assert done == {"long": 3000, "mid": 1500}
    from mini_engine_amd.engine.trace import TraceSession, build_session

    session = TraceSession(build_session(tiny_folders[name], dtype, 3008 + 1536, block_size=BLOCK_SIZES[name]))
    want = th.plain_logits(tiny_folders[name], reqs)
    for st in steps:
        out = torch.from_numpy(session.run_step({k: ([{kk: vv for kk, vv in e.items() if kk != "at"} for e in v] if k == "entries" else v)
                                                 for k, v in st.items()}).copy())
        r = 0
        for e in st["entries"]:
            th.assert_logits_close(out[r:r + len(e["at"])], want[e["id"]][e["at"]], dtype, f"{name} {dtype} step {st['step']} {e['id']}")
            r += len(e["at"])
        assert r == out.shape[0]
    assert not session.live


@pytest.mark.parametrize("name", ["C", "D"])
def test_one_long_request_decoded_alone(tiny_folders, name):
    """One item a step behind a context of 1,500: decode attention in two dozen splits, which the output projection
    adds up itself at these widths (no kernel of its own does; tests/test_product_choice.py says that these models take
    that path). The last twelve tokens one by one, every one's logits against the plain implementation."""
    vocab = tiny_configs()[name].vocab_size
    reqs = {"solo": random_prompt(1500, vocab, seed=33)}
    from mini_engine_amd.engine.trace import TraceSession, build_session

    session = TraceSession(build_session(tiny_folders[name], "bfloat16", 1536, block_size=BLOCK_SIZES[name]))
    want = th.plain_logits(tiny_folders[name], reqs)
    out = torch.from_numpy(session.run_step({"step": 0, "entries": [{"id": "solo", "tokens": reqs["solo"][:1488], "want": [1487]}],
                                             "end": []}).copy())
    th.assert_logits_close(out, want["solo"][[1487]], "bfloat16", f"{name} prompt")
    for i in range(1488, 1500):
        out = torch.from_numpy(session.run_step({"step": i, "entries": [{"id": "solo", "tokens": [reqs["solo"][i]], "want": [0]}],
                                                 "end": ["solo"] if i == 1499 else []}).copy())
        th.assert_logits_close(out, want["solo"][[i]], "bfloat16", f"{name} token {i}")
    assert not session.live


def test_first_tokens_of_a_sequence(tiny_folders):
    """Positions 0 and 1 alone: a one-token prompt, then its second token."""
    for name in ("A", "B"):
        toks = requests_for(name)["r3"][:2]
        steps = [{"step": 0, "entries": [{"id": "x", "tokens": toks[:1], "want": [0]}], "end": []},
                 {"step": 1, "entries": [{"id": "x", "tokens": toks[1:], "want": [0]}], "end": ["x"]}]
        for dtype in ("float32", "bfloat16"):
            session = session_for(tiny_folders, name, dtype, 320)
            got = th.collect(steps, th.replay_in_process(session, steps))["x"]
            want = th.plain_logits(tiny_folders[name], {"x": toks})["x"]
            th.assert_logits_close(got, want, dtype, f"{name} {dtype} first tokens")


def test_wanting_nothing_writes_nothing_and_still_fills_the_cache(tiny_folders):
    name, dtype = "A", "float32"
    toks = requests_for(name)["r2"]
    session = session_for(tiny_folders, name, dtype, 320)
    steps = [{"step": 0, "entries": [{"id": "q", "tokens": toks[:20], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "q", "tokens": toks[20:], "want": [len(toks) - 21]}], "end": ["q"]}]
    assert session.run_step(steps[0]) is None
    last = torch.from_numpy(session.run_step(steps[1]))
    want = th.plain_logits(tiny_folders[name], {"q": toks})["q"][-1:]
    th.assert_logits_close(last, want, dtype, "last row after a silent first portion")


def test_trace_run_program(tiny_folders, tmp_path):
    """The program itself, as a child process: stdin steps, `done <step>` lines, .f32 files."""
    name = "A"
    reqs = {k: v for k, v in list(requests_for(name).items())[:4]}
    steps = th.mixed(reqs, 256, seed=1)
    steps[0]["entries"][0]["want"] = []  # a step's entry may want nothing
    silent_first = all(not e["want"] for e in steps[0]["entries"])
    for dtype in ("float32", "bfloat16"):
        out_dir = tmp_path / dtype
        proc = subprocess.run(
            [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", tiny_folders[name], "--dtype", dtype,
             "--out", str(out_dir), "--max-tokens", "256"],
            input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=300)
        assert proc.returncode == 0, proc.stderr[-2000:]
        assert proc.stdout.split("\n")[: len(steps)] == [f"done {s['step']}" for s in steps]
        vocab = tiny_configs()[name].vocab_size
        outputs = {}
        for s in steps:
            path = out_dir / f"{s['step']}.f32"
            wanted = sum(len(e["want"]) for e in s["entries"])
            assert path.exists() == (wanted > 0)
            if wanted:
                outputs[s["step"]] = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(wanted, vocab))
        if silent_first:
            assert 0 not in outputs
        want = th.plain_logits(tiny_folders[name], reqs)
        # compare every wanted row with the plain logits at its position
        fed = {rid: 0 for rid in reqs}
        for s in steps:
            r = 0
            for e in s["entries"]:
                for w in e["want"]:
                    th.assert_logits_close(outputs[s["step"]][r : r + 1], want[e["id"]][fed[e["id"]] + w][None], dtype,
                                           f"program {dtype} step {s['step']} {e['id']}")
                    r += 1
                fed[e["id"]] += len(e["tokens"])


def test_trace_run_program_with_a_shape_and_a_seed(tmp_path):
    """``--random-shape ARCH:keys --seed`` stands for ``--model``, ``--block-size`` and ``--num-blocks``
    size the pool: Tiny B (pages of 8) replayed from the command line, mixed, in a pool of 40 pages."""
    from mini_engine_amd.weights import random_model_folder

    cfg = tiny_configs()["B"]
    keys = cfg.to_config_json()
    shape = "Qwen3ForCausalLM:" + ",".join(
        f"{k}={json.dumps(keys[k])}" for k in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                                               "num_attention_heads", "num_key_value_heads", "head_dim", "rms_norm_eps",
                                               "rope_theta", "max_position_embeddings", "tie_word_embeddings"))
    reqs = {k: v for k, v in list(requests_for("B").items())[:5]}
    steps = th.mixed(reqs, 320, seed=2)
    want = th.plain_logits(random_model_folder(shape, 13, "float32"), reqs)
    out_dir = tmp_path / "out"
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--random-shape", shape, "--seed", "13", "--dtype", "float32",
         "--out", str(out_dir), "--block-size", "8", "--num-blocks", "40"],
        input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    fed = {rid: 0 for rid in reqs}
    for s in steps:
        wanted = sum(len(e["want"]) for e in s["entries"])
        got = torch.from_numpy(np.fromfile(out_dir / f"{s['step']}.f32", dtype="<f4").reshape(wanted, cfg.vocab_size))
        r = 0
        for e in s["entries"]:
            n = len(e["tokens"])
            th.assert_logits_close(got[r : r + n], want[e["id"]][fed[e["id"]] : fed[e["id"]] + n], "float32",
                                   f"step {s['step']} {e['id']}")
            r += n
            fed[e["id"]] += n
