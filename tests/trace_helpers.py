"""Builders of replay traces (the JSON steps bin/trace_run reads) for the ways of cutting the same
requests, and the comparison of the replayed logits with the plain implementation."""

from __future__ import annotations

import random

import torch

import plain_qwen3 as plain


def round_up(n: int, m: int = 64) -> int:
    return -(-n // m) * m


def whole(requests: dict[str, list[int]]) -> list[dict]:
    """Each request alone and whole, one step each."""
    return [{"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]}
            for i, (rid, toks) in enumerate(requests.items())]


def tail_one_by_one(requests: dict[str, list[int]], tail: int = 32) -> list[dict]:
    """Most of a request in one step, then its last ``tail`` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        head = max(len(toks) - tail, 1)
        cuts = [(0, head)] + [(p, p + 1) for p in range(head, len(toks))]
        for j, (lo, hi) in enumerate(cuts):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[lo:hi], "want": list(range(hi - lo))}],
                          "end": [rid] if j == len(cuts) - 1 else []})
    return steps


def portions(requests: dict[str, list[int]], sizes=(7, 2, 13, 3, 2, 29, 5, 2, 64, 11)) -> list[dict]:
    """Portions of changing size, down to two tokens (the last portion takes what is left)."""
    steps = []
    for k, (rid, toks) in enumerate(requests.items()):
        lo, i = 0, k
        while lo < len(toks):
            hi = min(lo + sizes[i % len(sizes)], len(toks))
            if len(toks) - hi == 1:  # never leave a single token for a last "portion"
                hi = len(toks)
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[lo:hi], "want": list(range(hi - lo))}],
                          "end": [rid] if hi == len(toks) else []})
            lo, i = hi, i + 1
    return steps


def mixed(requests: dict[str, list[int]], max_tokens: int, seed: int = 0, max_live: int = 4, tail: int = 12) -> list[dict]:
    """Up to four live requests: portions of some beside single decoded tokens of others, requests
    sitting out steps, and a pool so small (``max_tokens``) that pages of ended requests are used
    again by later ones. Live requests never hold more than ``max_tokens`` (each rounded up to 64)."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live: dict[str, int] = {}  # id -> tokens fed so far
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live and (
                sum(round_up(len(requests[r])) for r in live) + round_up(len(waiting[0][1])) <= max_tokens):
            live[waiting.pop(0)[0]] = 0
        assert live, "max_tokens is too small for the next request"
        entries, ended = [], []
        ids = list(live)
        rng.shuffle(ids)
        for rid in ids:
            if len(ids) > 1 and rng.random() < 0.25:
                continue  # sits this step out
            toks, fed = requests[rid], live[rid]
            left = len(toks) - fed
            n = 1 if left <= tail else min(rng.choice([2, 3, 5, 8, 17, 40]), left - tail)
            entries.append({"id": rid, "tokens": toks[fed : fed + n], "want": list(range(n))})
            live[rid] = fed + n
            if fed + n == len(toks):
                ended.append(rid)
        if not entries:
            continue
        steps.append({"step": len(steps), "entries": entries, "end": ended})
        for rid in ended:
            del live[rid]
    return steps


def collect(steps: list[dict], outputs: dict[int, torch.Tensor]) -> dict[str, torch.Tensor]:
    """{request id: logits [len, vocab]} from the per-step outputs, in position order."""
    rows: dict[str, list[torch.Tensor]] = {}
    for st in steps:
        out = outputs.get(st["step"])
        r = 0
        for e in st["entries"]:
            assert e["want"] == list(range(len(e["tokens"])))
            for _ in e["want"]:
                rows.setdefault(e["id"], []).append(out[r])
                r += 1
        assert out is None or r == out.shape[0]
    return {rid: torch.stack(v) for rid, v in rows.items()}


def replay_in_process(session, steps: list[dict]) -> dict[int, torch.Tensor]:
    outputs = {}
    for st in steps:
        out = session.run_step(st)
        if out is not None:
            outputs[st["step"]] = torch.from_numpy(out.copy())
    assert not session.live, "the trace must end every request"
    return outputs


def plain_logits(folder: str, requests: dict[str, list[int]]) -> dict[str, torch.Tensor]:
    cfg, w = plain.read_config(folder), plain.read_weights(folder)
    return {rid: plain.forward_logits(w, cfg, toks) for rid, toks in requests.items()}


def assert_logits_close(got: torch.Tensor, want: torch.Tensor, dtype: str, what: str = "") -> None:
    """float32: the reference's own parity tolerance (tests/test_parity.py:76), tightened.
    bfloat16, row by row: no element further off than 2% of that row's largest logit, and the row's
    root-mean-square error at most 1.5% of the row's root mean square (measured on the tiny
    configurations: 0.9-1.3% and 0.8-1.1%; the reference's tests/test_gpu.py:42 takes 2e-2 on
    attention alone)."""
    assert got.shape == want.shape, (what, got.shape, want.shape)
    err = (got - want).abs()
    if dtype == "float32":
        bad = (err > 5e-5 + 1e-4 * want.abs()).any(dim=-1)
    else:
        bad = (err.max(dim=-1).values > 0.02 * want.abs().max(dim=-1).values) | (
            err.pow(2).mean(dim=-1).sqrt() > 0.015 * want.pow(2).mean(dim=-1).sqrt())
    if bad.any():
        pos = int(bad.nonzero()[0])
        raise AssertionError(f"{what}: first wrong position {pos} of {got.shape[0]}, max abs error "
                             f"{err.max().item():.3e} (at that position {err[pos].max().item():.3e}, "
                             f"the row's largest logit {want[pos].abs().max().item():.3e})")
