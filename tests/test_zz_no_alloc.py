"""The sampling entry point that allocates nothing (``me_sample_static``), called through ctypes:
its tokens equal those of ``me_sample`` (which takes a workspace from the caller) on two calls in a
row, the second with a smaller input, and sizes beyond its static buffer are refused."""

from __future__ import annotations

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _lib():
    from mini_engine_amd.ops.library import lib

    L = lib()
    L.me_last_error.restype = ctypes.c_char_p
    return L


def _sample(L, logits, temps, keys, static: bool):
    r, v = logits.shape
    out = torch.full((r,), -1, dtype=torch.int32, device=logits.device)
    vp = ctypes.c_void_p
    stream = vp(torch.cuda.current_stream().cuda_stream)
    args = [vp(logits.data_ptr()), r, v, vp(temps.data_ptr() if temps is not None else None),
            vp(keys.data_ptr() if keys is not None else None), vp(out.data_ptr())]
    if static:
        code = L.me_sample_static(*args, stream)
    else:
        ws = torch.empty((r * L.me_sample_chunks(v) * 2,), dtype=torch.float32, device=logits.device)
        code = L.me_sample(*args, vp(ws.data_ptr()), stream)
    assert code == 0, L.me_last_error().decode()
    torch.cuda.synchronize()
    return out.cpu()


def host_scores(logits_row, temperature: float, key: int):
    """What the kernel maximises for a tempered row, from its definition and in float64: logit / max(t, 1e-5) + g_i with
    g_i = -log(-log(u_i)), u_i = (top 32 bits of mix64(key ^ mix64(i)) + 0.5) / 2^32."""
    import numpy as np

    def mix64(z):
        z = z + np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))

    with np.errstate(over="ignore"):
        h = mix64(np.uint64(key & (2**64 - 1)) ^ mix64(np.arange(len(logits_row), dtype=np.uint64)))
    u = np.minimum(((h >> np.uint64(32)).astype(np.float64) + 0.5) / 2.0**32, 0.99999994)
    return logits_row.astype(np.float64) / max(temperature, 1e-5) - np.log(-np.log(u))


def test_static_sampling_matches_the_workspace_entry_point_twice_in_a_row():
    L = _lib()
    gen = torch.Generator().manual_seed(5)
    # the second call is smaller in rows and in vocabulary: it uses a part of what the first one left
    for rows, vocab, tempered in ((40, 151936, True), (3, 5003, True), (7, 5003, False)):
        logits = torch.randn((rows, vocab), generator=gen).cuda()
        temps = keys = None
        if tempered:
            temps = torch.tensor([0.0 if i % 3 == 0 else 0.7 + 0.1 * i for i in range(rows)], dtype=torch.float32).cuda()
            keys = torch.randint(-2**62, 2**62, (rows,), generator=gen, dtype=torch.int64).cuda()
        want = _sample(L, logits, temps, keys, static=False)
        got = _sample(L, logits, temps, keys, static=True)
        assert torch.equal(got, want), (rows, vocab)
        greedy = [i for i in range(rows) if not tempered or i % 3 == 0]
        assert torch.equal(got[greedy].long(), logits.cpu().argmax(-1)[greedy])
        if tempered:  # the tempered rows against the definition of the draw, worked out on the host
            for i in [i for i in range(rows) if i % 3][:6]:
                scores = host_scores(logits[i].cpu().numpy(), float(temps[i]), int(keys[i]))
                assert scores[int(got[i])] >= scores.max() - 1e-4, (i, int(got[i]), int(scores.argmax()))
                assert int(got[i]) != int(logits[i].argmax()) or scores.argmax() == int(got[i])


def test_static_sampling_refuses_what_its_buffer_cannot_hold():
    L = _lib()
    rows = L.me_sample_static_max_pairs() // L.me_sample_chunks(151936) + 1
    logits = torch.zeros((rows, 151936), dtype=torch.float32, device="cuda")
    out = torch.zeros((rows,), dtype=torch.int32, device="cuda")
    vp = ctypes.c_void_p
    code = L.me_sample_static(vp(logits.data_ptr()), rows, 151936, vp(None), vp(None), vp(out.data_ptr()),
                              vp(torch.cuda.current_stream().cuda_stream))
    assert code != 0 and "static" in L.me_last_error().decode()
