"""Each part of a layer alone, built from its spec and stepped on the GPU against the plain
implementation; then arrangements only the general decoder has: a layer run twice, a layer that
reads another layer's cache, layers with different windows (two cache groups), partial rotary and no
position encoding. These toy models exist only in this test."""

from __future__ import annotations

from dataclasses import replace

import pytest
import torch

import plain_qwen3 as plain
from conftest import tiny_configs

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def tol(dtype):
    return dict(rtol=1e-4, atol=2e-5) if dtype == "float32" else dict(rtol=3e-2, atol=3e-2)


def close(got, want, dtype):
    """Rounding errors are relative to the size of the values: the absolute part of the tolerance
    scales with the largest expected magnitude (at least 1)."""
    t = tol(dtype)
    torch.testing.assert_close(got, want, rtol=t["rtol"], atol=t["atol"] * max(1.0, want.abs().max().item()))


def batch_for(items, device="cuda", groups=1):
    """items: list of (tables per group, start, n tokens)."""
    from raw_batch import RawItem, make_raw_batch

    return make_raw_batch([RawItem(t, [0] * n, s, list(range(n))) for t, s, n in items], groups, device)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_part(dtype):
    from mini_engine_amd.config import NormSpec
    from mini_engine_amd.parts import NORMS

    norm = NORMS.build(NormSpec(dim=72, eps=1e-4), TORCH[dtype], torch.device("cuda"))
    assert set(norm.weight_wants("n.weight")) == {"n.weight"} and norm.weight_wants("n.weight")["n.weight"].role == "vector"
    w = 1 + 0.3 * torch.randn(72)
    norm.load({"n.weight": w.cuda()}, "n.weight")
    x = torch.randn(5, 72).to(TORCH[dtype])
    torch.testing.assert_close(norm(x.cuda()).float().cpu(), plain.rms_norm(x.float(), w, 1e-4), **tol(dtype))


def test_rotary_part_tables():
    from mini_engine_amd.config import RotarySpec
    from mini_engine_amd.parts import POSITION_ENCODINGS

    rot = POSITION_ENCODINGS.build(RotarySpec(rotary_dim=32, theta=1e6), torch.float32, torch.device("cuda"))
    want = 1.0 / (1e6 ** (torch.arange(0, 32, 2, dtype=torch.float32) / 32))
    assert torch.equal(rot.inv_freq.cpu(), want)  # model.py:75, bit for bit
    table = rot.tables(300).cpu()
    assert table.shape[0] >= 300 and table.shape[1:] == (2, 16)
    pos = torch.arange(table.shape[0], dtype=torch.float32)[:, None]
    torch.testing.assert_close(table[:, 0], torch.cos(pos * want), rtol=0, atol=2e-6)  # model.py:81-83
    torch.testing.assert_close(table[:, 1], torch.sin(pos * want), rtol=0, atol=2e-6)
    with pytest.raises(ValueError):
        POSITION_ENCODINGS.build(RotarySpec(rotary_dim=7, theta=1e4), torch.float32, torch.device("cuda"))


def attention_setup(dtype, spec, bs=16, pages=32):
    from mini_engine_amd.parts import MIXERS, KVBinding

    dt = TORCH[dtype]
    mixer = MIXERS.build(spec, dt, torch.device("cuda"))
    g = torch.Generator().manual_seed(1)
    w = {}
    for name, want in mixer.weight_wants("a").items():
        t = torch.randn(want.shape, generator=g)
        w[name] = (1 + 0.2 * t) if want.role == "vector" else (0.15 * t).to(dt).float()
    mixer.load({k: v.cuda().to(torch.float32 if v.dim() == 1 else dt) for k, v in w.items()}, "a")
    k = torch.zeros(pages, spec.num_kv_heads, bs, spec.head_dim, dtype=dt, device="cuda")
    v = torch.zeros(pages, spec.num_kv_heads, spec.head_dim, bs, dtype=dt, device="cuda")
    return mixer, w, KVBinding(0, k, v, bs)


def plain_attention(x, w, spec, positions):
    t = x.shape[0]
    q = (x @ w["a.q_proj.weight"].T).view(t, spec.num_heads, spec.head_dim)
    k = (x @ w["a.k_proj.weight"].T).view(t, spec.num_kv_heads, spec.head_dim)
    v = (x @ w["a.v_proj.weight"].T).view(t, spec.num_kv_heads, spec.head_dim)
    if spec.qk_norm_eps is not None:
        q, k = plain.rms_norm(q, w["a.q_norm.weight"], spec.qk_norm_eps), plain.rms_norm(k, w["a.k_norm.weight"], spec.qk_norm_eps)
    if spec.position is not None:
        rd = spec.position.rotary_dim
        cos, sin = plain.rope_tables(positions, rd, spec.position.theta)
        q = torch.cat((plain.apply_rope(q[..., :rd], cos, sin), q[..., rd:]), -1)
        k = torch.cat((plain.apply_rope(k[..., :rd], cos, sin), k[..., rd:]), -1)
    out = plain.grouped_causal_attention(q, k, v, spec.scale, spec.window)
    return out.reshape(t, -1) @ w["a.o_proj.weight"].T


def dense(out) -> torch.Tensor:
    """A part's output as a float32 tensor: in bfloat16 a delta of the residual stream comes back as float32 partial sums."""
    return out.to_tensor(torch.float32) if hasattr(out, "to_tensor") else out.float()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("variant", ["qwen", "no_norm_partial_rotary", "no_position_window", "mha_scaled"])
def test_attention_part_alone_whole_and_in_portions(dtype, variant):
    from mini_engine_amd.config import AttentionSpec, RotarySpec

    spec = {
        "qwen": AttentionSpec(hidden_size=72, num_heads=6, num_kv_heads=2, head_dim=32, scale=32**-0.5,
                              qk_norm_eps=1e-5, position=RotarySpec(32, 1e4)),
        "no_norm_partial_rotary": AttentionSpec(hidden_size=72, num_heads=4, num_kv_heads=4, head_dim=48, scale=0.2,
                                                qk_norm_eps=None, position=RotarySpec(16, 500.0)),
        "no_position_window": AttentionSpec(hidden_size=72, num_heads=3, num_kv_heads=1, head_dim=64, scale=0.11,
                                            qk_norm_eps=1e-6, window=9, position=None),
        "mha_scaled": AttentionSpec(hidden_size=72, num_heads=2, num_kv_heads=2, head_dim=128, scale=0.05,
                                    qk_norm_eps=1e-6, position=RotarySpec(128, 1e6)),
    }[variant]
    mixer, w, cache = attention_setup(dtype, spec)
    n = 45
    x = torch.randn(n, 72).to(TORCH[dtype])
    want = plain_attention(x.float(), w, spec, torch.arange(n))
    table = [[7, 3, 11]]
    whole = dense(mixer.forward(x.cuda(), batch_for([(table, 0, n)]), cache)).cpu()
    close(whole, want, dtype)
    # the same tokens in portions, from the cache the earlier portions left: 20 | 2 | 1 | 22
    cache.k_cache.zero_(), cache.v_cache.zero_()
    outs, lo = [], 0
    for m in (20, 2, 1, 22):
        outs.append(dense(mixer.forward(x[lo : lo + m].cuda(), batch_for([(table, lo, m)]), cache)).cpu())
        lo += m
    close(torch.cat(outs), want, dtype)


def test_attention_part_refuses_unsupported_head_sizes():
    from mini_engine_amd.config import AttentionSpec
    from mini_engine_amd.parts import MIXERS

    for d in (8, 24, 272):
        with pytest.raises(ValueError, match="head_dim"):
            MIXERS.build(AttentionSpec(hidden_size=64, num_heads=2, num_kv_heads=1, head_dim=d, scale=1.0),
                         torch.float32, torch.device("cuda"))
    with pytest.raises(ValueError, match="multiple"):
        MIXERS.build(AttentionSpec(hidden_size=64, num_heads=3, num_kv_heads=2, head_dim=16, scale=1.0),
                     torch.float32, torch.device("cuda"))
    for scale in (0.0, -0.25, float("inf"), float("nan")):  # the kernels scale before or after masking: only a positive scale agrees
        with pytest.raises(ValueError, match="scale"):
            MIXERS.build(AttentionSpec(hidden_size=64, num_heads=2, num_kv_heads=1, head_dim=16, scale=scale),
                         torch.float32, torch.device("cuda"))


@pytest.mark.parametrize("dtype", DTYPES)
def test_gated_mlp_part(dtype):
    from mini_engine_amd.config import GatedMlpSpec
    from mini_engine_amd.parts import FEED_FORWARDS

    dt = TORCH[dtype]
    for activation in ("silu", "gelu_tanh"):
        ffn = FEED_FORWARDS.build(GatedMlpSpec(hidden_size=72, intermediate_size=200, activation=activation), dt,
                                  torch.device("cuda"))
        w = {n: (0.2 * torch.randn(want.shape)).to(dt).float() for n, want in ffn.weight_wants("m").items()}
        ffn.load({k: v.cuda().to(dt) for k, v in w.items()}, "m")
        for rows in (3, 40, 150):
            x = torch.randn(rows, 72).to(dt)
            if activation == "silu":
                want = plain.swiglu_mlp(x.float(), w, "m")
            else:
                gate = torch.nn.functional.gelu(x.float() @ w["m.gate_proj.weight"].T, approximate="tanh")
                want = (gate * (x.float() @ w["m.up_proj.weight"].T)) @ w["m.down_proj.weight"].T
            scale = max(1.0, want.abs().max().item())  # bfloat16 rounding is relative to the values' size
            t = tol(dtype)
            out = ffn.forward(x.cuda())
            out = out.to_tensor(dt) if hasattr(out, "to_tensor") else out  # a delta may come back as partial sums
            torch.testing.assert_close(out.float().cpu(), want, rtol=t["rtol"], atol=t["atol"] * scale)
    with pytest.raises(ValueError, match="activations"):
        FEED_FORWARDS.build(GatedMlpSpec(hidden_size=8, intermediate_size=8, activation="gelu"), dt, torch.device("cuda"))


# ------------------------------------------------------------ arrangements of the general decoder
def build_runner(plan, dtype, seed=0, bs=16, num_blocks=64, **engine_over):
    from mini_engine_amd import EngineConfig
    from mini_engine_amd.engine.runner import ModelRunner
    from mini_engine_amd.parts import Decoder
    from mini_engine_amd.weights import RandomSource

    dec = Decoder(plan, TORCH[dtype], "cuda")
    src = RandomSource(dec.weight_wants(), seed, std=0.08, norm_std=0.1)
    # round the weights to bfloat16 so that both dtypes and the plain reference see the same values
    weights = {n: (src.get(n).to(torch.bfloat16).float() if w.role == "matrix" else src.get(n))
               for n, w in dec.weight_wants().items()}

    class Source:
        def shapes(self):
            return {n: tuple(t.shape) for n, t in weights.items()}

        def get(self, n):
            return weights[n]

    dec.load(Source())
    cfg = EngineConfig(block_size=bs, num_blocks=num_blocks, max_num_seqs=4, dtype=dtype, max_model_len=512,
                       enable_prefix_caching=False, **engine_over)
    return ModelRunner(dec, cfg), weights


def plain_general(plan, w, tokens):
    """The plain functions composed along plan.order, with per-layer window, rotary and cache source."""
    ids = torch.tensor(tokens)
    x = w[plan.embed_name][ids]
    pos = torch.arange(len(tokens))
    kv_of = {}  # layer -> keys and values of its latest run
    for i in plan.order:
        L = plan.layers[i]
        m = L.mixer
        h = plain.rms_norm(x, w[L.mixer_norm_name], L.mixer_norm.eps)
        t = h.shape[0]
        p = L.mixer_prefix
        q = (h @ w[f"{p}.q_proj.weight"].T).view(t, m.num_heads, m.head_dim)
        if m.qk_norm_eps is not None:
            q = plain.rms_norm(q, w[f"{p}.q_norm.weight"], m.qk_norm_eps)
        cos, sin = plain.rope_tables(pos, m.position.rotary_dim, m.position.theta)
        q = plain.apply_rope(q, cos, sin)
        if m.cache_from is None:
            k = (h @ w[f"{p}.k_proj.weight"].T).view(t, m.num_kv_heads, m.head_dim)
            v = (h @ w[f"{p}.v_proj.weight"].T).view(t, m.num_kv_heads, m.head_dim)
            if m.qk_norm_eps is not None:
                k = plain.rms_norm(k, w[f"{p}.k_norm.weight"], m.qk_norm_eps)
            kv_of[i] = (plain.apply_rope(k, cos, sin), v)
        k, v = kv_of[i if m.cache_from is None else m.cache_from]
        a = plain.grouped_causal_attention(q, k, v, m.scale, m.window).reshape(t, -1) @ w[f"{p}.o_proj.weight"].T
        x = x + a
        h = plain.rms_norm(x, w[L.ffn_norm_name], L.ffn_norm.eps)
        x = x + plain.swiglu_mlp(h, w, L.ffn_prefix)
    x = plain.rms_norm(x, w[plan.final_norm_name], plan.final_norm.eps)
    return x @ (w[plan.embed_name] if plan.tie_word_embeddings else w[plan.head_name]).T


def step_in_portions(runner, tokens, cuts):
    from mini_engine_amd.engine.batch import StepItem
    from mini_engine_amd.engine.sequence import Sequence

    bm = runner.new_block_manager()
    seq = Sequence(tokens)
    outs, lo = [], 0
    for n in cuts:
        assert bm.try_allocate(seq, lo + n)
        outs.append(runner.step([StepItem(seq, tokens[lo : lo + n], lo, list(range(n)))]).float().cpu().clone())
        lo += n
        seq.num_computed_tokens = lo
        bm.release_passed(seq)
    assert lo == len(tokens)
    held = [sum(1 for p in t if p >= 0) for t in seq.block_tables]
    bm.free(seq)
    return torch.cat(outs), held


@pytest.mark.parametrize("dtype", DTYPES)
def test_layer_run_twice_shared_cache_and_two_window_groups(dtype):
    """A four-layer toy: layer 1 keeps a 24-key window (a cache group of its own whose passed pages
    are given back), layer 2 reads layer 0's cache and has no k/v weights, and the order runs layer 3
    twice (same weights, a cache for each run)."""
    from mini_engine_amd.models.qwen3 import plan_from_config

    cfg = replace(tiny_configs()["B"], num_hidden_layers=4, head_dim=32)
    plan = plan_from_config(cfg)
    layers = list(plan.layers)
    layers[1] = replace(layers[1], mixer=replace(layers[1].mixer, window=24))
    layers[2] = replace(layers[2], mixer=replace(layers[2].mixer, cache_from=0))
    plan = replace(plan, layers=tuple(layers), order=(0, 1, 2, 3, 3))
    runner, w = build_runner(plan, dtype, bs=16)
    assert [g.window for g in runner.layout.groups] == [0, 24]
    assert "model.layers.2.self_attn.k_proj.weight" not in w and "model.layers.2.self_attn.k_norm.weight" not in w
    tokens = torch.randint(1, cfg.vocab_size, (90,), generator=torch.Generator().manual_seed(4)).tolist()
    want = plain_general(plan, w, tokens)
    # bfloat16: after five runs of a layer single logits of the 34,560 are off by 1.1-2.0% of their row's largest (3 to 3.5
    # here; measured over eight seeds of tokens, whole and cut alike), which a bound of 0.03 on every element sits in the
    # middle of; this file's bound for values of that size is relative to the largest of them. float32 keeps the plain one.
    check = (lambda got: torch.testing.assert_close(got, want, **tol(dtype))) if dtype == "float32" else (lambda got: close(got, want, dtype))
    whole, _ = step_in_portions(runner, tokens, [90])
    check(whole)
    cut, held = step_in_portions(runner, tokens, [30, 2, 17, 1, 1, 1, 38])
    check(cut)
    assert held[0] == 6 and held[1] <= 3  # the window group gave passed pages back on the way
