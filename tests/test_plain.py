"""Pins the plain implementation (tests/plain_qwen3.py) by what fixes each formula beside the
reference's text: special cases that reduce to a library routine, invariants, and the one mask
vector the reference's own tests hold. Each check is chosen so that a plausible mistake fails it.
The reference holds no numeric model vectors (its parity tests run an installed model's code, which
is no source here), so whole model parity with it is "parity unpinned" beyond these checks."""

from __future__ import annotations

import math

import torch
import torch.nn.functional as F

import plain_qwen3 as plain

torch.manual_seed(0)


# ------------------------------------------------------------------------------------- RMSNorm
def test_rms_norm_equals_library_routine():
    x, w = torch.randn(5, 7, 48), torch.randn(48)
    torch.testing.assert_close(plain.rms_norm(x, w, 1e-5), F.rms_norm(x, (48,), w, 1e-5), rtol=1e-6, atol=1e-6)


def test_rms_norm_mean_square_and_eps_inside_root():
    x = torch.randn(4, 32) * 3
    y = plain.rms_norm(x, torch.ones(32), 1e-6)
    ms = (x * x).mean(-1)
    torch.testing.assert_close((y * y).mean(-1), ms / (ms + 1e-6))  # exactly ms/(ms+eps)
    # eps outside the root (x / (sqrt(ms) + eps)) would give another value for a tiny input
    tiny = torch.full((1, 8), 1e-4)
    expected = 1e-4 / math.sqrt(1e-8 + 1e-2)
    torch.testing.assert_close(plain.rms_norm(tiny, torch.ones(8), 1e-2), torch.full((1, 8), expected))
    assert torch.equal(plain.rms_norm(torch.zeros(2, 8), torch.ones(8), 1e-6), torch.zeros(2, 8))


def test_rms_norm_weight_multiplies_directly_and_scale_invariance():
    x, w = torch.randn(3, 16), torch.randn(16)
    torch.testing.assert_close(plain.rms_norm(x, w, 0.0), w * plain.rms_norm(x, torch.ones(16), 0.0))
    torch.testing.assert_close(plain.rms_norm(7.0 * x, w, 0.0), plain.rms_norm(x, w, 0.0), rtol=1e-5, atol=1e-6)


def test_qk_norm_is_per_head_slice():
    x, w = torch.randn(5, 3, 16), torch.randn(16)
    whole = plain.rms_norm(x, w, 1e-6)
    for t in range(5):
        for h in range(3):
            torch.testing.assert_close(whole[t, h], plain.rms_norm(x[t, h], w, 1e-6))


# ---------------------------------------------------------------------------------------- RoPE
def test_rope_position_zero_is_identity_and_tables_have_equal_halves():
    cos, sin = plain.rope_tables(torch.arange(6), 16, 10000.0)
    assert torch.equal(cos[:, :8], cos[:, 8:]) and torch.equal(sin[:, :8], sin[:, 8:])
    x = torch.randn(6, 2, 16)
    assert torch.equal(plain.apply_rope(x, cos, sin)[0], x[0])


def test_rope_is_a_rotation_of_pairs_j_and_j_plus_half_by_pos_times_theta_pow():
    """Independent formula: (x_j + i x_{j+d/2}) * exp(i * pos * theta^(-2j/d)), in float64 complex.
    Interleaved pairing (2j, 2j+1), a flipped sign, or theta^(-j/d) all fail it."""
    d, theta = 16, 10000.0
    pos = torch.tensor([0, 1, 5, 77, 1000])
    x = torch.randn(5, 3, d, dtype=torch.float64)
    cos, sin = plain.rope_tables(pos, d, theta)
    got = plain.apply_rope(x, cos.double(), sin.double())
    z = torch.complex(x[..., : d // 2], x[..., d // 2 :])
    ang = pos[:, None].double() * torch.tensor([theta ** (-2.0 * j / d) for j in range(d // 2)], dtype=torch.float64)
    zr = z * torch.polar(torch.ones_like(ang), ang)[:, None, :]
    want = torch.cat((zr.real, zr.imag), dim=-1)
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)


def test_rope_on_a_vector_worked_by_hand_from_the_reference_lines():
    """model.py:75 with d = 4, theta = 10000: inv_freq = [10000^0, 10000^(-2/4)] = [1, 0.01]. model.py:86-90 at
    position 1 on x = [1, 2, 3, 4]: x1 = [1, 2], x2 = [3, 4], cat(-x2, x1) = [-3, -4, 1, 2], angles [1, 0.01, 1, 0.01]:
      out = [1 cos 1 - 3 sin 1, 2 cos 0.01 - 4 sin 0.01, 3 cos 1 + 1 sin 1, 4 cos 0.01 + 2 sin 0.01]
    with cos 1 = 0.5403023, sin 1 = 0.8414710, cos 0.01 = 0.99995, sin 0.01 = 0.00999983 (the literals below are
    worked out from these by hand). Pairs (2j, 2j+1) would give -1.1426 first; the exponent j/d would give the
    second angle as 0.1."""
    cos, sin = plain.rope_tables(torch.tensor([1]), 4, 10000.0)
    got = plain.apply_rope(torch.tensor([[[1.0, 2.0, 3.0, 4.0]]]), cos, sin)[0, 0]
    torch.testing.assert_close(got, torch.tensor([-1.9841107, 1.9599007, 2.4623779, 4.0197997]), rtol=0, atol=2e-6)
    # and at position 3 with d = 8, theta = 1e6 (the benchmark's theta): angle of pair (2, 6) is 3 * 1e6^(-4/8) = 0.003
    cos, sin = plain.rope_tables(torch.tensor([3]), 8, 1e6)
    x = torch.zeros(1, 1, 8)
    x[0, 0, 2] = 1.0
    got = plain.apply_rope(x, cos, sin)[0, 0]
    want = torch.zeros(8)
    want[2], want[6] = 0.9999955, 0.0029999955  # cos 0.003, sin 0.003: the unit vector of element 2 turns towards element 6
    torch.testing.assert_close(got, want, rtol=0, atol=1e-7)


def test_rope_scores_depend_on_distance_only():
    d = 32
    q, k = torch.randn(1, 1, d, dtype=torch.float64), torch.randn(1, 1, d, dtype=torch.float64)

    def score(m, n):
        cm, sm = plain.rope_tables(torch.tensor([m]), d, 1e6)
        cn, sn = plain.rope_tables(torch.tensor([n]), d, 1e6)
        return (plain.apply_rope(q, cm.double(), sm.double()) * plain.apply_rope(k, cn.double(), sn.double())).sum()

    torch.testing.assert_close(score(9, 4), score(105, 100), rtol=1e-4, atol=1e-5)
    assert abs(score(9, 4) - score(9, 5)) > 1e-3  # and does depend on the distance


# ------------------------------------------------------------------------- the attention block
def _block_inputs(seed: int, eps: float):
    g = torch.Generator().manual_seed(seed)
    cfg = plain.PlainConfig(vocab_size=11, hidden_size=24, intermediate_size=8, num_layers=1, num_heads=4, num_kv_heads=2,
                            head_dim=16, rms_norm_eps=eps, rope_theta=10000.0, tie_word_embeddings=True)
    w = {"a.q_proj.weight": torch.randn(64, 24, generator=g), "a.k_proj.weight": torch.randn(32, 24, generator=g),
         "a.v_proj.weight": torch.randn(32, 24, generator=g), "a.o_proj.weight": torch.randn(24, 64, generator=g),
         # weights that differ inside every rotated pair (j, j + d/2): where the norm sits then shows
         "a.q_norm.weight": 0.5 + torch.rand(16, generator=g), "a.k_norm.weight": 0.5 + torch.rand(16, generator=g)}
    return cfg, w, torch.randn(9, 24, generator=g)


def test_attention_block_depends_on_distances_only_so_qk_norm_sits_before_rope():
    """With the q/k norm before the rotation, scores are a function of position differences, so a
    shift of all positions changes nothing. A norm weight applied after the rotation scales the two
    elements of a rotated pair differently and the scores come to depend on the positions themselves:
    the same check on such a variant fails, which shows that it can."""
    cfg, w, x = _block_inputs(3, 1e-6)
    here = plain.attention_block(x, w, "a", cfg, torch.arange(9))
    shifted = plain.attention_block(x, w, "a", cfg, torch.arange(9) + 777)
    torch.testing.assert_close(shifted, here, rtol=1e-3, atol=1e-3)

    def norm_after_rope(positions):
        q = (x @ w["a.q_proj.weight"].T).view(9, 4, 16)
        k = (x @ w["a.k_proj.weight"].T).view(9, 2, 16)
        v = (x @ w["a.v_proj.weight"].T).view(9, 2, 16)
        cos, sin = plain.rope_tables(positions, 16, cfg.rope_theta)
        q = plain.rms_norm(plain.apply_rope(q, cos, sin), w["a.q_norm.weight"], 1e-6)
        k = plain.rms_norm(plain.apply_rope(k, cos, sin), w["a.k_norm.weight"], 1e-6)
        return plain.grouped_causal_attention(q, k, v, 16**-0.5).reshape(9, -1) @ w["a.o_proj.weight"].T

    assert (norm_after_rope(torch.arange(9)) - norm_after_rope(torch.arange(9) + 777)).abs().max() > 0.05
    assert (here - norm_after_rope(torch.arange(9))).abs().max() > 0.05  # and the two orders are different functions


def test_attention_block_equals_library_routines_put_together():
    """The whole block from library routines: ``F.rms_norm`` per head with the one [d] weight (and an
    eps large enough to matter, the configuration's only one), the rotation as a complex product,
    ``F.scaled_dot_product_attention`` with its default scale (1/sqrt(d)) and ``is_causal``. A scale
    from another size, a norm weight per head, a norm on v or an eps of its own would fail it."""
    cfg, w, x = _block_inputs(4, 0.3)
    t, nh, nkv, d = 9, cfg.num_heads, cfg.num_kv_heads, cfg.head_dim
    got = plain.attention_block(x, w, "a", cfg, torch.arange(t))
    q = F.rms_norm((x @ w["a.q_proj.weight"].T).view(t, nh, d), (d,), w["a.q_norm.weight"], 0.3)
    k = F.rms_norm((x @ w["a.k_proj.weight"].T).view(t, nkv, d), (d,), w["a.k_norm.weight"], 0.3)
    v = (x @ w["a.v_proj.weight"].T).view(t, nkv, d)
    ang = torch.arange(t)[:, None].double() * torch.tensor([cfg.rope_theta ** (-2.0 * j / d) for j in range(d // 2)],
                                                           dtype=torch.float64)
    turn = torch.polar(torch.ones_like(ang), ang)[:, None, :]

    def rotate(z):
        zc = torch.complex(z[..., : d // 2].double(), z[..., d // 2:].double()) * turn
        return torch.cat((zc.real, zc.imag), dim=-1).float()

    out = F.scaled_dot_product_attention(rotate(q).transpose(0, 1), rotate(k).repeat_interleave(nh // nkv, dim=1).transpose(0, 1),
                                         v.repeat_interleave(nh // nkv, dim=1).transpose(0, 1), is_causal=True).transpose(0, 1)
    torch.testing.assert_close(got, out.reshape(t, -1) @ w["a.o_proj.weight"].T, rtol=1e-4, atol=1e-4)


# ----------------------------------------------------------------------------------- attention
def test_visible_is_the_reference_tests_mask():
    """tests/test_attention.py:55 of the reference: ones(new, cached+new).tril(diagonal=cached)."""
    for cached, new in [(0, 7), (9, 1), (8, 5)]:
        want = torch.ones(new, cached + new, dtype=torch.bool).tril(diagonal=cached)
        assert torch.equal(plain.visible(new, cached + new), want)


def test_attention_equals_library_sdpa_with_repeated_kv_heads():
    """GQA: query head i uses kv head i // group (reference tests/test_attention.py:52-58)."""
    nh, nkv, d = 6, 2, 8
    for cached, new in [(0, 7), (9, 1), (8, 5)]:
        q = torch.randn(new, nh, d)
        k, v = torch.randn(cached + new, nkv, d), torch.randn(cached + new, nkv, d)
        got = plain.grouped_causal_attention(q, k, v, d**-0.5)
        mask = torch.ones(new, cached + new, dtype=torch.bool).tril(diagonal=cached)
        want = F.scaled_dot_product_attention(
            q.transpose(0, 1), k.repeat_interleave(nh // nkv, dim=1).transpose(0, 1),
            v.repeat_interleave(nh // nkv, dim=1).transpose(0, 1), attn_mask=mask).transpose(0, 1)
        torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)


def test_attention_single_key_returns_value_and_masked_keys_do_not_matter():
    q, k, v = torch.randn(1, 4, 8), torch.randn(1, 2, 8), torch.randn(1, 2, 8)
    out = plain.grouped_causal_attention(q, k, v, 8**-0.5)
    torch.testing.assert_close(out[0, 0], v[0, 0])
    torch.testing.assert_close(out[0, 3], v[0, 1])
    # the first of two query rows must not see the second key, whatever it holds
    q2, k2, v2 = torch.randn(2, 2, 8), torch.randn(2, 2, 8), torch.randn(2, 2, 8)
    a = plain.grouped_causal_attention(q2, k2, v2, 1.0)
    k2[1], v2[1] = 100.0, -50.0
    b = plain.grouped_causal_attention(q2, k2, v2, 1.0)
    torch.testing.assert_close(a[0], b[0])


def test_attention_window_hides_old_keys():
    q, k, v = torch.randn(6, 1, 4), torch.randn(6, 1, 4), torch.randn(6, 1, 4)
    full = plain.grouped_causal_attention(q, k, v, 0.5, window=0)
    win = plain.grouped_causal_attention(q, k, v, 0.5, window=3)
    torch.testing.assert_close(full[:3], win[:3])  # positions 0..2 see everything either way
    torch.testing.assert_close(win[5], plain.grouped_causal_attention(q[5:], k[3:], v[3:], 0.5)[0])


# -------------------------------------------------------------------------------------- SwiGLU
def test_silu_equals_library_and_zero_gate_gives_zero():
    z = torch.randn(100) * 4
    torch.testing.assert_close(plain.silu(z), F.silu(z), rtol=1e-6, atol=1e-6)
    w = {"m.gate_proj.weight": torch.zeros(12, 8), "m.up_proj.weight": torch.randn(12, 8),
         "m.down_proj.weight": torch.randn(8, 12)}
    assert torch.equal(plain.swiglu_mlp(torch.randn(3, 8), w, "m"), torch.zeros(3, 8))


def test_mlp_gate_and_up_are_not_swapped():
    x = torch.randn(4, 8)
    w = {"m.gate_proj.weight": torch.randn(12, 8), "m.up_proj.weight": torch.randn(12, 8),
         "m.down_proj.weight": torch.randn(8, 12)}
    want = F.linear(F.silu(F.linear(x, w["m.gate_proj.weight"])) * F.linear(x, w["m.up_proj.weight"]),
                    w["m.down_proj.weight"])
    torch.testing.assert_close(plain.swiglu_mlp(x, w, "m"), want, rtol=1e-5, atol=1e-5)


# --------------------------------------------------------------------------------- whole model
def _tiny(tied: bool):
    cfg = plain.PlainConfig(vocab_size=40, hidden_size=24, intermediate_size=36, num_layers=2, num_heads=3,
                            num_kv_heads=1, head_dim=8, rms_norm_eps=1e-5, rope_theta=100.0,
                            tie_word_embeddings=tied)
    g = torch.Generator().manual_seed(3)
    r = lambda *s: torch.randn(*s, generator=g) * 0.3
    w = {"model.embed_tokens.weight": r(40, 24), "model.norm.weight": 1 + r(24), "lm_head.weight": r(40, 24)}
    for l in range(2):
        p = f"model.layers.{l}"
        w.update({
            f"{p}.input_layernorm.weight": 1 + r(24), f"{p}.post_attention_layernorm.weight": 1 + r(24),
            f"{p}.self_attn.q_proj.weight": r(24, 24), f"{p}.self_attn.k_proj.weight": r(8, 24),
            f"{p}.self_attn.v_proj.weight": r(8, 24), f"{p}.self_attn.o_proj.weight": r(24, 24),
            f"{p}.self_attn.q_norm.weight": 1 + r(8), f"{p}.self_attn.k_norm.weight": 1 + r(8),
            f"{p}.mlp.gate_proj.weight": r(36, 24), f"{p}.mlp.up_proj.weight": r(36, 24),
            f"{p}.mlp.down_proj.weight": r(24, 36)})
    return cfg, w


def test_model_with_silent_layers_is_embedding_norm_head():
    """o_proj = down_proj = 0 leaves x = embedding: logits = head(final_norm(E[ids])). A missing final
    norm, a scaled embedding or an untied head where it is tied fails it."""
    for tied in (True, False):
        cfg, w = _tiny(tied)
        for l in range(2):
            w[f"model.layers.{l}.self_attn.o_proj.weight"].zero_()
            w[f"model.layers.{l}.mlp.down_proj.weight"].zero_()
        ids = [3, 9, 9, 31]
        x = F.rms_norm(w["model.embed_tokens.weight"][ids], (24,), w["model.norm.weight"], 1e-5)
        head = w["model.embed_tokens.weight"] if tied else w["lm_head.weight"]
        torch.testing.assert_close(plain.forward_logits(w, cfg, ids), x @ head.T, rtol=1e-5, atol=1e-5)


def test_layer_is_pre_norm_with_two_residual_adds():
    """With attention silenced a layer is x + mlp(norm2(x)): post-norm or a shared norm fails it."""
    cfg, w = _tiny(True)
    w["model.layers.0.self_attn.o_proj.weight"].zero_()
    x = torch.randn(5, 24)
    h = F.rms_norm(x, (24,), w["model.layers.0.post_attention_layernorm.weight"], 1e-5)
    want = x + plain.swiglu_mlp(h, w, "model.layers.0.mlp")
    torch.testing.assert_close(plain.decoder_layer(x, w, 0, cfg, torch.arange(5)), want, rtol=1e-5, atol=1e-5)


def test_model_is_causal_and_position_aware():
    cfg, w = _tiny(True)
    a = plain.forward_logits(w, cfg, [1, 2, 3, 4, 5])
    b = plain.forward_logits(w, cfg, [1, 2, 3, 9, 9])
    torch.testing.assert_close(a[:3], b[:3])  # a later token never changes earlier logits
    c = plain.forward_logits(w, cfg, [2, 1, 3, 4, 5])
    assert (a[4] - c[4]).abs().max() > 1e-4  # order matters: positions are encoded


def test_greedy_keeps_eos_and_stops():
    cfg, w = _tiny(True)
    free = plain.greedy_generate(w, cfg, [1, 2, 3], 6)
    assert len(free) == 6
    cut = plain.greedy_generate(w, cfg, [1, 2, 3], 6, eos=(free[2],))
    assert cut == free[: free.index(free[2]) + 1]


def test_temperature_probs():
    logits = torch.tensor([[1.0, 2.0, 4.0]])
    torch.testing.assert_close(plain.temperature_probs(logits, 0.5), torch.softmax(logits / 0.5, -1))
    assert plain.temperature_probs(logits, 0.0)[0, 2] > 0.999999  # clamp at 1e-5 acts as argmax
