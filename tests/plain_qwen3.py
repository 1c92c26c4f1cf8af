"""A plain, slow Qwen3 dense decoder: whole sequences, no cache, no batching, float32 on the CPU.

Written from the formulas of the reference (``src/mini_engine`` there), one function per
part, each citing the lines it restates. It shares no code with the package under test: it reads
``config.json`` with ``json`` and the weights with the ``safetensors`` library, and uses only
elementary torch operations (matmul, exp, sum, ...), so that each library routine that computes the
same thing (``F.rms_norm``, ``F.silu``, ``F.scaled_dot_product_attention``) stays free to pin it in
``test_plain.py``.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class PlainConfig:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool


def read_config(folder: str) -> PlainConfig:
    """Keys and defaults of ``model.py:35-56``."""
    with open(os.path.join(folder, "config.json")) as f:
        c = json.load(f)
    rope = c.get("rope_parameters") or {}
    return PlainConfig(
        vocab_size=c["vocab_size"],
        hidden_size=c["hidden_size"],
        intermediate_size=c["intermediate_size"],
        num_layers=c["num_hidden_layers"],
        num_heads=c["num_attention_heads"],
        num_kv_heads=c["num_key_value_heads"],
        head_dim=c.get("head_dim") or c["hidden_size"] // c["num_attention_heads"],  # model.py:51
        rms_norm_eps=c["rms_norm_eps"],
        rope_theta=float(rope.get("rope_theta", c.get("rope_theta", 10000.0))),  # model.py:53
        tie_word_embeddings=bool(c["tie_word_embeddings"]),
    )


def read_weights(folder: str, dtype: torch.dtype = torch.float32) -> dict[str, torch.Tensor]:
    """All tensors of the folder, up-cast to ``dtype`` (``engine.py:126-128``)."""
    from safetensors.torch import load_file

    out: dict[str, torch.Tensor] = {}
    for name in sorted(os.listdir(folder)):
        if name.endswith(".safetensors"):
            out.update(load_file(os.path.join(folder, name)))
    return {k: v.to(dtype) for k, v in out.items()}


# ------------------------------------------------------------------------------------------ parts


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``model.py:65-69``: ``x * rsqrt(mean(x^2, last) + eps)``, then times ``weight``.
    eps is inside the square root; the weight multiplies directly (not ``1 + w``)."""
    mean_square = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return weight * (x / torch.sqrt(mean_square + eps))


def rope_tables(positions: torch.Tensor, head_dim: int, theta: float) -> tuple[torch.Tensor, torch.Tensor]:
    """``model.py:75, 79-83``: ``inv_freq[j] = theta^(-2j/d)``, ``freqs = pos * inv_freq``,
    tables are ``cat(freqs, freqs)`` so both halves of a head see the same angles."""
    j = torch.arange(0, head_dim, 2, dtype=torch.float32)
    inv_freq = 1.0 / (theta ** (j / head_dim))
    freqs = positions.to(torch.float32)[:, None] * inv_freq[None, :]
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos(), emb.sin()


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """``model.py:86-90``: x is [T, heads, d]; ``x*cos + cat(-x2, x1)*sin`` with x1, x2 the two
    halves of the last dim (pairs ``(j, j + d/2)``)."""
    half = x.shape[-1] // 2
    x1, x2 = x[..., :half], x[..., half:]
    rotated = torch.cat((-x2, x1), dim=-1)
    return x * cos[:, None, :].to(x.dtype) + rotated * sin[:, None, :].to(x.dtype)


def visible(num_queries: int, num_keys: int, window: int = 0) -> torch.Tensor:
    """[Q, K] bool. The queries are the last Q of K positions. ``attention.py:79-86``: query at
    absolute position p sees keys at positions <= p. ``window > 0`` (not in the reference; used by
    the tests of the general attention part) also hides keys at positions <= p - window."""
    q_pos = torch.arange(num_keys - num_queries, num_keys)[:, None]
    k_pos = torch.arange(num_keys)[None, :]
    ok = k_pos <= q_pos
    if window > 0:
        ok = ok & (k_pos > q_pos - window)
    return ok


def grouped_causal_attention(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: int = 0
) -> torch.Tensor:
    """``attention.py:160-175`` for one sequence: q [Q, nh, d], k and v [K, nkv, d] -> [Q, nh, d].
    Query head i uses key/value head ``i // (nh // nkv)`` (``attention.py:162-163``); scores are
    ``q.k * scale`` (``:170``), hidden keys get -inf (``:171-172``), softmax over keys (``:173``)."""
    num_q, nh, d = q.shape
    num_k, nkv, _ = k.shape
    group = nh // nkv
    mask = visible(num_q, num_k, window)
    out = torch.empty_like(q)
    for head in range(nh):
        kv = head // group
        scores = (q[:, head, :] @ k[:, kv, :].T) * scale  # [Q, K]
        scores = scores.masked_fill(~mask, float("-inf"))
        scores = scores - scores.max(dim=-1, keepdim=True).values
        p = scores.exp()
        p = p / p.sum(dim=-1, keepdim=True)
        out[:, head, :] = p @ v[:, kv, :]
    return out


def attention_block(
    x: torch.Tensor, w: dict[str, torch.Tensor], prefix: str, cfg: PlainConfig, positions: torch.Tensor
) -> torch.Tensor:
    """``model.py:111-119``: project, view as heads, q/k RMSNorm over each head's d (one [d] weight
    for all heads) BEFORE rope, v untouched, rope on q and k, attention, output projection."""
    t = x.shape[0]
    q = (x @ w[f"{prefix}.q_proj.weight"].T).view(t, cfg.num_heads, cfg.head_dim)
    k = (x @ w[f"{prefix}.k_proj.weight"].T).view(t, cfg.num_kv_heads, cfg.head_dim)
    v = (x @ w[f"{prefix}.v_proj.weight"].T).view(t, cfg.num_kv_heads, cfg.head_dim)
    q = rms_norm(q, w[f"{prefix}.q_norm.weight"], cfg.rms_norm_eps)
    k = rms_norm(k, w[f"{prefix}.k_norm.weight"], cfg.rms_norm_eps)
    cos, sin = rope_tables(positions, cfg.head_dim, cfg.rope_theta)
    q, k = apply_rope(q, cos, sin), apply_rope(k, cos, sin)
    out = grouped_causal_attention(q, k, v, cfg.head_dim**-0.5)
    return out.reshape(t, -1) @ w[f"{prefix}.o_proj.weight"].T


def silu(z: torch.Tensor) -> torch.Tensor:
    """``z * sigmoid(z)``, the activation of ``model.py:130``."""
    return z / (1.0 + torch.exp(-z))


def swiglu_mlp(x: torch.Tensor, w: dict[str, torch.Tensor], prefix: str) -> torch.Tensor:
    """``model.py:129-131``: ``down(silu(gate(x)) * up(x))``, no biases."""
    gate = x @ w[f"{prefix}.gate_proj.weight"].T
    up = x @ w[f"{prefix}.up_proj.weight"].T
    return (silu(gate) * up) @ w[f"{prefix}.down_proj.weight"].T


def decoder_layer(
    x: torch.Tensor, w: dict[str, torch.Tensor], layer: int, cfg: PlainConfig, positions: torch.Tensor
) -> torch.Tensor:
    """``model.py:142-151``: ``x += attn(input_layernorm(x)); x += mlp(post_attention_layernorm(x))``."""
    p = f"model.layers.{layer}"
    h = rms_norm(x, w[f"{p}.input_layernorm.weight"], cfg.rms_norm_eps)
    x = x + attention_block(h, w, f"{p}.self_attn", cfg, positions)
    h = rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], cfg.rms_norm_eps)
    return x + swiglu_mlp(h, w, f"{p}.mlp")


def forward_logits(w: dict[str, torch.Tensor], cfg: PlainConfig, tokens: list[int]) -> torch.Tensor:
    """``model.py:172-188`` on one whole sequence: logits [T, V] at every position. Embedding is a
    plain row lookup (``:182``), positions count from 0 (``engine.py:209``), final norm then the
    head, which is the embedding table when tied (``:169-170, 186-187``)."""
    ids = torch.tensor(tokens, dtype=torch.long)
    x = w["model.embed_tokens.weight"][ids]
    positions = torch.arange(len(tokens))
    for layer in range(cfg.num_layers):
        x = decoder_layer(x, w, layer, cfg, positions)
    x = rms_norm(x, w["model.norm.weight"], cfg.rms_norm_eps)
    head = w["model.embed_tokens.weight"] if cfg.tie_word_embeddings else w["lm_head.weight"]
    return x @ head.T


def greedy_generate(w: dict[str, torch.Tensor], cfg: PlainConfig, prompt: list[int], max_tokens: int,
                    eos: tuple[int, ...] = ()) -> list[int]:
    """Recompute the whole sequence for every new token; argmax of the last row
    (``engine.py:286-288``); stop after ``max_tokens`` or at an EOS id, which is kept
    (``scheduler.py:145-148``)."""
    tokens = list(prompt)
    out: list[int] = []
    for _ in range(max_tokens):
        nxt = int(forward_logits(w, cfg, tokens)[-1].argmax())
        tokens.append(nxt)
        out.append(nxt)
        if nxt in eos:
            break
    return out


def temperature_probs(logits: torch.Tensor, temperature: float) -> torch.Tensor:
    """``engine.py:289``: ``softmax(float(logits) / clamp(temperature, min=1e-5))``."""
    z = logits.to(torch.float32) / max(temperature, 1e-5)
    z = z - z.max(dim=-1, keepdim=True).values
    p = z.exp()
    return p / p.sum(dim=-1, keepdim=True)


# ------------------------------------------------------------- the same model, as a bfloat16 engine rounds it


def _bf16(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.bfloat16).to(torch.float32)


def forward_logits_rounded(w: dict[str, torch.Tensor], cfg: PlainConfig, tokens: list[int]) -> torch.Tensor:
    """:func:`forward_logits` with every operand of a matrix product rounded to bfloat16 where a bfloat16 engine holds
    it in bfloat16 (the normed activations, q, k and v as projected and again as rotated, the softmax weights before
    they multiply the values, the attention output, the gated activation, the rows in front of the head) and every sum,
    the residual stream, the norms and the softmax in float32. The weights are expected to be bfloat16 values already.
    What is left between this and a bfloat16 engine is the order of float32 sums and the few places where kernels of
    different step sizes round differently; what is left between this and :func:`forward_logits` is bfloat16 itself."""
    ids = torch.tensor(tokens, dtype=torch.long)
    x = w["model.embed_tokens.weight"][ids]
    t = len(tokens)
    positions = torch.arange(t)
    group = cfg.num_heads // cfg.num_kv_heads
    mask = visible(t, t)
    for layer in range(cfg.num_layers):
        p = f"model.layers.{layer}"
        a = f"{p}.self_attn"
        h = _bf16(rms_norm(x, w[f"{p}.input_layernorm.weight"], cfg.rms_norm_eps))
        q = _bf16(h @ w[f"{a}.q_proj.weight"].T).view(t, cfg.num_heads, cfg.head_dim)
        k = _bf16(h @ w[f"{a}.k_proj.weight"].T).view(t, cfg.num_kv_heads, cfg.head_dim)
        v = _bf16(h @ w[f"{a}.v_proj.weight"].T).view(t, cfg.num_kv_heads, cfg.head_dim)
        cos, sin = rope_tables(positions, cfg.head_dim, cfg.rope_theta)
        q = _bf16(apply_rope(rms_norm(q, w[f"{a}.q_norm.weight"], cfg.rms_norm_eps), cos, sin))
        k = _bf16(apply_rope(rms_norm(k, w[f"{a}.k_norm.weight"], cfg.rms_norm_eps), cos, sin))
        out = torch.empty_like(q)
        for head in range(cfg.num_heads):
            kv = head // group
            s = (q[:, head] @ k[:, kv].T) * cfg.head_dim**-0.5
            s = s.masked_fill(~mask, float("-inf"))
            e = (s - s.max(dim=-1, keepdim=True).values).exp()
            out[:, head] = (_bf16(e) @ v[:, kv]) / e.sum(dim=-1, keepdim=True)
        x = x + _bf16(out.reshape(t, -1)) @ w[f"{a}.o_proj.weight"].T
        h = _bf16(rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], cfg.rms_norm_eps))
        m = f"{p}.mlp"
        act = _bf16(silu(h @ w[f"{m}.gate_proj.weight"].T) * (h @ w[f"{m}.up_proj.weight"].T))
        x = x + act @ w[f"{m}.down_proj.weight"].T
    x = _bf16(rms_norm(x, w["model.norm.weight"], cfg.rms_norm_eps))
    head = w["model.embed_tokens.weight"] if cfg.tie_word_embeddings else w["lm_head.weight"]
    return x @ head.T
