"""Configuration: config.json keys, defaults and rejections of the Qwen3 entry, and the registry."""

from __future__ import annotations

import json

import pytest

from conftest import tiny_configs
from mini_engine_amd.config import EngineConfig, architecture_name_of, get_architecture, plan_from_folder
from mini_engine_amd.models.qwen3 import Qwen3Config, as_id_tuple, plan_from_config

BASE = dict(vocab_size=100, hidden_size=48, intermediate_size=80, num_hidden_layers=3, num_attention_heads=6,
            num_key_value_heads=2, rms_norm_eps=1e-5, max_position_embeddings=128, tie_word_embeddings=False)


def test_defaults_follow_the_reference():
    c = Qwen3Config.from_dict(BASE)
    assert c.head_dim == 48 // 6  # model.py:51
    assert c.rope_theta == 10000.0  # model.py:53
    assert c.eos_token_ids == ()
    c = Qwen3Config.from_dict({**BASE, "head_dim": 16, "rope_theta": 5e5, "eos_token_id": 7})
    assert (c.head_dim, c.rope_theta, c.eos_token_ids) == (16, 5e5, (7,))
    c = Qwen3Config.from_dict({**BASE, "rope_theta": 5e5, "rope_parameters": {"rope_type": "default", "rope_theta": 1e6}})
    assert c.rope_theta == 1e6  # rope_parameters wins over the top level (model.py:45, 53)
    assert Qwen3Config.from_dict({**BASE, "head_dim": None}).head_dim == 8


def test_rejections():
    with pytest.raises(ValueError, match="qwen3"):
        Qwen3Config.from_dict({**BASE, "model_type": "llama"})
    with pytest.raises(ValueError, match="RoPE"):
        Qwen3Config.from_dict({**BASE, "rope_parameters": {"rope_type": "yarn"}})
    with pytest.raises(ValueError, match="sliding"):
        Qwen3Config.from_dict({**BASE, "use_sliding_window": True})
    with pytest.raises(ValueError, match="required keys: rms_norm_eps"):
        Qwen3Config.from_dict({k: v for k, v in BASE.items() if k != "rms_norm_eps"})
    with pytest.raises(ValueError, match="multiple"):
        Qwen3Config.from_dict({**BASE, "num_key_value_heads": 4})


def test_eos_forms():
    assert as_id_tuple(None) == () and as_id_tuple(3) == (3,) and as_id_tuple([3, 4]) == (3, 4)


def test_registry_chooses_by_architectures_then_model_type():
    assert architecture_name_of({"architectures": ["Qwen3ForCausalLM"]}) == "Qwen3ForCausalLM"
    assert architecture_name_of({"model_type": "qwen3"}) == "Qwen3ForCausalLM"
    assert architecture_name_of({}) == "Qwen3ForCausalLM"  # the reference's default model_type
    assert get_architecture("Qwen3ForCausalLM").plan_from_config is plan_from_config
    with pytest.raises(ValueError, match="unknown architecture"):
        get_architecture("NoSuchModel")
    with pytest.raises(ValueError, match="model_type"):
        architecture_name_of({"model_type": "gpt2"})


def test_folder_round_trip_and_generation_config_eos(tmp_path):
    for cfg in tiny_configs().values():
        (tmp_path / "config.json").write_text(json.dumps(cfg.to_config_json()))
        got, plan = plan_from_folder(str(tmp_path))
        assert got == cfg
        assert plan.architecture == "Qwen3ForCausalLM" and len(plan.layers) == cfg.num_hidden_layers
    (tmp_path / "generation_config.json").write_text(json.dumps({"eos_token_id": [5, 6]}))
    got, plan = plan_from_folder(str(tmp_path))
    assert plan.eos_token_ids == (5, 6)  # engine.py:130-133: generation_config first


def test_plan_carries_every_size_from_the_config():
    for cfg in tiny_configs().values():
        plan = plan_from_config(cfg)
        assert plan.order == tuple(range(cfg.num_hidden_layers))
        assert (plan.vocab_size, plan.hidden_size, plan.tie_word_embeddings) == (
            cfg.vocab_size, cfg.hidden_size, cfg.tie_word_embeddings)
        for i, layer in enumerate(plan.layers):
            m = layer.mixer
            assert (m.num_heads, m.num_kv_heads, m.head_dim) == (
                cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim)
            assert m.scale == cfg.head_dim**-0.5 and m.qk_norm_eps == cfg.rms_norm_eps and m.window == 0
            assert m.position.theta == cfg.rope_theta and m.position.rotary_dim == cfg.head_dim
            assert layer.ffn.intermediate_size == cfg.intermediate_size
            assert layer.mixer_norm.eps == layer.ffn_norm.eps == plan.final_norm.eps == cfg.rms_norm_eps
            assert layer.mixer_prefix == f"model.layers.{i}.self_attn"


def test_plan_order_is_checked():
    from dataclasses import replace

    plan = plan_from_config(tiny_configs()["A"])
    assert replace(plan, order=(0, 1, 1, 0)).order == (0, 1, 1, 0)  # a layer may run twice
    with pytest.raises(ValueError, match="names layer"):
        replace(plan, order=(0, 5))


def test_engine_config_defaults_and_checks():
    c = EngineConfig()
    assert (c.block_size, c.num_blocks, c.max_num_seqs, c.max_num_batched_tokens, c.max_model_len) == (16, 256, 16, 2048, 4096)
    assert c.enable_prefix_caching and c.dtype == "float32" and c.seed == 0 and c.cuda_graphs
    with pytest.raises(ValueError, match="dtype"):
        EngineConfig(dtype="float16")
    with pytest.raises(ValueError):
        EngineConfig(block_size=0)


def test_pool_sized_by_memory():
    """A share of the GPU's memory instead of a number of pages: what is left of the share after everything already
    on the GPU and after a step's workspaces, in pages of all layers (the reference's sizing helper,
    ``engine.py:54-56``: 2 x layers x kv heads x head size x element size per token)."""
    from mini_engine_amd.engine.llm_engine import blocks_that_fit, kv_cache_bytes_per_token

    a = tiny_configs()["A"]
    plan = plan_from_config(a)
    per_token = 2 * a.num_hidden_layers * a.num_key_value_heads * a.head_dim
    assert kv_cache_bytes_per_token(plan, "float32") == 4 * per_token and kv_cache_bytes_per_token(plan, "bfloat16") == 2 * per_token
    page = 2 * per_token * 16
    total = 1 << 30
    assert blocks_that_fit(total, total, 1.0, plan, "bfloat16", 16) == total // page
    assert blocks_that_fit(total // 2, total, 0.75, plan, "bfloat16", 16) == (total // 4) // page  # half is taken, a quarter stays free
    with_steps = blocks_that_fit(total, total, 1.0, plan, "bfloat16", 16, max_num_batched_tokens=2048)
    assert 0 < with_steps < total // page  # a step's workspaces come off first
    with pytest.raises(ValueError, match="no room"):
        blocks_that_fit(total // 4, total, 0.5, plan, "bfloat16", 16)  # the others already use more than is left of the share
    with pytest.raises(ValueError, match="kv_memory_fraction"):
        EngineConfig(kv_memory_fraction=0.0)
    with pytest.raises(ValueError, match="kv_memory_fraction"):
        EngineConfig(kv_memory_fraction=1.5)
    assert EngineConfig(kv_memory_fraction=0.9).kv_memory_fraction == 0.9
