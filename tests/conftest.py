"""Shared fixtures: tiny Qwen3 configurations with seeded random weights, written to temporary
model folders. Nothing is downloaded and nothing is committed."""

from __future__ import annotations

import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a GPU (run with -m gpu on the GPU box)")


def tiny_configs():
    """Configurations that differ in every size and option."""
    from mini_engine_amd.models.qwen3 import Qwen3Config

    a = Qwen3Config(vocab_size=256, hidden_size=64, intermediate_size=128, num_hidden_layers=2,
                    num_attention_heads=4, num_key_value_heads=2, head_dim=16, rms_norm_eps=1e-6,
                    rope_theta=10000.0, max_position_embeddings=512, tie_word_embeddings=True)
    b = Qwen3Config(vocab_size=384, hidden_size=96, intermediate_size=160, num_hidden_layers=3,
                    num_attention_heads=6, num_key_value_heads=1, head_dim=32, rms_norm_eps=1e-5,
                    rope_theta=1e6, max_position_embeddings=1024, tie_word_embeddings=False)
    # a third one whose head size and page size take the bfloat16 path through the matrix-core attention
    # kernels (A and B, with heads of 16 and pages of 8, run the general kernels)
    c = Qwen3Config(vocab_size=320, hidden_size=128, intermediate_size=256, num_hidden_layers=2,
                    num_attention_heads=4, num_key_value_heads=2, head_dim=64, rms_norm_eps=1e-6,
                    rope_theta=50000.0, max_position_embeddings=2048, tie_word_embeddings=True)
    # the head size, the group size and the page size of the benchmark's model, so that portions, tails and
    # pages that are used again pass through the kernels that serve it
    d = Qwen3Config(vocab_size=448, hidden_size=256, intermediate_size=384, num_hidden_layers=2,
                    num_attention_heads=16, num_key_value_heads=8, head_dim=128, rms_norm_eps=1e-6,
                    rope_theta=1e6, max_position_embeddings=4096, tie_word_embeddings=False)
    # widths that are no multiple of 8 or of 4 (the bfloat16 products fall to the kernels that take any size, the norms
    # to the scalar kernel), as many kv heads as heads, pages of 32
    e = Qwen3Config(vocab_size=5003, hidden_size=113, intermediate_size=101, num_hidden_layers=3,
                    num_attention_heads=5, num_key_value_heads=5, head_dim=64, rms_norm_eps=3e-6,
                    rope_theta=50000.0, max_position_embeddings=1024, tie_word_embeddings=True)
    # a head size that is no power of two and seven heads to a kv head
    f = Qwen3Config(vocab_size=1000, hidden_size=200, intermediate_size=344, num_hidden_layers=2,
                    num_attention_heads=21, num_key_value_heads=3, head_dim=96, rms_norm_eps=1e-5,
                    rope_theta=10000.0, max_position_embeddings=2048, tie_word_embeddings=False)
    return {"A": a, "B": b, "C": c, "D": d, "E": e, "F": f}


BLOCK_SIZES = {"A": 16, "B": 8, "C": 16, "D": 16, "E": 32, "F": 16}


def write_tiny(folder: str, cfg, seed: int = 0, std: float = 0.02, dtype=torch.bfloat16) -> str:
    from mini_engine_amd.models.qwen3 import plan_from_config
    from mini_engine_amd.parts.decoder import Decoder
    from mini_engine_amd.weights import write_model_folder

    wants = Decoder(plan_from_config(cfg), torch.float32, "cpu").weight_wants()
    write_model_folder(folder, cfg.to_config_json(), wants, seed=seed, dtype=dtype, std=std)
    return folder


@pytest.fixture(scope="session")
def tiny_folders(tmp_path_factory):
    """{"A": folder, "B": folder} with bfloat16 weights (both engine dtypes read the same values)."""
    out = {}
    for name, cfg in tiny_configs().items():
        out[name] = write_tiny(str(tmp_path_factory.mktemp(f"tiny_{name}")), cfg, seed=11 + len(out), std=0.05)
    return out


def random_prompt(length: int, vocab: int, seed: int) -> list[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(1, vocab, (length,), generator=g).tolist()
