"""Weights: the safetensors container, the loader's single error, dtype roles, random-weights mode."""

from __future__ import annotations

import json

import pytest
import torch

from conftest import tiny_configs, write_tiny
from mini_engine_amd.models.qwen3 import plan_from_config
from mini_engine_amd.parts.decoder import Decoder
from mini_engine_amd.weights import (FolderSource, RandomSource, TensorWant, WeightError, load_tensors,
                                     read_header, write_file)


def test_container_round_trip_against_the_safetensors_library(tmp_path):
    from safetensors.torch import load_file, save_file

    tensors = {"a": torch.randn(3, 5).to(torch.bfloat16), "b": torch.randn(7), "c": torch.arange(6, dtype=torch.int32).view(2, 3)}
    ours, theirs = str(tmp_path / "ours.safetensors"), str(tmp_path / "theirs.safetensors")
    write_file(ours, tensors)
    back = load_file(ours)
    assert all(torch.equal(back[k], v) and back[k].dtype == v.dtype for k, v in tensors.items())
    save_file(tensors, theirs)
    (tmp_path / "m").mkdir()
    save_file(tensors, str(tmp_path / "m" / "model.safetensors"))
    src = FolderSource(str(tmp_path / "m"))
    assert src.shapes() == {"a": (3, 5), "b": (7,), "c": (2, 3)}
    assert all(torch.equal(src.get(k), v) for k, v in tensors.items())
    assert read_header(theirs)["a"].dtype == "BF16"


def test_truncated_file_is_refused(tmp_path):
    p = tmp_path / "x.safetensors"
    write_file(str(p), {"a": torch.zeros(4)})
    raw = p.read_bytes()
    p.write_bytes(raw[:-4])
    with pytest.raises(ValueError, match="inconsistent offsets"):
        read_header(str(p))


def test_offsets_that_point_before_the_data_or_run_backwards_are_refused(tmp_path):
    """A header whose offsets are negative (they would point into the header itself) or whose shape has a
    negative size passes a length check alone; both are refused like any other inconsistent offsets."""
    import json
    import struct

    for offsets, shape in (([-16, 0], [4]), ([16, 0], [-4]), ([0, 16], [-2, -2])):
        header = json.dumps({"a": {"dtype": "F32", "shape": shape, "data_offsets": offsets}}).encode()
        p = tmp_path / "bad.safetensors"
        p.write_bytes(struct.pack("<Q", len(header)) + header + bytes(16))
        with pytest.raises(ValueError, match="inconsistent offsets"):
            read_header(str(p))


def _decoder(cfg):
    return Decoder(plan_from_config(cfg), torch.float32, "cpu")


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg = tiny_configs()["B"]
    folder = write_tiny(str(tmp_path), cfg)
    from safetensors.torch import load_file, save_file

    t = load_file(str(tmp_path / "model.safetensors"))
    del t["model.layers.1.mlp.up_proj.weight"]
    del t["model.norm.weight"]
    t["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)
    t["model.layers.2.self_attn.q_norm.weight"] = torch.zeros(cfg.head_dim + 1)
    save_file(t, str(tmp_path / "model.safetensors"))
    with pytest.raises(WeightError) as e:
        _decoder(cfg).load(FolderSource(folder))
    assert e.value.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert e.value.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert len(e.value.wrong_shape) == 1 and "q_norm" in e.value.wrong_shape[0]
    msg = str(e.value)
    assert "missing tensors (2)" in msg and "unexpected tensors (1)" in msg and "wrong shapes (1)" in msg


def test_tied_head_drops_a_stored_head_and_untied_needs_it(tmp_path):
    cfg_a, cfg_b = tiny_configs()["A"], tiny_configs()["B"]
    from safetensors.torch import load_file, save_file

    fa = write_tiny(str(tmp_path / "a"), cfg_a)
    t = load_file(fa + "/model.safetensors")
    assert "lm_head.weight" not in t
    t["lm_head.weight"] = torch.zeros(cfg_a.vocab_size, cfg_a.hidden_size)
    save_file(t, fa + "/model.safetensors")
    dec = _decoder(cfg_a)
    dec.load(FolderSource(fa))  # model.py:190-195: the stored head is dropped
    assert dec.head is dec.embed_table
    fb = write_tiny(str(tmp_path / "b"), cfg_b)
    t = load_file(fb + "/model.safetensors")
    del t["lm_head.weight"]
    save_file(t, fb + "/model.safetensors")
    with pytest.raises(WeightError, match="lm_head.weight"):
        _decoder(cfg_b).load(FolderSource(fb))


def test_roles_decide_device_dtypes(tmp_path):
    write_file(str(tmp_path / "model.safetensors"), {
        "w": torch.randn(4, 4).to(torch.bfloat16), "n": torch.randn(4).to(torch.bfloat16),
        "n32": torch.randn(4), "w32": torch.randn(4, 4), "t": torch.arange(4, dtype=torch.int64)})
    wants = {"w": TensorWant((4, 4)), "n": TensorWant((4,), "vector"), "n32": TensorWant((4,), "vector"),
             "w32": TensorWant((4, 4)), "t": TensorWant((4,), "int_table")}
    src = FolderSource(str(tmp_path))
    bf = load_tensors(src, wants, torch.bfloat16, "cpu")
    assert bf["w"].dtype is torch.bfloat16 and torch.equal(bf["w"], src.get("w"))  # kept as stored
    assert bf["n"].dtype is torch.float32 and bf["n32"].dtype is torch.float32  # 32-bit stays 32-bit
    assert torch.equal(bf["n32"], src.get("n32")) and bf["t"].dtype is torch.int32
    f32 = load_tensors(src, wants, torch.float32, "cpu")
    assert f32["w"].dtype is torch.float32 and torch.equal(f32["w"], src.get("w").float())
    assert torch.equal(f32["w32"], src.get("w32"))


def test_random_weights_mode_writes_a_loadable_deterministic_folder(tmp_path):
    cfg = tiny_configs()["A"]
    f1, f2, f3 = (write_tiny(str(tmp_path / n), cfg, seed=s) for n, s in (("1", 4), ("2", 4), ("3", 5)))
    assert json.load(open(f1 + "/config.json"))["architectures"] == ["Qwen3ForCausalLM"]
    h1, h2, h3 = (FolderSource(f) for f in (f1, f2, f3))
    name = "model.layers.1.self_attn.q_proj.weight"
    assert torch.equal(h1.get(name), h2.get(name)) and not torch.equal(h1.get(name), h3.get(name))
    assert h1.get(name).dtype is torch.bfloat16
    _decoder(cfg).load(h1)
    emb = h1.get("model.embed_tokens.weight").float()
    assert abs(emb.std().item() - 0.02) < 0.002 and abs(emb.mean().item()) < 0.002
    norm = h1.get("model.norm.weight").float()
    assert abs(norm.mean().item() - 1.0) < 0.02


def test_random_source_values_do_not_depend_on_the_other_tensors():
    a = RandomSource({"x": TensorWant((8, 8)), "y": TensorWant((3,), "vector")}, seed=1)
    b = RandomSource({"y": TensorWant((3,), "vector")}, seed=1)
    assert torch.equal(a.get("y"), b.get("y"))
