"""Seeded random weights: a tensor source, and a writer of whole model folders.

Projection and embedding tables are drawn from N(0, std) and norm weights from 1 + N(0, norm_std).
Every tensor has a random stream of its own, keyed on the seed and the tensor's name, so the values
of a tensor do not depend on which other tensors a model has or on the order they are drawn in.
"""

from __future__ import annotations

import hashlib
import json
import os

import torch

from .loader import TensorWant
from .safetensors_io import write_file


def _stream_seed(seed: int, name: str) -> int:
    digest = hashlib.blake2b(f"{seed}:{name}".encode(), digest_size=8).digest()
    return int.from_bytes(digest, "little") & ((1 << 63) - 1)


class RandomSource:
    """Generates each wanted tensor when asked for it (on ``device``, float32)."""

    def __init__(self, wants: dict[str, TensorWant], seed: int, std: float = 0.02, norm_std: float = 0.01,
                 device: str | torch.device = "cpu"):
        self.wants, self.seed, self.std, self.norm_std = wants, seed, std, norm_std
        self.device = torch.device(device)

    def shapes(self) -> dict[str, tuple[int, ...]]:
        return {n: w.shape for n, w in self.wants.items()}

    def get(self, name: str) -> torch.Tensor:
        want = self.wants[name]
        g = torch.Generator(device=self.device).manual_seed(_stream_seed(self.seed, name))
        if want.role == "int_table":
            return torch.zeros(want.shape, dtype=torch.int32, device=self.device)
        x = torch.randn(want.shape, generator=g, device=self.device, dtype=torch.float32)
        if want.role == "vector":
            return 1.0 + self.norm_std * x
        return self.std * x


def write_model_folder(
    folder: str,
    config_json: dict,
    wants: dict[str, TensorWant],
    seed: int,
    dtype: torch.dtype = torch.bfloat16,
    std: float = 0.02,
    norm_std: float = 0.01,
) -> None:
    """Write ``config.json`` and ``model.safetensors`` with seeded random weights in ``dtype``."""
    os.makedirs(folder, exist_ok=True)
    src = RandomSource(wants, seed, std, norm_std)
    tensors = {}
    for name, want in wants.items():
        t = src.get(name)
        tensors[name] = t if want.role == "int_table" else t.to(dtype)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config_json, f, indent=1)
    write_file(os.path.join(folder, "model.safetensors"), tensors, {"format": "pt", "seed": str(seed)})


def parse_shape(spec: str) -> tuple[str, dict]:
    """``ARCHITECTURE:key=value,...`` -> (architecture name, config.json keys); values are JSON
    (``true``/``false`` also capitalised)."""
    name, _, rest = spec.partition(":")
    values: dict = {}
    for pair in filter(None, rest.split(",")):
        key, eq, value = pair.partition("=")
        if not eq or not key.strip():
            raise ValueError(f"{pair!r}: key=value expected")
        text = value.strip()
        values[key.strip()] = json.loads(text.lower() if text in ("True", "False") else text)
    if not name.strip():
        raise ValueError("a shape starts with the architecture's name")
    values.setdefault("architectures", [name.strip()])
    return name.strip(), values


def random_model_folder(spec: str, seed: int, dtype: str, std: float = 0.02) -> str:
    """Write a model folder with seeded random weights for ``ARCHITECTURE:key=value,...`` (the keys of
    that architecture's config.json) into a temporary folder, which is removed when the process ends,
    and return its path."""
    import atexit
    import shutil
    import tempfile

    from .. import models as _models  # noqa: F401  (registers the architectures)
    from ..config.registry import get_architecture
    from ..parts.decoder import Decoder

    name, values = parse_shape(spec)
    entry = get_architecture(name)
    arch_config = entry.config_from_dict(values)
    folder = tempfile.mkdtemp(prefix="random_model_")
    atexit.register(shutil.rmtree, folder, True)
    wants = Decoder(entry.plan_from_config(arch_config), torch.float32, "cpu").weight_wants()
    write_model_folder(folder, arch_config.to_config_json(), wants, seed=seed,
                       dtype=torch.float32 if dtype == "float32" else torch.bfloat16, std=std)
    return folder
