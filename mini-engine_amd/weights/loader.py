"""Loading a model's tensors by their checkpoint names, with one error for everything that is wrong.

The model states what it expects as ``{name: TensorWant(shape, role)}``; the source (a folder of
safetensors, or a seeded random generator) provides tensors by name. Roles decide the dtype a
tensor gets on the device:

* ``matrix`` (projection and embedding tables): the compute dtype (bfloat16 stays bfloat16 in a
  bfloat16 engine; the 32-bit engine up-casts, which is exact);
* ``vector`` (norm weights and other small 1-D parameters): always float32, so a tensor stored in
  32-bit stays so and a bfloat16 one is up-cast exactly;
* ``int_table``: int32.

Mirrors the strictness of the reference's ``load_state_dict(strict=True)``
(``src/mini_engine/model.py:190-195``): missing, unexpected and wrongly shaped tensors are all
errors. A tied head drops a stored ``lm_head.weight`` as the reference does.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Iterable

import torch

from .safetensors_io import TensorEntry, TensorReader, read_folder_header

ROLES = ("matrix", "vector", "int_table")


@dataclass(frozen=True)
class TensorWant:
    shape: tuple[int, ...]
    role: str = "matrix"

    def __post_init__(self) -> None:
        if self.role not in ROLES:
            raise ValueError(f"unknown tensor role {self.role!r}")


class WeightError(ValueError):
    """Raised once per load with every problem listed."""

    def __init__(self, missing: list[str], unexpected: list[str], wrong_shape: list[str]):
        self.missing, self.unexpected, self.wrong_shape = missing, unexpected, wrong_shape
        parts = []
        if missing:
            parts.append(f"missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            parts.append(f"unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong_shape:
            parts.append(f"wrong shapes ({len(wrong_shape)}): " + "; ".join(wrong_shape))
        super().__init__("checkpoint does not match the model: " + " | ".join(parts))


def check_names_and_shapes(
    wants: dict[str, TensorWant], have: dict[str, tuple[int, ...]], ignorable: Iterable[str] = ()
) -> None:
    ignorable = set(ignorable)
    missing = sorted(n for n in wants if n not in have)
    unexpected = sorted(n for n in have if n not in wants and n not in ignorable)
    wrong = sorted(
        f"{n}: stored {list(have[n])}, model wants {list(w.shape)}"
        for n, w in wants.items()
        if n in have and tuple(have[n]) != tuple(w.shape)
    )
    if missing or unexpected or wrong:
        raise WeightError(missing, unexpected, wrong)


def device_dtype_for(role: str, compute_dtype: torch.dtype) -> torch.dtype:
    if role == "matrix":
        return compute_dtype
    if role == "vector":
        return torch.float32
    return torch.int32


class FolderSource:
    """Tensors of a model folder (every ``*.safetensors`` in it)."""

    def __init__(self, folder: str):
        self.folder = folder
        self.entries: dict[str, TensorEntry] = read_folder_header(folder)
        self._reader = TensorReader()

    def shapes(self) -> dict[str, tuple[int, ...]]:
        return {n: e.shape for n, e in self.entries.items()}

    def get(self, name: str) -> torch.Tensor:
        return self._reader.read(self.entries[name])


def load_tensors(
    source,
    wants: dict[str, TensorWant],
    compute_dtype: torch.dtype,
    device: torch.device | str,
    ignorable: Iterable[str] = (),
    progress: Callable[[str], None] | None = None,
) -> dict[str, torch.Tensor]:
    """Check the source against ``wants``, then copy every wanted tensor to the device."""
    check_names_and_shapes(wants, source.shapes(), ignorable)
    out: dict[str, torch.Tensor] = {}
    for i, (name, want) in enumerate(wants.items()):
        t = source.get(name)
        out[name] = t.to(device=device, dtype=device_dtype_for(want.role, compute_dtype)).contiguous()
        if progress is not None and i % 64 == 0:
            progress(f"loaded {i + 1}/{len(wants)} tensors")
    return out
