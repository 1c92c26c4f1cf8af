"""Reading and writing the safetensors container: 8-byte little-endian header length, a JSON
header ``{name: {dtype, shape, data_offsets}}``, then the raw little-endian tensor bytes.

Files are memory-mapped, so a tensor's bytes are read from disk only when it is copied to the GPU.
"""

from __future__ import annotations

import glob
import json
import os
import struct
from dataclasses import dataclass

import numpy as np
import torch

# safetensors dtype tag -> (numpy dtype used to view the bytes, torch dtype of the result)
_DTYPES = {
    "F32": (np.float32, torch.float32),
    "F16": (np.float16, torch.float16),
    "BF16": (np.uint16, torch.bfloat16),
    "F64": (np.float64, torch.float64),
    "I64": (np.int64, torch.int64),
    "I32": (np.int32, torch.int32),
    "I16": (np.int16, torch.int16),
    "I8": (np.int8, torch.int8),
    "U8": (np.uint8, torch.uint8),
    "BOOL": (np.bool_, torch.bool),
}
_TAG_OF_TORCH = {v[1]: k for k, v in _DTYPES.items()}


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: str
    shape: tuple[int, ...]
    file: str
    begin: int  # absolute byte offset in the file
    end: int


def read_header(path: str) -> dict[str, TensorEntry]:
    with open(path, "rb") as f:
        raw = f.read(8)
        if len(raw) != 8:
            raise ValueError(f"{path}: too short to be a safetensors file")
        (n,) = struct.unpack("<Q", raw)
        size = os.path.getsize(path)
        if n > size - 8:
            raise ValueError(f"{path}: header length {n} exceeds the file size")
        header = json.loads(f.read(n).decode("utf-8"))
    base = 8 + n
    entries = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        tag = info["dtype"]
        if tag not in _DTYPES:
            raise ValueError(f"{path}: tensor {name!r} has unsupported dtype {tag}")
        b, e = (int(v) for v in info["data_offsets"])
        shape = tuple(int(s) for s in info["shape"])
        want = int(np.prod(shape, dtype=np.int64)) * np.dtype(_DTYPES[tag][0]).itemsize
        if min(shape, default=0) < 0 or b < 0 or e < b or e - b != want or base + e > size:
            raise ValueError(f"{path}: tensor {name!r} has inconsistent offsets {b}..{e} for shape {shape}")
        entries[name] = TensorEntry(name, tag, shape, path, base + b, base + e)
    return entries


def read_folder_header(folder: str) -> dict[str, TensorEntry]:
    """All tensors of every ``*.safetensors`` in the folder, files in sorted order, later files
    overriding earlier ones (as the reference merges them, ``src/mini_engine/engine.py:126-128``)."""
    files = sorted(glob.glob(os.path.join(folder, "*.safetensors")))
    if not files:
        raise FileNotFoundError(f"{folder!r} holds no *.safetensors file")
    merged: dict[str, TensorEntry] = {}
    for path in files:
        merged.update(read_header(path))
    return merged


class TensorReader:
    """Memory-maps each file once and hands out CPU tensors that view the mapping."""

    def __init__(self) -> None:
        self._maps: dict[str, np.memmap] = {}

    def read(self, entry: TensorEntry) -> torch.Tensor:
        mm = self._maps.get(entry.file)
        if mm is None:
            mm = np.memmap(entry.file, dtype=np.uint8, mode="r")
            self._maps[entry.file] = mm
        np_dtype, torch_dtype = _DTYPES[entry.dtype]
        flat = np.frombuffer(mm, dtype=np_dtype, count=(entry.end - entry.begin) // np.dtype(np_dtype).itemsize,
                             offset=entry.begin)
        # The mapping is read-only; torch only warns about that, and the tensor is copied to the
        # device before anything could write to it.
        import warnings

        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            t = torch.from_numpy(flat)
        if torch_dtype is torch.bfloat16:
            t = t.view(torch.bfloat16)
        return t.reshape(entry.shape)


def write_file(path: str, tensors: dict[str, torch.Tensor], metadata: dict[str, str] | None = None) -> None:
    """Write CPU tensors in the order of the dictionary."""
    header: dict[str, object] = {}
    if metadata:
        header["__metadata__"] = metadata
    offset = 0
    blobs = []
    for name, t in tensors.items():
        t = t.detach().contiguous().cpu()
        if t.dtype not in _TAG_OF_TORCH:
            raise ValueError(f"tensor {name!r}: dtype {t.dtype} cannot be written")
        raw = t.view(torch.uint8).numpy().tobytes() if t.numel() else b""
        header[name] = {"dtype": _TAG_OF_TORCH[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + len(raw)]}
        offset += len(raw)
        blobs.append(raw)
    head = json.dumps(header, separators=(",", ":")).encode("utf-8")
    head += b" " * ((8 - len(head) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(head)))
        f.write(head)
        for raw in blobs:
            f.write(raw)
