"""Reading and writing safetensors files without touching tensor data early.

File layout: an 8-byte little-endian header length, a JSON header mapping each
tensor name to ``{"dtype", "shape", "data_offsets": [begin, end]}`` (offsets
relative to the end of the header), then the raw little-endian data.  A model
folder holds either ``model.safetensors`` or ``model.safetensors.index.json``
with a ``weight_map`` from tensor name to shard file.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass
from typing import Dict, Iterable, Mapping

import numpy as np
import torch

_DTYPES = {
    "F32": (torch.float32, 4),
    "BF16": (torch.bfloat16, 2),
    "F16": (torch.float16, 2),
    "F64": (torch.float64, 8),
    "I64": (torch.int64, 8),
    "I32": (torch.int32, 4),
    "I16": (torch.int16, 2),
    "I8": (torch.int8, 1),
    "U8": (torch.uint8, 1),
    "BOOL": (torch.bool, 1),
}
_NAMES = {dtype: name for name, (dtype, _) in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype_name: str
    shape: tuple
    begin: int
    end: int
    file: str

    @property
    def dtype(self) -> torch.dtype:
        try:
            return _DTYPES[self.dtype_name][0]
        except KeyError:
            raise SafetensorsError(f"{self.name}: unsupported element type {self.dtype_name}") from None

    @property
    def nbytes(self) -> int:
        return self.end - self.begin


def read_header(path: str) -> tuple[Dict[str, TensorEntry], int]:
    """Returns the tensor entries of one file and the offset where data starts."""
    size = os.path.getsize(path)
    with open(path, "rb") as handle:
        head = handle.read(8)
        if len(head) != 8:
            raise SafetensorsError(f"{path}: too short for a safetensors header")
        (length,) = struct.unpack("<Q", head)
        if length <= 0 or 8 + length > size:
            raise SafetensorsError(f"{path}: header length {length} does not fit the file")
        try:
            header = json.loads(handle.read(length).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as error:
            raise SafetensorsError(f"{path}: header is not valid JSON: {error}") from None
    entries: Dict[str, TensorEntry] = {}
    data_start = 8 + length
    for name, info in header.items():
        if name == "__metadata__":
            continue
        try:
            begin, end = info["data_offsets"]
            entry = TensorEntry(name, info["dtype"], tuple(int(d) for d in info["shape"]), int(begin), int(end), path)
        except (KeyError, TypeError, ValueError):
            raise SafetensorsError(f"{path}: malformed entry for {name!r}") from None
        if entry.dtype_name in _DTYPES:
            expected = int(np.prod(entry.shape, dtype=np.int64)) * _DTYPES[entry.dtype_name][1]
            if expected != entry.nbytes:
                raise SafetensorsError(
                    f"{path}: {name}: {entry.nbytes} bytes stored, shape {entry.shape} needs {expected}")
        if begin < 0 or end < begin or data_start + end > size:
            raise SafetensorsError(f"{path}: {name}: data range [{begin}, {end}) lies outside the file")
        entries[name] = entry
    return entries, data_start


class ModelFiles:
    """The tensors of a model folder, addressed by name, read lazily through mmap."""

    def __init__(self, model_dir: str):
        self.model_dir = model_dir
        self.entries: Dict[str, TensorEntry] = {}
        self._data_start: Dict[str, int] = {}
        self._maps: Dict[str, mmap.mmap] = {}
        single = os.path.join(model_dir, "model.safetensors")
        index = os.path.join(model_dir, "model.safetensors.index.json")
        if os.path.exists(single):
            files = [single]
        elif os.path.exists(index):
            with open(index, "r", encoding="utf-8") as handle:
                weight_map = json.load(handle).get("weight_map", {})
            files = sorted({os.path.join(model_dir, f) for f in weight_map.values()})
            if not files:
                raise SafetensorsError(f"{index}: empty weight_map")
        else:
            raise SafetensorsError(f"{model_dir}: neither model.safetensors nor model.safetensors.index.json")
        for path in files:
            entries, start = read_header(path)
            self._data_start[path] = start
            for name, entry in entries.items():
                if name in self.entries:
                    raise SafetensorsError(f"{name}: stored in both {self.entries[name].file} and {path}")
                self.entries[name] = entry

    def names(self) -> Iterable[str]:
        return self.entries.keys()

    def _map(self, path: str) -> mmap.mmap:
        if path not in self._maps:
            with open(path, "rb") as handle:
                self._maps[path] = mmap.mmap(handle.fileno(), 0, access=mmap.ACCESS_READ)
        return self._maps[path]

    def read(self, name: str) -> torch.Tensor:
        """A CPU tensor with the stored type and shape (a copy, safe after close)."""
        entry = self.entries[name]
        start = self._data_start[entry.file] + entry.begin
        raw = np.frombuffer(self._map(entry.file), dtype=np.uint8, count=entry.nbytes, offset=start)
        tensor = torch.from_numpy(raw.copy()).view(entry.dtype)
        return tensor.reshape(entry.shape)

    def close(self) -> None:
        for mapped in self._maps.values():
            mapped.close()
        self._maps.clear()


def file_digests(model_dir: str, whole_up_to: int = 1 << 30) -> list:
    """What identifies the weight files of a model folder: name, size and SHA-256 of the header (names,
    types, shapes and offsets) of each; of the whole file too if it has at most ``whole_up_to`` bytes."""
    import hashlib
    files = sorted({entry.file for entry in ModelFiles(model_dir).entries.values()})
    out = []
    for path in files:
        size = os.path.getsize(path)
        with open(path, "rb") as handle:
            length = int.from_bytes(handle.read(8), "little")
            record = {"file": os.path.basename(path), "bytes": size,
                      "header_sha256": hashlib.sha256(handle.read(length)).hexdigest()}
            if size <= whole_up_to:
                handle.seek(0)
                digest = hashlib.sha256()
                for block in iter(lambda: handle.read(1 << 22), b""):
                    digest.update(block)
                record["sha256"] = digest.hexdigest()
        out.append(record)
    return out


def write_file(path: str, tensors: Mapping[str, torch.Tensor], metadata: Mapping[str, str] | None = None) -> None:
    """Writes CPU tensors as one safetensors file, names in sorted order."""
    header: dict = {}
    if metadata:
        header["__metadata__"] = dict(metadata)
    offset = 0
    order = sorted(tensors)
    for name in order:
        tensor = tensors[name]
        if tensor.dtype not in _NAMES:
            raise SafetensorsError(f"{name}: cannot store element type {tensor.dtype}")
        nbytes = tensor.numel() * tensor.element_size()
        header[name] = {"dtype": _NAMES[tensor.dtype], "shape": list(tensor.shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as handle:
        handle.write(struct.pack("<Q", len(blob)))
        handle.write(blob)
        for name in order:
            tensor = tensors[name].detach().cpu().contiguous()
            handle.write(tensor.reshape(-1).view(torch.uint8).numpy().tobytes() if tensor.numel() else b"")
    os.replace(tmp, path)
