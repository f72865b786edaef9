"""Binding tensors to a model by name.

The model's parts say which tensors they need (name, shape, role).  The loader
compares that list with what a model folder (or an in-memory dictionary) holds
and reports every problem in one error: missing tensors, unexpected tensors and
wrong shapes.  The reference does the same checks one error at a time
(crates/leone/src/model.rs:1060-1075 missing and shape, :684-714 unexpected).

Element types: with a bfloat16 engine, matrices and embedding tables are kept
in bfloat16 and vectors (norm gains) keep the type the file stores, so a gain
stored in 32-bit stays 32-bit; integer tables become int32.  With a float32
engine every floating tensor is widened to float32, which is exact for
bfloat16 data.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Iterable, List, Mapping

import torch

from .safetensors_io import ModelFiles, SafetensorsError

MATRIX, VECTOR, INT_TABLE = "matrix", "vector", "int_table"
_FLOATS = (torch.float32, torch.bfloat16, torch.float16, torch.float64)


@dataclass(frozen=True)
class TensorSpec:
    """One tensor a part needs: its name in the file, its shape and its role."""
    name: str
    shape: tuple
    role: str = MATRIX
    optional: bool = False


class WeightsError(ValueError):
    """Tensors of a model folder do not match what the model needs."""

    def __init__(self, source: str, missing: List[str], unexpected: List[str], wrong_shape: List[str],
                 wrong_type: List[str]):
        self.missing, self.unexpected = missing, unexpected
        self.wrong_shape, self.wrong_type = wrong_shape, wrong_type
        lines = [f"weights in {source} do not match the model:"]
        for title, items in (("missing", missing), ("unexpected", unexpected), ("wrong shape", wrong_shape),
                             ("wrong type", wrong_type)):
            if items:
                lines.append(f"  {title} ({len(items)}):")
                lines.extend(f"    {item}" for item in items)
        super().__init__("\n".join(lines))


def target_dtype(stored: torch.dtype, role: str, engine_dtype: torch.dtype) -> torch.dtype:
    if role == INT_TABLE:
        return torch.int32
    if engine_dtype == torch.float32:
        return torch.float32
    if role == VECTOR and stored == torch.float32:
        return torch.float32
    return engine_dtype


def check(specs: Iterable[TensorSpec], found: Mapping[str, tuple], source: str,
          ignore: Iterable[str] = ()) -> None:
    """``found`` maps name -> (shape, dtype).  Raises one WeightsError listing every mismatch."""
    specs = list(specs)
    wanted = {spec.name: spec for spec in specs}
    ignored = set(ignore)
    missing = [s.name + f" {tuple(s.shape)}" for s in specs if s.name not in found and not s.optional]
    unexpected = sorted(name for name in found if name not in wanted and name not in ignored)
    wrong_shape, wrong_type = [], []
    for name, spec in wanted.items():
        if name not in found:
            continue
        shape, dtype = found[name]
        if tuple(shape) != tuple(spec.shape):
            wrong_shape.append(f"{name}: expected {tuple(spec.shape)}, found {tuple(shape)}")
        if spec.role == INT_TABLE:
            if dtype in _FLOATS or dtype == torch.bool:
                wrong_type.append(f"{name}: expected an integer type, found {dtype}")
        elif dtype not in (torch.float32, torch.bfloat16):
            wrong_type.append(f"{name}: expected float32 or bfloat16, found {dtype}")
    if missing or unexpected or wrong_shape or wrong_type:
        raise WeightsError(source, missing, unexpected, wrong_shape, wrong_type)


def load_from_dir(model_dir: str, specs: Iterable[TensorSpec], engine_dtype: torch.dtype, device,
                  ignore: Iterable[str] = ()) -> Dict[str, torch.Tensor]:
    specs = list(specs)
    try:
        files = ModelFiles(model_dir)
    except SafetensorsError as error:
        raise WeightsError(model_dir, [str(error)], [], [], []) from None
    try:
        found = {}
        for name, entry in files.entries.items():
            try:
                found[name] = (entry.shape, entry.dtype)
            except SafetensorsError:
                found[name] = (entry.shape, entry.dtype_name)
        check(specs, found, model_dir, ignore)
        out: Dict[str, torch.Tensor] = {}
        for spec in specs:
            if spec.name not in files.entries:
                continue
            tensor = files.read(spec.name)
            out[spec.name] = tensor.to(target_dtype(tensor.dtype, spec.role, engine_dtype)).to(device)
        return out
    finally:
        files.close()


def load_from_tensors(tensors: Mapping[str, torch.Tensor], specs: Iterable[TensorSpec],
                      engine_dtype: torch.dtype, device, source: str = "memory",
                      ignore: Iterable[str] = ()) -> Dict[str, torch.Tensor]:
    specs = list(specs)
    check(specs, {n: (tuple(t.shape), t.dtype) for n, t in tensors.items()}, source, ignore)
    out = {}
    for spec in specs:
        if spec.name in tensors:
            t = tensors[spec.name]
            out[spec.name] = t.to(device=device, dtype=target_dtype(t.dtype, spec.role, engine_dtype))
    return out
