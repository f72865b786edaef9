"""Random weights from a configuration and a seed.

Matrices and embedding tables are drawn from N(0, 0.02), norm gains from
1 + N(0, 0.02).  Each tensor has its own generator keyed by (seed, tensor name),
so a tensor's values do not depend on which other tensors exist or in which
order they are made.  ``write_model_dir`` writes a model folder (config.json,
model.safetensors) that loads like any other; ``device_tensors`` makes the same
kind of weights directly on the GPU for models too large to be worth a file.
"""
from __future__ import annotations

import json
import os
import zlib
from typing import Dict, Iterable

import numpy as np
import torch

from .loader import INT_TABLE, VECTOR, TensorSpec
from .safetensors_io import write_file

STD = 0.02


def _key(seed: int, name: str) -> list:
    return [int(seed) & 0xFFFFFFFFFFFFFFFF, zlib.crc32(name.encode("utf-8"))]


def host_tensor(spec: TensorSpec, seed: int, dtype: torch.dtype) -> torch.Tensor:
    rng = np.random.Generator(np.random.Philox(key=_key(seed, spec.name)))
    if spec.role == INT_TABLE:
        raise ValueError(f"{spec.name}: no rule for random integer tables")
    values = rng.standard_normal(size=spec.shape, dtype=np.float32) * np.float32(STD)
    if spec.role == VECTOR:
        values += np.float32(1.0)
    return torch.from_numpy(values).to(dtype)


def host_tensors(specs: Iterable[TensorSpec], seed: int, dtype: torch.dtype) -> Dict[str, torch.Tensor]:
    return {spec.name: host_tensor(spec, seed, dtype) for spec in specs}


def device_tensors(specs: Iterable[TensorSpec], seed: int, dtype: torch.dtype, device) -> Dict[str, torch.Tensor]:
    out = {}
    for spec in specs:
        gen = torch.Generator(device=device)
        gen.manual_seed((int(seed) * 1000003 + zlib.crc32(spec.name.encode("utf-8"))) & 0x7FFFFFFFFFFFFFFF)
        t = torch.randn(spec.shape, generator=gen, device=device, dtype=torch.float32) * STD
        if spec.role == VECTOR:
            t += 1.0
        out[spec.name] = t.to(dtype)
        del t
    return out


def write_model_dir(path: str, config, seed: int, dtype: torch.dtype = torch.bfloat16) -> str:
    """Writes config.json and model.safetensors for ``config`` with weights from ``seed``."""
    from ..architectures import model_spec_for
    from ..parts.model import DecoderModel

    if dtype not in (torch.float32, torch.bfloat16):
        raise ValueError(f"weights are stored as float32 or bfloat16, not {dtype}")
    os.makedirs(path, exist_ok=True)
    raw = config.to_dict()
    raw["torch_dtype"] = "bfloat16" if dtype == torch.bfloat16 else "float32"
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as handle:
        json.dump(raw, handle, indent=2)
    specs = DecoderModel(model_spec_for(config), torch.float32, "cpu").tensor_specs()
    write_file(os.path.join(path, "model.safetensors"), host_tensors(specs, seed, dtype),
               metadata={"format": "pt", "seed": str(seed)})
    return path
