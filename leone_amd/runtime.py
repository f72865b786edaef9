"""Loading a model: config.json -> typed configuration -> parts -> weights bound by name."""
from __future__ import annotations

from typing import Optional, Union

import torch

from .architectures import config_from_dict, config_from_dir, model_spec_for
from .parts.model import DecoderModel
from .weights import loader, random_init

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
           "f32": torch.float32}


def parse_dtype(name: Union[str, torch.dtype]) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"engine type must be bfloat16 or float32, found {name}")
        return name
    try:
        return _DTYPES[name]
    except KeyError:
        raise ValueError(f"unknown dtype {name!r}; use bfloat16 or float32") from None


def require_gpu(device: Optional[str] = None) -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU is visible; this engine has no CPU path")
    return torch.device(device or "cuda:0")


def load_model(model_dir: str, dtype: Union[str, torch.dtype] = "bfloat16", device: Optional[str] = None) -> DecoderModel:
    """Builds the model that config.json names and binds the folder's safetensors to it."""
    dev = require_gpu(device)
    config = config_from_dir(model_dir)
    spec = model_spec_for(config)
    model = DecoderModel(spec, parse_dtype(dtype), dev)
    model.config = config
    tensors = loader.load_from_dir(model_dir, model.tensor_specs(), model.dtype, dev, ignore=spec.ignore_tensors)
    model.bind(tensors)
    return model


def random_model(config, seed: int = 0, dtype: Union[str, torch.dtype] = "bfloat16",
                 device: Optional[str] = None) -> DecoderModel:
    """A model of ``config`` (a typed configuration or a config.json mapping) with seeded random weights on the GPU."""
    dev = require_gpu(device)
    if isinstance(config, dict):
        config = config_from_dict(config)
    model = DecoderModel(model_spec_for(config), parse_dtype(dtype), dev)
    model.config = config
    specs = model.tensor_specs()
    tensors = random_init.device_tensors(specs, seed, model.dtype if model.dtype == torch.bfloat16 else torch.float32, dev)
    model.bind(loader.load_from_tensors(tensors, specs, model.dtype, dev, source="random weights"))
    return model
