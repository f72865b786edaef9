"""Normalisation parts."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import ops
from ..weights.loader import TensorSpec, VECTOR
from .base import NORMS, Part, PartSpec


@NORMS.register("rmsnorm")
class RmsNorm(Part):
    """y = (x * gain) / sqrt(mean(x^2) + eps); the gain multiplies directly (not 1 + gain).

    Reference: crates/leone/src/cpu.rs:1642-1663.  Parameters: ``size``, ``eps``, ``weight`` (tensor name).
    """

    graph_safe = True

    def __init__(self, spec: PartSpec, **_):
        self.size = int(spec["size"])
        self.eps = float(spec["eps"])
        self.weight_name = spec["weight"]
        self.gain: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.weight_name, (self.size,), VECTOR)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.gain = tensors[self.weight_name].contiguous()

    def add_norm(self, x: torch.Tensor, delta: Optional[torch.Tensor], out_dtype: torch.dtype,
                 rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        if isinstance(delta, ops.PreparedRows):
            delta = None                      # the product that made it has added into the stream already
        return ops.add_rmsnorm(x, delta, self.gain, self.eps, out_dtype, rows)

    def folded(self, out_dtype: torch.dtype):
        """(gain, eps, type) for a product that can leave this norm's operand behind when it adds into the
        stream (``ops.linear(..., next_norm=)``)."""
        return (self.gain, self.eps, out_dtype)

    def lazy(self, x: torch.Tensor, delta: Optional[torch.Tensor], out_dtype: torch.dtype,
             rows: Optional[torch.Tensor] = None):
        """The same, but if there is nothing to add the norm is only described (``ops.NormedRows``), so
        that the product that consumes it can carry it out itself."""
        if isinstance(delta, ops.PreparedRows):
            if rows is None and delta.gain is self.gain and delta.eps == self.eps and delta.dtype == out_dtype:
                return delta
            delta = None                      # made for another norm: the stream itself is up to date
        if delta is not None:
            return self.add_norm(x, delta, out_dtype, rows)
        return ops.NormedRows(x, self.gain, self.eps, out_dtype, rows)
