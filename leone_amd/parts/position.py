"""Position encodings."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .. import ops
from .base import POSITIONS, Part, PartSpec


@POSITIONS.register("rope_half_split")
class RotaryHalfSplit(Part):
    """Rotates the pairs (i, i + D/2) of a head by pos * theta^(-2i/D).

    Reference: crates/leone/src/cpu.rs:1721-1779 (inverse frequencies and the
    rotation), pairing HalfSplit for this architecture (crates/leone/src/model.rs:299-304).
    Parameters: ``rotary_dim`` (the whole head), ``theta``.  The cos/sin table is
    evaluated in double on the device and kept as float.
    """

    graph_safe = True

    def __init__(self, spec: PartSpec, **_):
        self.rotary_dim = int(spec["rotary_dim"])
        self.theta = float(spec["theta"])
        if self.rotary_dim <= 0 or self.rotary_dim % 2:
            raise ValueError(f"rotary_dim must be even and positive, found {self.rotary_dim}")
        self.cos: Optional[torch.Tensor] = None
        self.sin: Optional[torch.Tensor] = None

    def prepare(self, max_positions: int, device) -> None:
        self.cos, self.sin = ops.rope_table(self.theta, self.rotary_dim, max_positions, device)

    def tables(self) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
        return self.cos, self.sin


@POSITIONS.register("none")
class NoPosition(Part):
    """No position encoding: queries and keys are used as projected."""

    graph_safe = True

    def __init__(self, spec: PartSpec, **_):
        pass

    def prepare(self, max_positions: int, device) -> None:
        pass

    def tables(self):
        return None, None
