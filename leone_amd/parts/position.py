"""Position encodings."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from .. import ops
from .base import POSITIONS, Part, PartSpec


@dataclass(frozen=True)
class Rotation:
    """What a rotary position part hands to a mixer: the rotation's whole shape, so that the mixer and its
    kernels assume none.  ``cos`` and ``sin`` are float32 ``[positions, rotary_dim / 2]`` (None: no rotation);
    the first ``rotary_dim`` elements of a head are rotated, the rest is left alone; ``pairing`` says which two
    elements turn together: "half_split" (i, i + rotary_dim / 2) or "adjacent" (2 i, 2 i + 1)
    (crates/leone/src/cpu.rs:1765-1774)."""
    cos: Optional[torch.Tensor]
    sin: Optional[torch.Tensor]
    pairing: str = "half_split"
    elements: Optional[int] = None     # rotary_dim, for a part that knows it before its tables are made

    @property
    def rotary_dim(self) -> int:
        """How many elements of a head are rotated (0: none)."""
        if self.elements is not None:
            return self.elements
        return 0 if self.cos is None else 2 * self.cos.shape[1]


def rotation_of(position) -> Rotation:
    """The rotation of a position part: what its ``rotation()`` says, or, for a part that only has
    ``tables()``, those tables in half-split pairs; no part, no rotation."""
    if position is None:
        return Rotation(None, None)
    if hasattr(position, "rotation"):
        return position.rotation()
    return Rotation(*position.tables())


@POSITIONS.register("rope_half_split")
class RotaryHalfSplit(Part):
    """Rotates the pairs (i, i + R/2) of a head's first R elements by pos * theta^(-2i/R).

    Reference: crates/leone/src/cpu.rs:1721-1779 (inverse frequencies and the
    rotation), pairing HalfSplit for this architecture (crates/leone/src/model.rs:299-304).
    Parameters: ``rotary_dim`` (R; the whole head for this architecture, fewer elements leave the rest of
    the head unrotated), ``theta``.  The cos/sin table is evaluated in double on the device and kept as float.
    """

    graph_safe = True
    pairing = "half_split"

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

    def rotation(self) -> Rotation:
        return Rotation(self.cos, self.sin, self.pairing, self.rotary_dim)


@POSITIONS.register("rope_adjacent")
class RotaryAdjacent(RotaryHalfSplit):
    """The same angles on the pairs (2i, 2i + 1) (the reference's Adjacent pairing, crates/leone/src/cpu.rs:1765-1774)."""

    pairing = "adjacent"


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

    def rotation(self) -> Rotation:
        return Rotation(None, None)
