"""Feed-forward parts."""
from __future__ import annotations

from typing import Dict, List

import torch

from .. import ops
from ..weights.loader import MATRIX, TensorSpec
from .base import FEED_FORWARDS, Part, PartSpec
from .context import StepContext


@FEED_FORWARDS.register("swiglu")
class SwiGluMlp(Part):
    """down(silu(gate y) * (up y)), no bias, silu(g) = g / (1 + exp(-g)).

    Reference: crates/leone/src/runtime.rs:9283-9319, crates/leone/src/cpu.rs:892-907.
    Parameters: ``hidden``, ``intermediate`` and tensor names ``gate``, ``up``, ``down``.
    """

    graph_safe = True

    def __init__(self, spec: PartSpec, **_):
        p = spec.params
        self.hidden = int(p["hidden"])
        self.intermediate = int(p["intermediate"])
        self.names = {k: p[k] for k in ("gate", "up", "down")}
        self.w_gate_up = self.w_down = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.names["gate"], (self.intermediate, self.hidden), MATRIX),
                TensorSpec(self.names["up"], (self.intermediate, self.hidden), MATRIX),
                TensorSpec(self.names["down"], (self.hidden, self.intermediate), MATRIX)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        # Gate rows first, then up rows: one product, then the activation splits the columns.
        self.w_gate_up = torch.cat([tensors.pop(self.names["gate"]), tensors.pop(self.names["up"])],
                                   dim=0).contiguous()
        self.w_down = tensors.pop(self.names["down"]).contiguous()

    def forward(self, y: torch.Tensor, step: StepContext) -> torch.Tensor:
        gate_up = ops.linear(y, self.w_gate_up)
        return ops.linear(ops.swiglu(gate_up), self.w_down)
