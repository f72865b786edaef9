"""Feed-forward parts."""
from __future__ import annotations

from typing import Dict, List, Optional

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

    fused_io = True
    prepares_next = True

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        # One product for gate and up: 8 gate rows, their 8 up rows, and so on (a pure re-layout), which
        # lets the activation be applied where the product is finished.  An intermediate size that is no
        # multiple of 8 is filled up with zero rows; they give silu(0) * 0 = 0 and meet zero columns of
        # the down projection, so the result is unchanged.
        gate, up, down = (tensors.pop(self.names[k]) for k in ("gate", "up", "down"))
        pad = -self.intermediate % 8
        if pad:
            gate = torch.nn.functional.pad(gate, (0, 0, 0, pad))
            up = torch.nn.functional.pad(up, (0, 0, 0, pad))
            down = torch.nn.functional.pad(down, (0, pad))
        self.w_gate_up = ops.interleave_gate_up(gate, up).contiguous()
        self.w_down = down.contiguous()

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_gate_up, self.w_down]

    def forward(self, y, step: StepContext, residual: Optional[torch.Tensor] = None, next_norm=None):
        """``y`` may be a norm still to be done; with ``residual`` the result may be added there (None returned),
        and with ``next_norm`` the norm that follows may come back prepared (see ``ops.linear``)."""
        activated = ops.linear(y, self.w_gate_up, gated=True)
        return ops.linear(activated, self.w_down, residual=residual, next_norm=next_norm)
