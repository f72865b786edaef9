"""How norm, mixer and feed-forward are arranged in one layer."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..weights.loader import TensorSpec
from .base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, Part, PartSpec
from .context import CacheView, StepContext


@BLOCKS.register("prenorm")
class PreNormBlock(Part):
    """x1 = x + mixer(norm1(x)); x2 = x1 + feed_forward(norm2(x1)).

    Reference layer order: crates/leone/src/runtime.rs:9019-9050.
    Parameters: ``norm1``, ``mixer``, ``norm2``, ``feed_forward`` (part specs).
    The residual stream is float32; each delta is added by the following norm's
    kernel, so the block returns its last delta instead of adding it.
    """

    def __init__(self, spec: PartSpec, **context):
        self.norm1 = NORMS.build(spec["norm1"], **context)
        self.mixer = MIXERS.build(spec["mixer"], **context)
        self.norm2 = NORMS.build(spec["norm2"], **context)
        self.feed_forward = FEED_FORWARDS.build(spec["feed_forward"], **context)

    def parts(self):
        return (self.norm1, self.mixer, self.norm2, self.feed_forward)

    @property
    def graph_safe(self) -> bool:
        return all(getattr(part, "graph_safe", False) for part in self.parts())

    def tensor_specs(self) -> List[TensorSpec]:
        return [s for part in self.parts() for s in part.tensor_specs()]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for part in self.parts():
            part.bind(tensors)

    def streamed_weights(self) -> List[torch.Tensor]:
        return [w for part in self.parts() if hasattr(part, "streamed_weights") for w in part.streamed_weights()]

    def cache_need(self):
        return self.mixer.cache_need()

    def row_tilings(self):
        """The tilings its parts declare (``RowTiling``)."""
        return [part.row_tiling() for part in self.parts() if hasattr(part, "row_tiling")]

    prepares_next = True

    def entry_norm(self, out_dtype):
        """What the block before may prepare for this block's first norm (``RmsNorm.folded``), or None."""
        if getattr(self.mixer, "fused_io", False) and hasattr(self.norm1, "folded"):
            return self.norm1.folded(out_dtype)
        return None

    def forward(self, x: torch.Tensor, pending, step: StepContext, cache: Optional[CacheView], next_norm=None):
        """Returns the delta that is still to be added to ``x``, None if everything has been added, or, if
        ``next_norm`` (the next block's ``entry_norm``) was given and the last product could do it, that
        norm's operand (``ops.PreparedRows``; everything has been added then)."""
        y = self._normed(self.norm1, x, pending, step, self.mixer)
        if getattr(self.mixer, "fused_io", False):
            inner = None
            if getattr(self.mixer, "prepares_next", False) and getattr(self.feed_forward, "fused_io", False) \
                    and hasattr(self.norm2, "folded"):
                inner = self.norm2.folded(step.dtype)
            delta = (self.mixer.forward(y, step, cache, residual=x, next_norm=inner) if inner is not None
                     else self.mixer.forward(y, step, cache, residual=x))
        else:
            delta = self.mixer.forward(y, step, cache)
        y = self._normed(self.norm2, x, delta, step, self.feed_forward)
        if getattr(self.feed_forward, "fused_io", False):
            if next_norm is not None and getattr(self.feed_forward, "prepares_next", False):
                return self.feed_forward.forward(y, step, residual=x, next_norm=next_norm)
            return self.feed_forward.forward(y, step, residual=x)
        return self.feed_forward.forward(y, step)

    @staticmethod
    def _normed(norm, x, delta, step, consumer):
        # A consumer with fused_io takes a norm that is only described and may fold it into its first
        # product; any other gets the normalised rows.
        if getattr(consumer, "fused_io", False) and hasattr(norm, "lazy"):
            return norm.lazy(x, delta, step.dtype)
        return norm.add_norm(x, delta, step.dtype)
