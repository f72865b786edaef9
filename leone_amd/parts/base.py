"""Interfaces of the parts a model is assembled from, and their registries.

A part is described by a ``PartSpec`` (a kind plus parameters: sizes,
constants and tensor names) and built from it by the class registered for that
kind.  Parts never look at a model configuration and do not know which model
they are in; an architecture's builder turns its configuration into specs.

Families and what each must provide
-----------------------------------
norm          ``tensor_specs()``, ``bind(tensors)``, ``add_norm(x, delta, out_dtype, rows=None)``:
              adds ``delta`` into the float32 stream ``x`` (if given) and
              returns the normalised rows in ``out_dtype``.
position      ``prepare(max_positions, device)``; what it exposes to a mixer is
              the position part's own affair (the rotary part exposes tables).
mixer         ``tensor_specs()``, ``bind(tensors)``, ``cache_need()`` -> ``KvNeed`` /
              ``StateNeed`` / ``None``, ``forward(y, step, cache)`` -> delta ``[rows, hidden]``.
feed_forward  ``tensor_specs()``, ``bind(tensors)``, ``forward(y, step)`` -> delta.
              A mixer or feed-forward that sets ``fused_io = True`` is instead called with
              ``forward(y, step[, cache], residual=x)``: ``y`` may then be an ``ops.NormedRows`` (a norm
              not yet carried out, which ``ops.linear`` folds into the product), and the part may add its
              result into the float32 stream ``residual`` itself and return None.  One that also sets
              ``prepares_next = True`` takes ``next_norm=`` (what ``RmsNorm.folded`` gives for the norm
              that runs next) and may then return ``ops.PreparedRows``: the result has been added and
              that norm's operand lies ready, so no norm kernel runs between the two products.
block         ``tensor_specs()``, ``bind(tensors)``, ``cache_need()``,
              ``forward(x, pending, step, cache)`` -> new pending delta.  Optional: ``entry_norm(dtype)``
              (what the block before may prepare) and ``prepares_next = True`` with
              ``forward(..., next_norm=)``, as above.

``x`` is the residual stream, float32 ``[rows, hidden]``; ``pending`` is a delta
not yet added to it (the next norm adds it, so add and norm are one kernel).
A delta is ``[rows, hidden]`` or a stack of planes ``[p, rows, hidden]`` whose sum
is meant (what ``ops.linear`` returns when it cut a product's inner dimension);
``ops.add_rmsnorm`` takes either, and a norm of another kind can sum the planes first.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional

import torch

from ..weights.loader import TensorSpec


@dataclass(frozen=True)
class PartSpec:
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)

    def __getitem__(self, key: str) -> Any:
        return self.params[key]

    def get(self, key: str, default: Any = None) -> Any:
        return self.params.get(key, default)


@dataclass(frozen=True)
class KvNeed:
    """A mixer that caches one key and one value vector per token and kv head."""
    kv_heads: int
    head_dim: int
    window: Optional[int] = None   # only the last `window` positions are ever read


@dataclass(frozen=True)
class StateNeed:
    """A mixer that keeps per-request state of fixed size (float32 unless said otherwise)."""
    shape: tuple
    dtype: torch.dtype = torch.float32


class Registry:
    """Kind name -> class, for one family of parts."""

    def __init__(self, family: str):
        self.family = family
        self._classes: Dict[str, Callable[..., Any]] = {}

    def register(self, kind: str, cls: Optional[Callable[..., Any]] = None):
        def add(target):
            if kind in self._classes and self._classes[kind] is not target:
                raise ValueError(f"{self.family} kind {kind!r} is already registered")
            self._classes[kind] = target
            return target
        return add(cls) if cls is not None else add

    def unregister(self, kind: str) -> None:
        self._classes.pop(kind, None)

    def build(self, spec: PartSpec, **context) -> Any:
        try:
            cls = self._classes[spec.kind]
        except KeyError:
            raise ValueError(
                f"unknown {self.family} kind {spec.kind!r}; registered: {', '.join(sorted(self._classes))}") from None
        part = cls(spec, **context)
        try:
            part.family = self.family            # what the model's byte accounting files its tensors under
        except AttributeError:
            pass
        return part

    def kinds(self) -> List[str]:
        return sorted(self._classes)


NORMS = Registry("norm")
POSITIONS = Registry("position")
MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed_forward")
BLOCKS = Registry("block")


class Part:
    """Common behaviour: a part states its tensors and later receives them.

    ``graph_safe`` says that the part's forward work depends on the step only through the
    device arrays of the StepContext and cache views (never through host-side lists, sizes
    of data or values read back), so that it can be recorded once and replayed.  A model is
    replayed from a graph only if all its parts say so.
    """
    graph_safe = False

    def tensor_specs(self) -> List[TensorSpec]:
        return []

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        pass
