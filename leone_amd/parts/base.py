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
              Optional: ``row_tiling()`` -> ``RowTiling`` if it has a kernel that works on tiles of rows.
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


# ---- what a mixer keeps between steps --------------------------------------------------------------------
# A need says what kind of storage a cache slot wants and how to make, view, clear and spoil it; the pools
# (``cache/pools.py``) know needs only through these methods, so another kind of cache is another class here
# or beside the mixer that uses it.  Two families:
#   paged = True   one entry per token, in pages handed out by the cache manager.  Slots with equal
#                  ``group_key()`` share page ids and block tables (a group); ``window`` and ``page_tokens``
#                  (None: the engine's) are the group's.  ``allocate(pages, page_tokens, dtype, device)`` ->
#                  storage, ``view(storage, block_table, page_tokens)`` -> what the mixer's forward receives,
#                  ``poison(storage, page index tensor)``, ``bytes_per_token(element size)``.
#   paged = False  storage of fixed size per request slot.  ``allocate_slots(max_requests, device)`` -> storage,
#                  ``view(storage)``, ``zero(storage, slot)``, ``snapshot(storage, slots)`` -> saved,
#                  ``restore(storage, slots, saved)`` (a failed step puts the state back).

@dataclass(frozen=True)
class KvNeed:
    """A mixer that caches one key and one value vector per token and kv head, packed in runs of 8:
    keys ``[pages, kv_heads, head_dim/8, page_tokens, 8]``, values ``[pages, kv_heads, page_tokens/8, head_dim, 8]``."""
    kv_heads: int
    head_dim: int
    window: Optional[int] = None   # only the last `window` positions are ever read
    page_tokens: Optional[int] = None   # tokens a page of this group holds; None: the engine's choice

    paged = True

    def group_key(self):
        return self

    def allocate(self, pages: int, page_tokens: int, dtype: torch.dtype, device):
        if self.head_dim % 8 or page_tokens % 8:
            raise ValueError(f"the cache packs runs of 8: head_dim {self.head_dim} and page_tokens "
                             f"{page_tokens} must be multiples of 8")
        return (torch.zeros((pages, self.kv_heads, self.head_dim // 8, page_tokens, 8), dtype=dtype, device=device),
                torch.zeros((pages, self.kv_heads, page_tokens // 8, self.head_dim, 8), dtype=dtype, device=device))

    def view(self, storage, block_table, page_tokens: int):
        from .context import KvCacheView
        return KvCacheView(writes=True, k_pool=storage[0], v_pool=storage[1], block_table=block_table,
                           page_tokens=page_tokens)

    def poison(self, storage, index: torch.Tensor) -> None:
        for pool in storage:
            pool.index_fill_(0, index, float("nan"))

    def bytes_per_token(self, element_size: int) -> int:
        return 2 * self.kv_heads * self.head_dim * element_size


@dataclass(frozen=True)
class StateNeed:
    """A mixer that keeps per-request state of fixed size (float32 unless said otherwise)."""
    shape: tuple
    dtype: torch.dtype = torch.float32

    paged = False

    def allocate_slots(self, max_requests: int, device):
        return torch.zeros((max_requests, *self.shape), dtype=self.dtype, device=device)

    def view(self, storage):
        from .context import StateCacheView
        return StateCacheView(writes=True, state=storage)

    def zero(self, storage, slot: int) -> None:
        storage[slot].zero_()

    def snapshot(self, storage, slots: torch.Tensor):
        return storage.index_select(0, slots)

    def restore(self, storage, slots: torch.Tensor, saved) -> None:
        storage.index_copy_(0, slots, saved)


@dataclass(frozen=True)
class RowTiling:
    """How a part wants long portions cut for a kernel of its own: portions of at least ``min_rows`` rows in
    tiles of ``tile_rows`` consecutive rows of one request, ``group_tiles`` tiles to a group (a portion's last
    group is filled up with tiles of no rows).  A part that declares one (``row_tiling()``) finds the tile
    list of every step in ``StepContext.tiled[tiling]``; the step's layout knows nothing else about it."""
    tile_rows: int
    group_tiles: int
    min_rows: int


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

    def streamed_weights(self) -> List[torch.Tensor]:
        """The matrices this part hands to ``ops.linear`` as weights in decode steps, every one streamed
        through once a step: the model may keep a second copy of them in the order the weight-streaming
        kernels read fastest (``ops.keep_streamed_copy``).  Naming none is always right."""
        return []
