"""What a step hands to the parts: row metadata on the device and cache views.

A step runs ``rows`` tokens as one batch.  Row r belongs to entry
``row_entry[r]`` (one entry per request in the step) and sits at absolute
position ``positions[r]`` of that request.  Parts see only these arrays, the
block tables of their cache group and the state slots; they never see requests.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch


@dataclass(frozen=True)
class EntryInfo:
    """Host-side description of one request's share of a step."""
    request: object
    slot: int          # per-request state slot
    first_row: int     # index of its first row in the step
    count: int         # number of rows (tokens) it brings
    start: int         # absolute position of its first row


@dataclass
class TiledRows:
    """What a step holds for one ``RowTiling``: rows [0, rows) belong to the portions it cuts, ``tiles`` is
    int32 [n, 3] (entry, first row, rows) in groups, places of no rows filling a group up."""
    rows: int
    tiles: torch.Tensor
    mean_keys: int = 0                 # positions a row of these portions looks back on, on average (a hint for grids)


@dataclass
class StepContext:
    rows: int
    dtype: torch.dtype                 # activation type of the engine
    device: torch.device
    positions: torch.Tensor            # int32 [rows]
    row_entry: torch.Tensor            # int32 [rows]
    entries: List[EntryInfo]
    entry_slots: torch.Tensor          # int32 [entries]: state slot of each entry
    want_rows: Optional[torch.Tensor]  # int32 [wanted] rows whose logits are asked for
    block_tables: Dict[int, torch.Tensor] = field(default_factory=dict)  # group -> int32 [entries, max_blocks]
    max_position: int = 0              # largest position in the step (an upper bound when the step is replayed)
    decode_only: bool = False          # every entry brings exactly one row
    # Long portions come first in a step.  For every tiling a part of the model declared (``RowTiling``) that
    # cuts at least one portion of this step: the tile list and the rows it covers.
    tiled: Dict[object, TiledRows] = field(default_factory=dict)


@dataclass
class CacheView:
    """The cache a layer run works on."""
    writes: bool = True


@dataclass
class KvCacheView(CacheView):
    k_pool: torch.Tensor = None        # [pages, kv_heads, head_dim / 8, page_tokens, 8]
    v_pool: torch.Tensor = None        # [pages, kv_heads, page_tokens / 8, head_dim, 8]
    block_table: torch.Tensor = None   # int32 [entries, max_blocks] of the layer's group
    page_tokens: int = 0


@dataclass
class StateCacheView(CacheView):
    state: torch.Tensor = None         # [slots, *shape]: row entry_slots[e] belongs to entry e
