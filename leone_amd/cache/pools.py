"""Device storage behind the cache manager: pages per group, state per slot."""
from __future__ import annotations

from typing import Dict, List, Union

import torch

from ..parts.context import CacheView
from .manager import GroupSpec


class DevicePools:
    """Allocates, once, the tensors that layer runs read and write.

    What a cache slot holds is its need's affair (``parts/base.py``: ``KvNeed``, ``StateNeed``, or any class
    with the same methods): the pools only sort the slots.  Paged needs with the same ``group_key()`` form one
    group and share page ids and block tables, each slot with storage of its own; a group's pages hold
    the need's ``page_tokens`` tokens, or the engine's if it names none.  The other needs get storage per
    request slot.
    """

    def __init__(self, needs: Dict[int, object], dtype: torch.dtype, device, num_pages: Union[int, Dict[int, int]],
                 page_tokens: int, max_requests: int):
        self.dtype, self.device = dtype, torch.device(device)
        self.page_tokens = page_tokens
        self.needs = dict(needs)
        self.group_needs: List[object] = []
        self.group_of_slot: Dict[int, int] = {}
        self.paged: Dict[int, object] = {}        # slot -> storage of a paged need
        self.state: Dict[int, object] = {}        # slot -> storage of a per-request need
        for slot in sorted(needs):
            need = needs[slot]
            if not hasattr(need, "paged"):
                raise TypeError(f"cache slot {slot}: {need!r} is no cache need (see parts/base.py)")
            if need.paged:
                key = need.group_key()
                if key not in [n.group_key() for n in self.group_needs]:
                    self.group_needs.append(need)
                self.group_of_slot[slot] = [n.group_key() for n in self.group_needs].index(key)
            else:
                self.state[slot] = need.allocate_slots(max_requests, self.device)
        self.group_specs: List[GroupSpec] = []
        for gi, need in enumerate(self.group_needs):
            pages = num_pages[gi] if isinstance(num_pages, dict) else num_pages
            self.group_specs.append(GroupSpec(pages, getattr(need, "page_tokens", None) or page_tokens,
                                              getattr(need, "window", None)))
        for slot, gi in self.group_of_slot.items():
            spec = self.group_specs[gi]
            self.paged[slot] = needs[slot].allocate(spec.num_pages, spec.page_tokens, dtype, self.device)

    @property
    def kv(self) -> Dict[int, tuple]:
        """slot -> (key pool, value pool) of the slots whose need is a ``KvNeed``."""
        return {slot: storage for slot, storage in self.paged.items() if isinstance(storage, tuple) and len(storage) == 2}

    def bytes_per_token(self) -> int:
        size = torch.empty((), dtype=self.dtype).element_size()
        return sum(self.needs[slot].bytes_per_token(size) for slot in self.group_of_slot)

    def views(self, block_tables: Dict[int, torch.Tensor]) -> Dict[int, CacheView]:
        out: Dict[int, CacheView] = {}
        for slot, gi in self.group_of_slot.items():
            out[slot] = self.needs[slot].view(self.paged[slot], block_tables[gi], self.group_specs[gi].page_tokens)
        for slot, storage in self.state.items():
            out[slot] = self.needs[slot].view(storage)
        return out

    def zero_state(self, slot_index: int) -> None:
        for slot, storage in self.state.items():
            self.needs[slot].zero(storage, slot_index)

    def copy_state(self, from_slot: int, to_slot: int) -> None:
        """Gives request slot ``to_slot`` a copy of what ``from_slot`` holds (a request that takes over another's
        prefix at the other's latest position), through the needs' own ``snapshot`` and ``restore``."""
        source = torch.tensor([from_slot], dtype=torch.long, device=self.device)
        target = torch.tensor([to_slot], dtype=torch.long, device=self.device)
        for slot, storage in self.state.items():
            self.needs[slot].restore(storage, target, self.needs[slot].snapshot(storage, source))

    def snapshot_state(self, slot_indices: List[int]):
        """What the per-request storage of these request slots holds, to be put back by ``restore_state``."""
        if not self.state:
            return None
        index = torch.tensor(sorted(set(slot_indices)), dtype=torch.long, device=self.device)
        return index, {slot: self.needs[slot].snapshot(storage, index) for slot, storage in self.state.items()}

    def restore_state(self, saved) -> None:
        if saved is None:
            return
        index, kept = saved
        for slot, value in kept.items():
            self.needs[slot].restore(self.state[slot], index, value)

    def poison_pages(self, group: int, pages: List[int]) -> None:
        """Fills pages with NaN so that a read of a page that was given back shows up."""
        if not pages:
            return
        index = torch.tensor(pages, dtype=torch.long, device=self.device)
        for slot, gi in self.group_of_slot.items():
            if gi == group:
                self.needs[slot].poison(self.paged[slot], index)
