"""Device storage behind the cache manager: key/value pages per group, state per slot."""
from __future__ import annotations

from typing import Dict, List, Union

import torch

from ..parts.base import KvNeed, StateNeed
from ..parts.context import CacheView, KvCacheView, StateCacheView
from .manager import GroupSpec


class DevicePools:
    """Allocates, once, the tensors that layer runs read and write.

    Cache slots with the same key/value need (heads, head size, window) form one
    group and share page ids and block tables; each slot has its own key and
    value tensor, packed in runs of 8 (keys ``[pages, kv_heads, head_dim/8, page_tokens, 8]``,
    values ``[pages, kv_heads, page_tokens/8, head_dim, 8]``).  A slot with a state
    need gets ``[max_requests, *shape]``.
    """

    def __init__(self, needs: Dict[int, object], dtype: torch.dtype, device, num_pages: Union[int, Dict[int, int]],
                 page_tokens: int, max_requests: int):
        self.dtype, self.device = dtype, torch.device(device)
        self.page_tokens = page_tokens
        self.group_needs: List[KvNeed] = []
        self.group_of_slot: Dict[int, int] = {}
        self.kv: Dict[int, tuple] = {}
        self.state: Dict[int, torch.Tensor] = {}
        for slot in sorted(needs):
            need = needs[slot]
            if isinstance(need, KvNeed):
                if need not in self.group_needs:
                    self.group_needs.append(need)
                self.group_of_slot[slot] = self.group_needs.index(need)
            elif isinstance(need, StateNeed):
                self.state[slot] = torch.zeros((max_requests, *need.shape), dtype=need.dtype, device=self.device)
            else:
                raise TypeError(f"cache slot {slot}: unknown need {need!r}")
        self.group_specs: List[GroupSpec] = []
        for gi, need in enumerate(self.group_needs):
            pages = num_pages[gi] if isinstance(num_pages, dict) else num_pages
            self.group_specs.append(GroupSpec(pages, page_tokens, need.window))
        for slot, gi in self.group_of_slot.items():
            need, pages = self.group_needs[gi], self.group_specs[gi].num_pages
            # keys [page][head][element / 8][token][8]; values [page][head][token / 8][element][8]
            if need.head_dim % 8 or page_tokens % 8:
                raise ValueError(f"the cache packs runs of 8: head_dim {need.head_dim} and page_tokens "
                                 f"{page_tokens} must be multiples of 8")
            self.kv[slot] = (torch.zeros((pages, need.kv_heads, need.head_dim // 8, page_tokens, 8), dtype=dtype,
                                         device=self.device),
                             torch.zeros((pages, need.kv_heads, page_tokens // 8, need.head_dim, 8), dtype=dtype,
                                         device=self.device))

    def bytes_per_token(self) -> int:
        size = torch.empty((), dtype=self.dtype).element_size()
        return sum(2 * self.group_needs[g].kv_heads * self.group_needs[g].head_dim * size
                   for g in self.group_of_slot.values())

    def views(self, block_tables: Dict[int, torch.Tensor]) -> Dict[int, CacheView]:
        out: Dict[int, CacheView] = {}
        for slot, gi in self.group_of_slot.items():
            k, v = self.kv[slot]
            out[slot] = KvCacheView(writes=True, k_pool=k, v_pool=v, block_table=block_tables[gi],
                                    page_tokens=self.page_tokens)
        for slot, tensor in self.state.items():
            out[slot] = StateCacheView(writes=True, state=tensor)
        return out

    def zero_state(self, slot_index: int) -> None:
        for tensor in self.state.values():
            tensor[slot_index].zero_()

    def poison_pages(self, group: int, pages: List[int]) -> None:
        """Fills pages with NaN so that a read of a page that was given back shows up."""
        if not pages:
            return
        index = torch.tensor(pages, dtype=torch.long, device=self.device)
        for slot, gi in self.group_of_slot.items():
            if gi == group:
                for pool in self.kv[slot]:
                    pool.index_fill_(0, index, float("nan"))
