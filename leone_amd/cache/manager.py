"""The cache manager: pages, block tables and state slots (host side, no tensors).

The reference keeps a request's keys and values in growable segments and stages
every append as a transaction: ``prepare_append`` reserves room, kernels write
only there, ``commit_append`` makes it visible, any error rolls back exactly
(crates/leone/src/kv.rs:326-370, 856-927).  Here the same contract is kept over
fixed-size pages:

* a *group* is a set of layers with the same cache need; it has its own pages,
  free list and one block table per request (logical block -> page id, -1 where
  no page is mapped);
* ``reserve`` maps pages for the positions a step is about to write, in every
  group, all or nothing; ``commit`` advances the request's length and, for a
  windowed group, hands back pages that no later query can reach; ``rollback``
  undoes an uncommitted reservation; ``release`` returns everything a request
  holds, pages and state slot, at once;
* a *state slot* is an index into per-request storage of fixed size, handed out
  on admission and returned on release;
* ``fork`` lets a new request share the full pages of another request's prefix
  (the reference's fork shares committed, immutable segments and gives the writer
  a private tail, crates/leone/src/kv.rs:307-324, 676-691): pages carry reference
  counts, a page goes back to the free list when its last holder lets go, and a
  shared page is never written because sharing stops at a page boundary and all
  appends go to pages of the request's own; ``truncate`` cuts a request back
  (crates/leone/src/kv.rs:929-950).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Hashable, List, Optional


def _gcd(a: int, b: int) -> int:
    while b:
        a, b = b, a % b
    return a


class OutOfPages(RuntimeError):
    """A reservation needs more free pages than a group has; nothing was changed."""

    def __init__(self, group: int, needed: int, free: int):
        super().__init__(f"cache group {group} needs {needed} free pages, has {free}")
        self.group, self.needed, self.free = group, needed, free


class OutOfSlots(RuntimeError):
    """Every per-request state slot is taken."""


class CacheError(RuntimeError):
    """The manager was used against its contract (unknown request, double free, ...)."""


@dataclass(frozen=True)
class GroupSpec:
    """Pages of one group: ``window`` None keeps every position, else only the last ``window``."""
    num_pages: int
    page_tokens: int
    window: Optional[int] = None


class _Request:
    __slots__ = ("slot", "length", "tables", "pending_pages", "pending_tokens")

    def __init__(self, slot: int, n_groups: int):
        self.slot = slot
        self.length = 0                                   # committed tokens
        self.tables: List[List[int]] = [[] for _ in range(n_groups)]
        self.pending_pages: List[List[int]] = [[] for _ in range(n_groups)]  # block indices mapped by reserve
        self.pending_tokens = 0


class CacheManager:
    def __init__(self, groups: List[GroupSpec], max_requests: int, max_context: int):
        if max_requests <= 0 or max_context <= 0:
            raise ValueError("max_requests and max_context must be positive")
        for g in groups:
            if g.num_pages <= 0 or g.page_tokens <= 0 or (g.window is not None and g.window <= 0):
                raise ValueError(f"invalid cache group {g}")
        self.groups = list(groups)
        self.max_requests = max_requests
        self.max_context = max_context
        # LIFO free lists: a page given back is the next one handed out.
        self._free: List[List[int]] = [list(range(g.num_pages - 1, -1, -1)) for g in self.groups]
        self._free_slots: List[int] = list(range(max_requests - 1, -1, -1))
        self._refs: List[List[int]] = [[0] * g.num_pages for g in self.groups]   # holders of every page
        self._requests: Dict[Hashable, _Request] = {}
        self.pages_high_water = [0 for _ in self.groups]

    # ---- queries -------------------------------------------------------------
    def max_blocks(self, group: int) -> int:
        pt = self.groups[group].page_tokens
        return (self.max_context + pt - 1) // pt

    def has(self, request: Hashable) -> bool:
        return request in self._requests

    def live_requests(self) -> List[Hashable]:
        return list(self._requests)

    def _get(self, request: Hashable) -> _Request:
        try:
            return self._requests[request]
        except KeyError:
            raise CacheError(f"request {request!r} is not admitted") from None

    def length(self, request: Hashable) -> int:
        return self._get(request).length

    def slot(self, request: Hashable) -> int:
        return self._get(request).slot

    def table(self, request: Hashable, group: int) -> List[int]:
        return self._get(request).tables[group]

    def free_pages(self, group: int) -> int:
        return len(self._free[group])

    def free_slots(self) -> int:
        return len(self._free_slots)

    def pages_needed(self, request: Hashable, tokens: int) -> List[int]:
        """How many new pages each group must map to append ``tokens`` to ``request`` now."""
        state = self._get(request)
        return [len(self._blocks_to_map(state, gi, state.length + state.pending_tokens, tokens))
                for gi in range(len(self.groups))]

    # ---- life cycle -------------------------------------------------------------
    def admit(self, request: Hashable) -> int:
        if request in self._requests:
            raise CacheError(f"request {request!r} is already admitted")
        if not self._free_slots:
            raise OutOfSlots(f"all {self.max_requests} state slots are in use")
        slot = self._free_slots.pop()
        self._requests[request] = _Request(slot, len(self.groups))
        return slot

    def _take(self, gi: int) -> int:
        page = self._free[gi].pop()
        self._refs[gi][page] = 1
        return page

    def _drop(self, gi: int, page: int) -> None:
        """One holder lets go of a page; the last one puts it back on the free list."""
        if self._refs[gi][page] <= 0:
            raise CacheError(f"group {gi}: page {page} is given back more often than it was taken")
        self._refs[gi][page] -= 1
        if self._refs[gi][page] == 0:
            self._free[gi].append(page)

    def holders(self, group: int, page: int) -> int:
        return self._refs[group][page]

    def shared_pages(self, group: int) -> int:
        return sum(1 for r in self._refs[group] if r > 1)

    def fork(self, parent: Hashable, child: Hashable, tokens: Optional[int] = None) -> int:
        """Admits ``child`` holding the full pages of the first ``tokens`` tokens of ``parent`` (all it has
        committed if None).  Returns how many tokens the child holds: ``tokens`` rounded down to a page
        boundary of every group; what lies beyond, the child computes for itself."""
        source = self._get(parent)
        if source.pending_tokens:
            raise CacheError(f"request {parent!r} has an uncommitted reservation")
        limit = source.length if tokens is None else min(int(tokens), source.length)
        if limit < 0:
            raise CacheError("a fork cannot share a negative number of tokens")
        unit = 1
        for g in self.groups:
            unit = unit * g.page_tokens // _gcd(unit, g.page_tokens)
        shared = limit // unit * unit
        plans = []
        for gi, g in enumerate(self.groups):
            blocks = shared // g.page_tokens
            first = 0 if g.window is None else max(0, shared - (g.window - 1)) // g.page_tokens
            table = source.tables[gi]
            for b in range(first, blocks):
                if b >= len(table) or table[b] < 0:
                    raise CacheError(f"group {gi}: the parent's window has passed block {b}; fork later tokens")
            plans.append([table[b] if first <= b else -1 for b in range(blocks)])
        self.admit(child)
        state = self._requests[child]
        for gi, pages in enumerate(plans):
            state.tables[gi] = list(pages)
            for page in pages:
                if page >= 0:
                    self._refs[gi][page] += 1
        state.length = shared
        return shared

    def truncate(self, request: Hashable, position: int) -> None:
        """Cuts a request back to ``position`` tokens.  Pages wholly beyond go back; the page that holds
        ``position`` stays and must be the request's own unless ``position`` is a page boundary."""
        state = self._get(request)
        if state.pending_tokens:
            raise CacheError(f"request {request!r} has an uncommitted reservation")
        if not 0 <= position <= state.length:
            raise CacheError(f"cannot truncate {request!r} of length {state.length} to {position}")
        for gi, g in enumerate(self.groups):
            table = state.tables[gi]
            keep = (position + g.page_tokens - 1) // g.page_tokens
            if position % g.page_tokens and keep <= len(table) and table[keep - 1] >= 0 \
                    and self._refs[gi][table[keep - 1]] > 1:
                raise CacheError(f"group {gi}: the page holding position {position} is shared; "
                                 f"truncate to a multiple of {g.page_tokens}")
        for gi, g in enumerate(self.groups):
            table = state.tables[gi]
            keep = (position + g.page_tokens - 1) // g.page_tokens
            if g.window is not None:
                reach = max(0, position - (g.window - 1)) // g.page_tokens
                for b in range(reach, min(keep, len(table))):
                    if table[b] < 0:
                        raise CacheError(f"group {gi}: keys before position {position} have left the window; "
                                         f"they cannot be brought back by truncation")
            for b in range(keep, len(table)):
                if table[b] >= 0:
                    self._drop(gi, table[b])
            del table[keep:]
        state.length = position

    def _blocks_to_map(self, state: _Request, gi: int, start: int, tokens: int) -> List[int]:
        if tokens <= 0:
            return []
        g = self.groups[gi]
        table = state.tables[gi]
        # Every position of the range is written, also in a windowed group: rows of the same
        # step read them.  Blocks that fall behind the window are handed back at commit.
        first_block = start // g.page_tokens
        last_block = (start + tokens - 1) // g.page_tokens
        return [b for b in range(first_block, last_block + 1) if b >= len(table) or table[b] < 0]

    def reserve(self, request: Hashable, tokens: int) -> None:
        """Maps pages so that positions [length, length + tokens) can be written.  All groups or none."""
        state = self._get(request)
        if tokens <= 0:
            raise CacheError("a reservation must cover at least one token")
        if state.pending_tokens:
            raise CacheError(f"request {request!r} already has an uncommitted reservation")
        start = state.length
        if start + tokens > self.max_context:
            raise CacheError(f"request {request!r}: {start} + {tokens} tokens exceed the context of {self.max_context}")
        plans = []
        for gi in range(len(self.groups)):
            blocks = self._blocks_to_map(state, gi, start, tokens)
            if len(blocks) > len(self._free[gi]):
                raise OutOfPages(gi, len(blocks), len(self._free[gi]))
            plans.append(blocks)
        for gi, blocks in enumerate(plans):
            table = state.tables[gi]
            for b in blocks:
                while len(table) <= b:
                    table.append(-1)
                table[b] = self._take(gi)
            state.pending_pages[gi] = blocks
            used = self.groups[gi].num_pages - len(self._free[gi])
            self.pages_high_water[gi] = max(self.pages_high_water[gi], used)
        state.pending_tokens = tokens

    def commit(self, request: Hashable, tokens: Optional[int] = None) -> None:
        """The reserved positions now hold data.  Window groups give back pages no later query reaches."""
        state = self._get(request)
        if not state.pending_tokens:
            raise CacheError(f"request {request!r} has no reservation to commit")
        if tokens is not None and tokens != state.pending_tokens:
            raise CacheError(f"commit of {tokens} tokens does not match the reservation of {state.pending_tokens}")
        state.length += state.pending_tokens
        state.pending_tokens = 0
        for gi, g in enumerate(self.groups):
            state.pending_pages[gi] = []
            if g.window is None:
                continue
            # The next query sits at position `length` and reads keys >= length - window + 1.
            reach = state.length - (g.window - 1)
            table = state.tables[gi]
            for b in range(min(len(table), max(0, reach) // g.page_tokens)):
                if table[b] >= 0:
                    self._drop(gi, table[b])
                    table[b] = -1

    def rollback(self, request: Hashable) -> None:
        """Undoes an uncommitted reservation exactly."""
        state = self._get(request)
        for gi in range(len(self.groups)):
            table = state.tables[gi]
            for b in reversed(state.pending_pages[gi]):
                self._drop(gi, table[b])
                table[b] = -1
            while table and table[-1] < 0 and len(table) * self.groups[gi].page_tokens > self._covered(state, gi):
                table.pop()
            state.pending_pages[gi] = []
        state.pending_tokens = 0

    def _covered(self, state: _Request, gi: int) -> int:
        pt = self.groups[gi].page_tokens
        return ((state.length + pt - 1) // pt) * pt

    def release(self, request: Hashable) -> None:
        """Returns every page and the state slot of a request (finished, cancelled or preempted)."""
        state = self._requests.pop(request, None)
        if state is None:
            raise CacheError(f"request {request!r} is not admitted (released twice?)")
        for gi in range(len(self.groups)):
            for page in state.tables[gi]:
                if page >= 0:
                    self._drop(gi, page)
        self._free_slots.append(state.slot)

    # ---- invariants ---------------------------------------------------------------
    def check(self) -> None:
        """No page lost, held twice or free twice; slots likewise.  Raises CacheError."""
        for gi, g in enumerate(self.groups):
            free = set()
            for page in self._free[gi]:
                if page in free:
                    raise CacheError(f"group {gi}: page {page} is on the free list twice")
                free.add(page)
            holders = [0] * g.num_pages
            for request, state in self._requests.items():
                mine = set()
                for page in state.tables[gi]:
                    if page < 0:
                        continue
                    if not 0 <= page < g.num_pages:
                        raise CacheError(f"group {gi}: {request!r} holds page {page}, which does not exist")
                    if page in mine:
                        raise CacheError(f"group {gi}: {request!r} holds page {page} twice")
                    if page in free:
                        raise CacheError(f"group {gi}: page {page} held by {request!r} is also free")
                    mine.add(page)
                    holders[page] += 1
            for page in range(g.num_pages):
                if holders[page] != self._refs[gi][page]:
                    raise CacheError(f"group {gi}: page {page} has {holders[page]} holders but a count of "
                                     f"{self._refs[gi][page]}")
                if holders[page] == 0 and page not in free:
                    raise CacheError(f"group {gi}: page {page} is lost (neither held nor free)")
            for request, state in self._requests.items():
                total = state.length + state.pending_tokens
                first = 0 if g.window is None else max(0, state.length - (g.window - 1)) // g.page_tokens
                if total:
                    for b in range(first, (total - 1) // g.page_tokens + 1):
                        if b >= len(state.tables[gi]) or state.tables[gi][b] < 0:
                            raise CacheError(f"group {gi}: {request!r} has no page for block {b}")
        slots = list(self._free_slots) + [s.slot for s in self._requests.values()]
        if sorted(slots) != list(range(self.max_requests)):
            raise CacheError("state slots are lost or held twice")
