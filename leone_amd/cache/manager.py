"""The cache manager: pages, block tables and state slots (host side, no tensors).

The manager itself is C++ (``csrc/host/cache_manager.cpp``); this class binds it.
Requests are named by any hashable value here and by a 64-bit key there.

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

import ctypes
import re
from ctypes import c_int, c_int64
from dataclasses import dataclass
from typing import Dict, Hashable, List, Optional

from .. import hostlib


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


class RequestKeys:
    """Names of requests on this side, 64-bit keys on the native side.  Keys are never used again.

    A name stays known while the cache holds the request or while someone has pinned it (a scheduler
    pins the requests it queues, because a preempted request leaves the cache and comes back)."""

    def __init__(self):
        self._key: Dict[Hashable, int] = {}
        self._name: Dict[int, Hashable] = {}
        self._pinned: set = set()
        self._next = 1

    def key(self, name: Hashable, create: bool = False) -> Optional[int]:
        found = self._key.get(name)
        if found is None and create:
            found = self._next
            self._next += 1
            self._key[name] = found
            self._name[found] = name
        return found

    def name(self, key: int) -> Hashable:
        return self._name[key]

    def named(self, message: str) -> str:
        """A message of the native side with its request keys turned back into names."""
        def swap(match):
            key = int(match.group(1))
            return f"request {self._name[key]!r}" if key in self._name else match.group(0)
        return re.sub(r"request (\d+)", swap, message)

    def pin(self, name: Hashable) -> int:
        key = self.key(name, create=True)
        self._pinned.add(name)
        return key

    def unpin(self, name: Hashable, held: bool) -> None:
        self._pinned.discard(name)
        if not held:
            self.forget(name)

    def forget(self, name: Hashable) -> None:
        if name in self._pinned:
            return
        key = self._key.pop(name, None)
        if key is not None:
            del self._name[key]


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
        self.keys = RequestKeys()
        self._lib = hostlib.library()
        flat = (c_int * (3 * len(groups)))()
        for i, g in enumerate(groups):
            flat[3 * i], flat[3 * i + 1], flat[3 * i + 2] = g.num_pages, g.page_tokens, g.window or 0
        self.handle = self._lib.leone_cache_create(flat, len(groups), max_requests, max_context)
        if not self.handle:
            raise ValueError(hostlib.last_error())
        self._max_blocks = [self._lib.leone_cache_max_blocks(self.handle, g) for g in range(len(groups))]
        self._table_buffers = [(c_int * max(1, width))() for width in self._max_blocks]

    def __del__(self):
        handle, self.handle = getattr(self, "handle", None), None
        if handle:
            self._lib.leone_cache_destroy(handle)

    # ---- errors ---------------------------------------------------------------
    def _raise(self, code: int):
        message = self.keys.named(hostlib.last_error())
        if code == hostlib.OUT_OF_PAGES:
            group, needed, free = c_int(), c_int(), c_int()
            self._lib.leone_cache_shortage(ctypes.byref(group), ctypes.byref(needed), ctypes.byref(free))
            raise OutOfPages(group.value, needed.value, free.value)
        if code == hostlib.OUT_OF_SLOTS:
            raise OutOfSlots(message)
        raise CacheError(message)

    def _checked(self, code: int) -> int:
        if code < 0:
            self._raise(code)
        return code

    def _key(self, request: Hashable) -> int:
        key = self.keys.key(request)
        if key is None:
            raise CacheError(f"request {request!r} is not admitted")
        return key

    # ---- queries -------------------------------------------------------------
    def max_blocks(self, group: int) -> int:
        return self._max_blocks[group]

    def has(self, request: Hashable) -> bool:
        key = self.keys.key(request)
        return key is not None and self._lib.leone_cache_has(self.handle, key) == 1

    def live_requests(self) -> List[Hashable]:
        buffer = (c_int64 * self.max_requests)()
        n = self._checked(self._lib.leone_cache_requests(self.handle, buffer, self.max_requests))
        return [self.keys.name(buffer[i]) for i in range(n)]

    def length(self, request: Hashable) -> int:
        return self._checked(self._lib.leone_cache_length(self.handle, self._key(request)))

    def slot(self, request: Hashable) -> int:
        return self._checked(self._lib.leone_cache_slot(self.handle, self._key(request)))

    def table(self, request: Hashable, group: int) -> List[int]:
        buffer = self._table_buffers[group]
        n = self._checked(self._lib.leone_cache_table(self.handle, self._key(request), group, buffer, len(buffer)))
        return buffer[:n]

    def free_pages(self, group: int) -> int:
        return self._checked(self._lib.leone_cache_free_pages(self.handle, group))

    def free_slots(self) -> int:
        return self._checked(self._lib.leone_cache_free_slots(self.handle))

    def pages_needed(self, request: Hashable, tokens: int) -> List[int]:
        """How many new pages each group must map to append ``tokens`` to ``request`` now."""
        out = (c_int * len(self.groups))()
        self._checked(self._lib.leone_cache_pages_needed(self.handle, self._key(request), tokens, out))
        return list(out)

    def holders(self, group: int, page: int) -> int:
        return self._checked(self._lib.leone_cache_holders(self.handle, group, page))

    def shared_pages(self, group: int) -> int:
        return self._checked(self._lib.leone_cache_shared_pages(self.handle, group))

    def log_freed(self, on: bool = True) -> None:
        """Has the manager note every page whose last holder lets go, whoever frees it (``drain_freed``)."""
        self._checked(self._lib.leone_cache_log_freed(self.handle, 1 if on else 0))

    def drain_freed(self, group: int) -> List[int]:
        """Pages of ``group`` that became free since the last call (the log must be on); some may have been
        handed out again already, to a holder that has not written them yet."""
        buffer = (c_int * self.groups[group].num_pages)()
        n = self._checked(self._lib.leone_cache_drain_freed(self.handle, group, buffer, self.groups[group].num_pages))
        return list(buffer[:n])

    @property
    def pages_high_water(self) -> List[int]:
        return [self._lib.leone_cache_high_water(self.handle, g) for g in range(len(self.groups))]

    # ---- life cycle -------------------------------------------------------------
    def admit(self, request: Hashable) -> int:
        known = self.keys.key(request) is not None
        key = self.keys.key(request, create=True)
        code = self._lib.leone_cache_admit(self.handle, key)
        if code < 0:
            if not known:
                self.keys.forget(request)
            self._raise(code)
        return code

    def fork(self, parent: Hashable, child: Hashable, tokens: Optional[int] = None) -> int:
        """Admits ``child`` holding the full pages of the first ``tokens`` tokens of ``parent`` (all it has
        committed if None).  Returns how many tokens the child holds: ``tokens`` rounded down to a page
        boundary of every group; what lies beyond, the child computes for itself."""
        if tokens is not None and tokens < 0:
            raise CacheError("a fork cannot share a negative number of tokens")
        source = self._key(parent)
        known = self.keys.key(child) is not None
        key = self.keys.key(child, create=True)
        code = self._lib.leone_cache_fork(self.handle, source, key, -1 if tokens is None else int(tokens))
        if code < 0:
            if not known:
                self.keys.forget(child)
            self._raise(code)
        return code

    def truncate(self, request: Hashable, position: int) -> None:
        """Cuts a request back to ``position`` tokens.  Pages wholly beyond go back; the page that holds
        ``position`` stays and must be the request's own unless ``position`` is a page boundary."""
        self._checked(self._lib.leone_cache_truncate(self.handle, self._key(request), position))

    def reserve(self, request: Hashable, tokens: int) -> None:
        """Maps pages so that positions [length, length + tokens) can be written.  All groups or none."""
        self._checked(self._lib.leone_cache_reserve(self.handle, self._key(request), tokens))

    def commit(self, request: Hashable, tokens: Optional[int] = None) -> None:
        """The reserved positions now hold data.  Window groups give back pages no later query reaches."""
        self._checked(self._lib.leone_cache_commit(self.handle, self._key(request), -1 if tokens is None else tokens))

    def rollback(self, request: Hashable) -> None:
        """Undoes an uncommitted reservation exactly."""
        self._checked(self._lib.leone_cache_rollback(self.handle, self._key(request)))

    def release(self, request: Hashable) -> None:
        """Returns every page and the state slot of a request (finished, cancelled or preempted)."""
        key = self.keys.key(request)
        if key is None:
            raise CacheError(f"request {request!r} is not admitted (released twice?)")
        self._checked(self._lib.leone_cache_release(self.handle, key))
        self.keys.forget(request)

    # ---- invariants ---------------------------------------------------------------
    def check(self) -> None:
        """No page lost, held twice or free twice; slots likewise.  Raises CacheError.

        Works from what the native manager reports (tables, free lists, counts), not from its internals."""
        requests = self.live_requests()
        for gi, g in enumerate(self.groups):
            buffer = (c_int * g.num_pages)()
            n = self._checked(self._lib.leone_cache_free_list(self.handle, gi, buffer, g.num_pages))
            if n > g.num_pages:
                raise CacheError(f"group {gi}: the free list holds {n} of {g.num_pages} pages")
            free = set()
            for page in buffer[:n]:
                if page in free:
                    raise CacheError(f"group {gi}: page {page} is on the free list twice")
                free.add(page)
            holders = [0] * g.num_pages
            for request in requests:
                mine = set()
                table = self.table(request, gi)
                for page in table:
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
                length = self.length(request)
                total = length + self._checked(self._lib.leone_cache_pending(self.handle, self._key(request)))
                first = 0 if g.window is None else max(0, length - (g.window - 1)) // g.page_tokens
                if total:
                    for b in range(first, (total - 1) // g.page_tokens + 1):
                        if b >= len(table) or table[b] < 0:
                            raise CacheError(f"group {gi}: {request!r} has no page for block {b}")
            for page in range(g.num_pages):
                if holders[page] != self.holders(gi, page):
                    raise CacheError(f"group {gi}: page {page} has {holders[page]} holders but a count of "
                                     f"{self.holders(gi, page)}")
                if holders[page] == 0 and page not in free:
                    raise CacheError(f"group {gi}: page {page} is lost (neither held nor free)")
        buffer = (c_int * self.max_requests)()
        n = self._checked(self._lib.leone_cache_free_slot_list(self.handle, buffer, self.max_requests))
        slots = list(buffer[:min(n, self.max_requests)]) + [self.slot(r) for r in requests]
        if n > self.max_requests or sorted(slots) != list(range(self.max_requests)):
            raise CacheError("state slots are lost or held twice")
