"""The scheduler: admission, prompt portions under a token budget, continuous decoding, finishing.

It decides; it runs nothing.  Each ``plan()`` yields the entries of one step
with their pages already reserved; the caller runs them (which commits the
cache) and reports the sampled tokens to ``complete()``.  It needs only the
host-side cache manager, so its decisions can be tested without a GPU.

What is kept from the reference's scheduler (crates/leone/src/scheduler.rs):
typed admission rejects with nothing reserved on rejection (:99-110, :587-636);
one budget per request and step, a prompt portion of at most
``prefill_chunk_tokens`` or one decoded token (:341-378); a request is finished
on its end token or when its output budget is used up, and its reservation is
released at once (:445-448, :1341-1343); cancellation of a queued request is
immediate, of a running one at the next step boundary (:540-554); an executor
error aborts the whole batch (:520-538, crates/leone/src/service.rs:270-297);
counters (:171-192).

What differs: the reference reserves a request's whole lifetime of cache at
admission, so it never runs out in flight (:652-667).  Here pages are taken as
tokens arrive.  When a decode row cannot get a page, the most recently admitted
live request is preempted: everything it holds is released and it goes back to
the head of the queue with its generated tokens appended to its prompt, to be
recomputed (the reference's replay of a token checkpoint as prefill,
crates/leone/src/runtime.rs:699-716).  Sampling draws are keyed by absolute
position, so the continuation is unchanged.  A prompt portion that does not fit
is shortened to the free pages or waits; it never preempts.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from enum import Enum
from typing import Deque, Dict, Hashable, List, Optional, Sequence

from ..cache.manager import CacheManager, OutOfPages


class Reject(Enum):
    PROMPT_LIMIT = "prompt-limit"        # empty, or longer than the policy allows
    OUTPUT_LIMIT = "output-limit"        # zero, or more than the policy allows
    CONTEXT_LIMIT = "context-limit"      # prompt + output - 1 exceeds the model's context
    KV_CAPACITY = "kv-capacity"          # could never fit the page pool, even alone
    QUEUE_LIMIT = "queue-limit"
    DUPLICATE = "duplicate"


class SchedulerError(RuntimeError):
    pass


@dataclass(frozen=True)
class SchedulerPolicy:
    max_live_requests: int = 64
    max_queued_requests: int = 1024
    max_step_tokens: int = 2048          # token budget of one step (decode rows + prompt portions)
    prefill_chunk_tokens: int = 512      # longest prompt portion of one request in one step
    max_prompt_tokens: int = 1 << 30
    max_output_tokens: int = 1 << 30

    def validate(self) -> "SchedulerPolicy":
        for name in ("max_live_requests", "max_queued_requests", "max_step_tokens", "prefill_chunk_tokens",
                     "max_prompt_tokens", "max_output_tokens"):
            if getattr(self, name) <= 0:
                raise SchedulerError(f"policy: {name} must be positive")
        return self


@dataclass
class Request:
    id: Hashable
    prompt: Sequence[int]
    max_new_tokens: int
    sampling: object = None              # opaque to the scheduler
    eos_token_id: Optional[int] = None


@dataclass
class PlannedEntry:
    request: Hashable
    tokens: List[int]
    start: int                           # absolute position of tokens[0]
    sample: bool                         # the portion ends the known tokens: its last row's logits are wanted

    @property
    def sample_position(self) -> int:
        """Absolute index of the token whose logits are sampled."""
        return self.start + len(self.tokens) - 1


@dataclass
class Finished:
    id: Hashable
    prompt: List[int]
    tokens: List[int]
    reason: str                          # "eos", "length", "cancelled", "aborted"
    preemptions: int = 0


@dataclass
class SchedulerStats:
    submitted: int = 0
    admitted: int = 0
    rejected: int = 0
    steps: int = 0
    prefill_portions: int = 0
    prefill_tokens: int = 0
    decode_rows: int = 0
    emitted_tokens: int = 0
    finished: int = 0
    cancelled: int = 0
    aborted: int = 0
    preemptions: int = 0
    max_queue_depth: int = 0
    max_step_rows: int = 0
    max_live: int = 0


class _Live:
    __slots__ = ("request", "tokens", "prompt_len", "order", "cancelled", "preemptions")

    def __init__(self, request: Request, order: int):
        self.request = request
        self.tokens: List[int] = list(request.prompt)   # prompt, then generated tokens
        self.prompt_len = len(self.tokens)
        self.order = order
        self.cancelled = False
        self.preemptions = 0

    @property
    def generated(self) -> List[int]:
        return self.tokens[self.prompt_len:]


class Scheduler:
    def __init__(self, policy: SchedulerPolicy, cache: CacheManager):
        self.policy = policy.validate()
        self.cache = cache
        self.queue: Deque[_Live] = deque()
        self.live: Dict[Hashable, _Live] = {}
        self.finished: List[Finished] = []
        self.stats = SchedulerStats()
        self.events: List[tuple] = []
        self._order = 0
        self._planned: Optional[List[PlannedEntry]] = None

    # ---- admission ---------------------------------------------------------------------
    def submit(self, request: Request) -> Optional[Reject]:
        """Queues a request, or says why not.  A rejected request holds nothing."""
        self.stats.submitted += 1
        reason = self._reject_reason(request)
        if reason is not None:
            self.stats.rejected += 1
            self.events.append(("reject", request.id, reason.value))
            return reason
        self._order += 1
        self.queue.append(_Live(request, self._order))
        self.stats.max_queue_depth = max(self.stats.max_queue_depth, len(self.queue))
        self.events.append(("submit", request.id))
        return None

    def _reject_reason(self, request: Request) -> Optional[Reject]:
        prompt, out = len(request.prompt), request.max_new_tokens
        if request.id in self.live or any(q.request.id == request.id for q in self.queue):
            return Reject.DUPLICATE
        if prompt == 0 or prompt > self.policy.max_prompt_tokens:
            return Reject.PROMPT_LIMIT
        if out <= 0 or out > self.policy.max_output_tokens:
            return Reject.OUTPUT_LIMIT
        # The last generated token is never fed back, so the cache holds prompt + out - 1 tokens
        # (crates/leone/src/runtime.rs:3597-3615).
        held = prompt + out - 1
        if held > self.cache.max_context:
            return Reject.CONTEXT_LIMIT
        for g in self.cache.groups:
            if g.window is None:
                need = (held + g.page_tokens - 1) // g.page_tokens
            else:
                span = min(held, g.window - 1 + min(self.policy.prefill_chunk_tokens, self.policy.max_step_tokens))
                need = (span + g.page_tokens - 1) // g.page_tokens + 1
            if need > g.num_pages:
                return Reject.KV_CAPACITY
        if len(self.queue) >= self.policy.max_queued_requests:
            return Reject.QUEUE_LIMIT
        return None

    def cancel(self, request_id: Hashable) -> bool:
        """A queued request goes at once; a live one at the next step boundary."""
        for queued in list(self.queue):
            if queued.request.id == request_id:
                self.queue.remove(queued)
                self._finish(queued, "cancelled", held=False)
                return True
        if request_id in self.live:
            self.live[request_id].cancelled = True
            return True
        return False

    # ---- planning ------------------------------------------------------------------------
    def has_work(self) -> bool:
        return bool(self.queue or self.live)

    def plan(self) -> List[PlannedEntry]:
        """Decides the next step and reserves its pages.  Empty only if there is nothing to do."""
        if self._planned is not None:
            raise SchedulerError("the previous step was neither completed nor aborted")
        for state in [s for s in self.live.values() if s.cancelled]:
            self._finish(state, "cancelled", held=True)
        entries: List[PlannedEntry] = []
        for _ in range(len(self.live) + len(self.queue) + 1):
            entries = self._plan_once()
            if entries or not self.live:
                break
            # Every live request waits for pages that only another live request could free.
            self._preempt(self._newest(), planned=[])
        if not entries and (self.live or self.queue):
            raise SchedulerError("no request can make progress")
        self._planned = entries
        if entries:
            self.stats.steps += 1
            rows = sum(len(e.tokens) for e in entries)
            self.stats.max_step_rows = max(self.stats.max_step_rows, rows)
            self.events.append(("step", [(e.request, e.start, len(e.tokens), e.sample) for e in entries]))
        return entries

    def _newest(self) -> _Live:
        return max(self.live.values(), key=lambda s: s.order)

    def _plan_once(self) -> List[PlannedEntry]:
        entries: List[PlannedEntry] = []
        budget = self.policy.max_step_tokens
        by_age = sorted(self.live.values(), key=lambda s: s.order)
        # 1. one token for every request that is decoding, oldest first
        for state in by_age:
            if budget == 0:
                break
            if state.request.id not in self.live:
                continue  # preempted a moment ago
            cached = self.cache.length(state.request.id)
            if len(state.tokens) - cached != 1:
                continue
            while True:
                try:
                    self.cache.reserve(state.request.id, 1)
                except OutOfPages:
                    victim = self._newest()
                    self._preempt(victim, entries)
                    if victim is state:
                        break
                    continue
                entries.append(PlannedEntry(state.request.id, [state.tokens[cached]], cached, True))
                budget -= 1
                self.stats.decode_rows += 1
                break
        # 2. prompt portions for the live requests that still have some, oldest first
        starved = False
        for state in by_age:
            if budget == 0 or starved:
                break
            if state.request.id not in self.live:
                continue
            cached = self.cache.length(state.request.id)
            remaining = len(state.tokens) - cached
            if remaining <= 1:
                continue
            taken = self._reserve_portion(state, cached, min(remaining, self.policy.prefill_chunk_tokens, budget))
            if taken == 0:
                starved = True   # younger requests must not take the pages an older one waits for
                break
            entries.append(PlannedEntry(state.request.id, state.tokens[cached:cached + taken], cached,
                                        taken == remaining))
            budget -= taken
            self.stats.prefill_portions += 1
            self.stats.prefill_tokens += taken
        # 3. admit from the queue
        while (self.queue and not starved and budget > 0 and len(self.live) < self.policy.max_live_requests
               and self.cache.free_slots() > 0):
            state = self.queue[0]
            remaining = len(state.tokens)
            # Admit only when the pages for everything the request already holds are free now,
            # so that a request just preempted is not taken back in only to be preempted again.
            if self.live and not self._room_for(remaining):
                break
            self.cache.admit(state.request.id)
            taken = self._reserve_portion(state, 0, min(remaining, self.policy.prefill_chunk_tokens, budget))
            if taken == 0:
                self.cache.release(state.request.id)
                break
            self.queue.popleft()
            self.live[state.request.id] = state
            self.stats.admitted += 1
            self.stats.max_live = max(self.stats.max_live, len(self.live))
            self.events.append(("admit", state.request.id))
            entries.append(PlannedEntry(state.request.id, state.tokens[:taken], 0, taken == remaining))
            budget -= taken
            if remaining > 1 or taken > 1:
                self.stats.prefill_portions += 1
                self.stats.prefill_tokens += taken
            else:
                self.stats.decode_rows += 1
        return entries

    def _reserve_portion(self, state: _Live, cached: int, wanted: int) -> int:
        """Reserves the longest portion of at most ``wanted`` tokens that the free pages allow."""
        rid = state.request.id
        n = wanted
        while n > 0:
            try:
                self.cache.reserve(rid, n)
                return n
            except OutOfPages:
                lo, hi = 0, n - 1       # largest count whose pages are free
                while lo < hi:
                    mid = (lo + hi + 1) // 2
                    if self._fits(rid, mid):
                        lo = mid
                    else:
                        hi = mid - 1
                n = lo
        return 0

    def _room_for(self, tokens: int) -> bool:
        for gi, g in enumerate(self.cache.groups):
            span = tokens if g.window is None else min(tokens, g.window - 1 + self.policy.prefill_chunk_tokens)
            if (span + g.page_tokens - 1) // g.page_tokens > self.cache.free_pages(gi):
                return False
        return True

    def _fits(self, rid: Hashable, tokens: int) -> bool:
        if tokens == 0:
            return True
        needed = self.cache.pages_needed(rid, tokens)
        return all(needed[g] <= self.cache.free_pages(g) for g in range(len(needed)))

    def _preempt(self, victim: _Live, planned: List[PlannedEntry]) -> None:
        rid = victim.request.id
        for entry in [e for e in planned if e.request == rid]:
            planned.remove(entry)
        self.cache.rollback(rid)
        self.cache.release(rid)
        del self.live[rid]
        victim.preemptions += 1
        self.queue.appendleft(victim)
        self.stats.preemptions += 1
        self.events.append(("preempt", rid, len(victim.tokens)))

    # ---- after the step ----------------------------------------------------------------------
    def complete(self, sampled: Dict[Hashable, int]) -> List[Finished]:
        """The planned step ran and its cache writes are committed.  ``sampled`` holds a token for
        every entry planned with ``sample``.  Returns the requests that finished."""
        if self._planned is None:
            raise SchedulerError("no step is planned")
        planned, self._planned = self._planned, None
        done: List[Finished] = []
        for entry in planned:
            state = self.live[entry.request]
            if self.cache.length(entry.request) != entry.start + len(entry.tokens):
                raise SchedulerError(f"request {entry.request!r}: the step was not committed to the cache")
            if not entry.sample:
                continue
            if entry.request not in sampled:
                raise SchedulerError(f"request {entry.request!r}: the step returned no token")
            token = int(sampled[entry.request])
            state.tokens.append(token)
            self.stats.emitted_tokens += 1
            self.events.append(("token", entry.request, entry.sample_position, token))
            eos = state.request.eos_token_id
            if eos is not None and token == eos:
                done.append(self._finish(state, "eos", held=True))
            elif len(state.generated) >= state.request.max_new_tokens:
                done.append(self._finish(state, "length", held=True))
        return done

    def abort(self) -> List[Finished]:
        """The planned step failed: every request in it ends as aborted and gives back what it holds."""
        if self._planned is None:
            raise SchedulerError("no step is planned")
        planned, self._planned = self._planned, None
        out = []
        for entry in planned:
            state = self.live[entry.request]
            self.cache.rollback(entry.request)
            out.append(self._finish(state, "aborted", held=True))
        return out

    def _finish(self, state: _Live, reason: str, held: bool) -> Finished:
        rid = state.request.id
        if held:
            self.cache.release(rid)
            del self.live[rid]
        result = Finished(rid, list(state.request.prompt), state.generated, reason, state.preemptions)
        self.finished.append(result)
        if reason == "cancelled":
            self.stats.cancelled += 1
        elif reason == "aborted":
            self.stats.aborted += 1
        else:
            self.stats.finished += 1
        self.events.append(("finish", rid, reason))
        return result
