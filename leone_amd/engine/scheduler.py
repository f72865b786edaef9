"""The scheduler: admission, prompt portions under a token budget, continuous decoding, finishing.

It decides; it runs nothing.  Each ``plan()`` yields the entries of one step
with their pages already reserved; the caller runs them (which commits the
cache) and reports the sampled tokens to ``complete()``.  It needs only the
host-side cache manager, so its decisions can be tested without a GPU.  The
scheduler itself is C++ (``csrc/host/scheduler.cpp``); this class binds it and
keeps what only this side knows: the requests' names and sampling settings.

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

import ctypes
from ctypes import c_int, c_int32, c_int64
from dataclasses import dataclass
from enum import Enum
from typing import Dict, Hashable, List, Optional, Sequence

from .. import hostlib
from ..cache.manager import CacheManager


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
    """``max_step_tokens`` is the number of rows a full step has: decoded tokens first, prompt portions cut to
    what is left of it.  The vendor library's products, which a step of more than 128 rows uses, are built for
    round row counts (at the 8B layer sizes a step of 2,049 rows takes 25 % longer than one of 2,048, one of
    544 rows 17 % longer than one of 512): keep it a multiple of 256."""
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
    deferred: bool = False               # planned ahead: the token is the one the step before is still choosing

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


_REJECTS = [None, Reject.PROMPT_LIMIT, Reject.OUTPUT_LIMIT, Reject.CONTEXT_LIMIT, Reject.KV_CAPACITY,
            Reject.QUEUE_LIMIT, Reject.DUPLICATE]
_REASONS = ["eos", "length", "cancelled", "aborted"]


class _Known:
    """A queued or live request as this side sees it; its tokens are read from the native scheduler."""
    __slots__ = ("request", "_scheduler", "_key")

    def __init__(self, request: Request, scheduler: "Scheduler", key: int):
        self.request, self._scheduler, self._key = request, scheduler, key

    @property
    def tokens(self) -> List[int]:
        """Prompt, then generated tokens."""
        return self._scheduler._history(self._key)

    @property
    def prompt_len(self) -> int:
        return self._scheduler._info(self._key)[0]

    @property
    def preemptions(self) -> int:
        return self._scheduler._info(self._key)[1]

    @property
    def generated(self) -> List[int]:
        return self.tokens[self.prompt_len:]


class Scheduler:
    def __init__(self, policy: SchedulerPolicy, cache: CacheManager):
        self.policy = policy.validate()
        self.cache = cache
        self.finished: List[Finished] = []
        self._lib = hostlib.library()
        values = (c_int64 * 6)(policy.max_live_requests, policy.max_queued_requests, policy.max_step_tokens,
                               policy.prefill_chunk_tokens, policy.max_prompt_tokens, policy.max_output_tokens)
        self.handle = self._lib.leone_scheduler_create(cache.handle, values)
        if not self.handle:
            raise SchedulerError(hostlib.last_error())
        self._known: Dict[Hashable, _Known] = {}        # queued and live requests
        self._names: Dict[int, Hashable] = {}           # every key ever used, for the event log
        self._capacity = 0
        self._grow(64)

    def __del__(self):
        handle, self.handle = getattr(self, "handle", None), None
        if handle:
            self._lib.leone_scheduler_destroy(handle)

    def _grow(self, n: int) -> None:
        if n > self._capacity:
            self._capacity = max(n, 2 * self._capacity)
            self._keys = (c_int64 * self._capacity)()
            self._starts = (c_int * self._capacity)()
            self._counts = (c_int * self._capacity)()
            self._samples = (c_int * self._capacity)()
            self._sampled = (c_int32 * self._capacity)()

    def _checked(self, code: int) -> int:
        if code < 0:
            raise SchedulerError(self.cache.keys.named(hostlib.last_error()))
        return code

    def _history(self, key: int) -> List[int]:
        n = self._checked(self._lib.leone_scheduler_history(self.handle, key, None, 0))
        out = (c_int32 * max(1, n))()
        self._checked(self._lib.leone_scheduler_history(self.handle, key, out, n))
        return out[:n]

    def _info(self, key: int):
        prompt, preemptions = c_int(), c_int()
        self._checked(self._lib.leone_scheduler_request_info(self.handle, key, ctypes.byref(prompt),
                                                             ctypes.byref(preemptions)))
        return prompt.value, preemptions.value

    # ---- admission ---------------------------------------------------------------------
    def submit(self, request: Request) -> Optional[Reject]:
        """Queues a request, or says why not.  A rejected request holds nothing."""
        known = request.id in self._known
        key = self.cache.keys.pin(request.id)
        self._names[key] = request.id
        prompt = (c_int32 * max(1, len(request.prompt)))(*[int(t) for t in request.prompt])
        eos = -1 if request.eos_token_id is None else int(request.eos_token_id)
        code = self._checked(self._lib.leone_scheduler_submit(self.handle, key, prompt, len(request.prompt),
                                                              int(request.max_new_tokens), eos))
        if code != 0:
            if not known:
                self.cache.keys.unpin(request.id, held=self.cache.has(request.id))
            return _REJECTS[code]
        self._known[request.id] = _Known(request, self, key)
        return None

    def cancel(self, request_id: Hashable) -> bool:
        """A queued request goes at once; a live one at the next step boundary."""
        state = self._known.get(request_id)
        if state is None:
            return False
        found = self._checked(self._lib.leone_scheduler_cancel(self.handle, state._key)) == 1
        self._collect_finished()
        return found

    # ---- views ---------------------------------------------------------------------------
    def _listed(self, call) -> List[_Known]:
        n = self._checked(call(self.handle, None, 0))
        self._grow(n)
        self._checked(call(self.handle, self._keys, self._capacity))
        return [self._known[self._names[self._keys[i]]] for i in range(n)]

    @property
    def live(self) -> Dict[Hashable, _Known]:
        """Admitted requests, oldest first."""
        return {state.request.id: state for state in self._listed(self._lib.leone_scheduler_live)}

    @property
    def queue(self) -> List[_Known]:
        """Waiting requests, the next to be admitted first."""
        return self._listed(self._lib.leone_scheduler_queued)

    def history(self, request_id: Hashable) -> List[int]:
        """Prompt, then generated tokens, of a queued or live request."""
        return self._known[request_id].tokens

    @property
    def stats(self) -> SchedulerStats:
        values = (c_int64 * 15)()
        self._lib.leone_scheduler_stats(self.handle, values)
        return SchedulerStats(*values)

    @property
    def events(self) -> List[tuple]:
        """The decision log: ("reject", id, reason), ("submit", id, prompt tokens, most new tokens),
        ("step", [(id, start, tokens, sample)]), ("ahead", [...]) for a step planned before the tokens of the one
        before it were known,
        ("admit", id), ("preempt", id, tokens known), ("token", id, position, token), ("finish", id, reason)."""
        n = self._checked(self._lib.leone_scheduler_event_count(self.handle))
        kinds, a, b, c = (c_int * max(1, n))(), (c_int * max(1, n))(), (c_int * max(1, n))(), (c_int * max(1, n))()
        keys = (c_int64 * max(1, n))()
        self._checked(self._lib.leone_scheduler_events(self.handle, 0, n, kinds, keys, a, b, c))
        out: List[tuple] = []
        i = 0
        while i < n:
            kind = kinds[i]
            name = self._names.get(keys[i])
            if kind == 0:
                out.append(("reject", name, _REJECTS[a[i]].value))
            elif kind == 1:
                out.append(("submit", name, a[i], b[i]))
            elif kind == 2:
                rows = [(self._names[keys[j]], a[j], b[j], bool(c[j])) for j in range(i + 1, i + 1 + a[i])]
                out.append(("step", rows))
                i += a[i]
            elif kind == 4:
                out.append(("admit", name))
            elif kind == 5:
                out.append(("preempt", name, a[i]))
            elif kind == 6:
                out.append(("token", name, a[i], b[i]))
            elif kind == 7:
                out.append(("finish", name, _REASONS[a[i]]))
            elif kind == 8:
                rows = [(self._names[keys[j]], a[j], b[j], bool(c[j])) for j in range(i + 1, i + 1 + a[i])]
                out.append(("ahead", rows))
                i += a[i]
            i += 1
        return out

    # ---- planning ------------------------------------------------------------------------
    def has_work(self) -> bool:
        return self._lib.leone_scheduler_has_work(self.handle) == 1

    def plan(self) -> List[PlannedEntry]:
        """Decides the next step and reserves its pages.  Empty only if there is nothing to do."""
        n = self._lib.leone_scheduler_plan(self.handle)
        self._collect_finished()            # requests cancelled since the last step end here
        self._checked(n)
        self._grow(n)
        self._checked(self._lib.leone_scheduler_planned(self.handle, self._keys, self._starts, self._counts,
                                                        self._samples, self._capacity))
        entries = []
        for i in range(n):
            key, start, count = self._keys[i], self._starts[i], self._counts[i]
            tokens = (c_int32 * count)()
            self._checked(self._lib.leone_scheduler_tokens(self.handle, key, start, count, tokens))
            entries.append(PlannedEntry(self._names[key], list(tokens), start, bool(self._samples[i])))
        return entries

    def plan_ahead(self) -> List[PlannedEntry]:
        """One step beyond the planned one, before that one's tokens are known: every request of the planned step
        once more, one row at its next position, in the same order, pages reserved; the rows' tokens (``tokens``
        holds a stand-in, ``deferred`` says so) are the ones the planned step is choosing, which the caller feeds
        from the device.  Empty, with nothing reserved, wherever the next step cannot be known without those
        tokens (a request uses up its budget, somebody waits for a free place, a page is missing, a portion of a
        prompt is not the last): then the planned step is completed first, as always.  The planned step must
        have run.  Once the planned step is completed the step ahead is the planned one; a request that ended
        on its end token meanwhile is no longer in it, and a token reported for it is ignored."""
        n = self._checked(self._lib.leone_scheduler_plan_ahead(self.handle))
        if n == 0:
            return []
        self._grow(n)
        self._checked(self._lib.leone_scheduler_ahead(self.handle, self._keys, self._starts, self._counts,
                                                      self._samples, self._capacity))
        return [PlannedEntry(self._names[self._keys[i]], [0], self._starts[i], True, deferred=True) for i in range(n)]

    # ---- after the step ----------------------------------------------------------------------
    def complete(self, sampled: Dict[Hashable, int]) -> List[Finished]:
        """The planned step ran and its cache writes are committed.  ``sampled`` holds a token for
        every entry planned with ``sample``.  Returns the requests that finished."""
        self._grow(len(sampled))
        n = 0
        for name, token in sampled.items():
            state = self._known.get(name)
            if state is None:
                continue
            self._keys[n], self._sampled[n] = state._key, int(token)
            n += 1
        self._checked(self._lib.leone_scheduler_complete(self.handle, self._keys, self._sampled, n))
        return self._collect_finished()

    def abort(self) -> List[Finished]:
        """The planned step failed: every request in it ends as aborted and gives back what it holds."""
        self._checked(self._lib.leone_scheduler_abort(self.handle))
        return self._collect_finished()

    def _collect_finished(self) -> List[Finished]:
        total = self._checked(self._lib.leone_scheduler_finished_count(self.handle))
        new: List[Finished] = []
        for index in range(len(self.finished), total):
            key, reason, preemptions, n_prompt, n_out = c_int64(), c_int(), c_int(), c_int(), c_int()
            self._checked(self._lib.leone_scheduler_finished_info(
                self.handle, index, ctypes.byref(key), ctypes.byref(reason), ctypes.byref(preemptions),
                ctypes.byref(n_prompt), ctypes.byref(n_out)))
            prompt, out = (c_int32 * max(1, n_prompt.value))(), (c_int32 * max(1, n_out.value))()
            self._checked(self._lib.leone_scheduler_finished_tokens(self.handle, index, prompt, out))
            name = self._names[key.value]
            record = Finished(name, prompt[:n_prompt.value], out[:n_out.value], _REASONS[reason.value],
                              preemptions.value)
            self.finished.append(record)
            new.append(record)
            self._known.pop(name, None)
            self.cache.keys.unpin(name, held=False)
        return new
