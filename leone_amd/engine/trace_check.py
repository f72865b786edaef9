"""A checker of the scheduler's decision log that knows nothing of the scheduler.

It takes ``Scheduler.events`` (plain tuples) and the figures of the run (pages, page size, budgets) and
re-derives from the events alone what must hold: every request goes submit, admit, (preempt, admit)*,
finish; one step is in flight at a time and each of its sampling rows is answered by exactly one
token before the next step, except that one step may be planned ahead of a step whose rows all owe their
tokens: the same requests once more, one row each at the next position, none of them at the end of its
output, and nothing else may be decided until the owed tokens have come (a request that ends on its end
token then drops out of the step ahead); a request's portions follow each other without a gap or an overlap from
position 0 after every (re)admission; steps keep the token budget, the portion limit and the limit of
live requests; the pages that the live requests' positions need never exceed the pool; nothing
happens to a request that has finished; output limits hold.  It returns what each request was fed and
what it was given, so that a caller can compare the transcript with the request run alone.

The reference keeps such a verifier beside its scheduler (crates/leone/src/scheduler.rs:1349-1655: a
replay of service events against a capacity, one dispatch in flight, emitted counts).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, Iterable, List, Optional, Sequence, Tuple


class TraceError(ValueError):
    """The log breaks a rule; the message names the event's index."""


@dataclass(frozen=True)
class PoolFigures:
    """One cache group: its pages, their size, and the window of its layers (0: all keys)."""
    num_pages: int
    page_tokens: int
    window: int = 0

    def first_page(self, held: int) -> int:
        """The first page a request still holds once ``held`` positions are committed: the next row sits
        at position ``held`` and reads keys from ``held - window + 1`` on; pages wholly before that have
        been given back (crates/leone/src/kv.rs keeps whole segments in the same way)."""
        return 0 if self.window == 0 else max(0, held - (self.window - 1)) // self.page_tokens

    def pages_for(self, before: int, after: int) -> int:
        """Pages a request holds while a step takes it from ``before`` to ``after`` positions: what it
        kept after its last step, and every page up to the new end."""
        if after <= 0:
            return 0
        return (after - 1) // self.page_tokens - self.first_page(before) + 1


@dataclass
class RunFigures:
    pools: Sequence[PoolFigures]
    max_live_requests: int
    max_step_tokens: int
    prefill_chunk_tokens: int


@dataclass
class RequestTrace:
    prompt_tokens: int
    max_new_tokens: int
    state: str = "queued"                    # queued, live, finished
    held: int = 0                            # positions in the cache since the last (re)admission
    held_before: int = 0                     # the same before the step in flight
    emitted: Dict[int, int] = field(default_factory=dict)    # position of the row -> token it gave
    preemptions: int = 0
    reason: Optional[str] = None
    fed: int = 0                             # rows run for it, recomputation included

    @property
    def tokens(self) -> List[int]:
        """Generated tokens in order of position."""
        return [self.emitted[p] for p in sorted(self.emitted)]


@dataclass
class TraceReport:
    requests: Dict[Hashable, RequestTrace]
    rejected: List[Tuple[Hashable, str]]
    steps: int
    peak_pages: List[int]
    peak_live: int
    peak_step_tokens: int


def verify_events(events: Iterable[tuple], figures: RunFigures) -> TraceReport:
    requests: Dict[Hashable, RequestTrace] = {}
    rejected: List[Tuple[Hashable, str]] = []
    awaiting: Dict[Hashable, int] = {}       # rows of the step in flight that still owe a token: id -> position
    in_flight: List[Hashable] = []           # requests of the step in flight
    ahead: Optional[Dict[Hashable, int]] = None   # rows of a step planned ahead of it: id -> position
    steps = 0
    peak_pages = [0 for _ in figures.pools]
    peak_live = peak_tokens = 0

    def fail(index: int, text: str):
        raise TraceError(f"event {index}: {text}")

    def known(index: int, name, *states: str) -> RequestTrace:
        trace = requests.get(name)
        if trace is None:
            fail(index, f"request {name!r} was never submitted")
        if states and trace.state not in states:
            fail(index, f"request {name!r} is {trace.state}, expected {' or '.join(states)}")
        return trace

    def pages_now() -> List[int]:
        live = [t for t in requests.values() if t.state == "live"]
        return [sum(pool.pages_for(t.held_before, t.held) for t in live) for pool in figures.pools]

    events_list = list(events)
    for index, event in enumerate(events_list):
        kind = event[0]
        if kind == "reject":
            rejected.append((event[1], event[2]))
        elif kind == "submit":
            _, name, prompt_tokens, max_new = event
            if name in requests and requests[name].state != "finished":
                fail(index, f"request {name!r} submitted twice")
            if prompt_tokens <= 0 or max_new <= 0:
                fail(index, f"request {name!r} accepted with {prompt_tokens} prompt tokens and {max_new} to make")
            requests[name] = RequestTrace(prompt_tokens, max_new)
        elif kind == "admit":
            trace = known(index, event[1], "queued")
            trace.state, trace.held, trace.held_before = "live", 0, 0
            live = sum(1 for t in requests.values() if t.state == "live")
            peak_live = max(peak_live, live)
            if live > figures.max_live_requests:
                fail(index, f"{live} live requests, the limit is {figures.max_live_requests}")
        elif kind == "preempt":
            if ahead is not None:
                fail(index, f"request {event[1]!r} preempted while a step is planned ahead")
            trace = known(index, event[1], "live")
            if event[1] in in_flight and event[1] in awaiting:
                fail(index, f"request {event[1]!r} preempted while its row is in flight")
            if event[2] != trace.prompt_tokens + len(trace.emitted):
                fail(index, f"request {event[1]!r} preempted knowing {event[2]} tokens, the log shows "
                            f"{trace.prompt_tokens + len(trace.emitted)}")
            trace.state, trace.held = "queued", 0
            trace.preemptions += 1
        elif kind == "ahead":
            rows = event[1]
            if ahead is not None:
                fail(index, "a second step planned ahead")
            if not in_flight or sorted(map(str, awaiting)) != sorted(map(str, in_flight)):
                fail(index, "a step is planned ahead, but not every row of the step in flight owes a token")
            if [name for name, _, _, _ in rows] != in_flight:
                fail(index, "the step planned ahead does not hold the requests of the step in flight in their order")
            live = [name for name, t in requests.items() if t.state == "live"]
            if sorted(map(str, live)) != sorted(map(str, in_flight)):
                fail(index, "a step is planned ahead although a live request is not in the step in flight")
            steps += 1
            ahead = {}
            for name, start, count, sample in rows:
                trace = known(index, name, "live")
                if count != 1 or not sample:
                    fail(index, f"request {name!r}: a step planned ahead holds one sampling row a request")
                if start != trace.held or start != awaiting[name] + 1:
                    fail(index, f"request {name!r} runs ahead from position {start}, it holds {trace.held} and is "
                                f"owed the token of position {awaiting[name]}")
                if len(trace.emitted) + 1 >= trace.max_new_tokens:
                    fail(index, f"request {name!r} is planned beyond the last token it may be given")
                trace.held_before = trace.held       # the step in flight is committed: what its window passed is back
                trace.held += 1
                trace.fed += 1
                ahead[name] = start
            peak_tokens = max(peak_tokens, len(rows))
            if len(rows) > figures.max_step_tokens:
                fail(index, f"a step of {len(rows)} tokens, the budget is {figures.max_step_tokens}")
            for g, (pool, used) in enumerate(zip(figures.pools, pages_now())):
                peak_pages[g] = max(peak_pages[g], used)
                if used > pool.num_pages:
                    fail(index, f"group {g} needs {used} pages, the pool has {pool.num_pages}")
        elif kind == "step":
            if ahead is not None:
                fail(index, "a step starts while another is planned ahead and not yet in flight")
            if awaiting:
                fail(index, f"a step starts while rows of the last one still owe tokens: {sorted(map(str, awaiting))}")
            rows = event[1]
            if not rows:
                fail(index, "a step without entries")
            steps += 1
            in_flight, total = [], 0
            for trace in requests.values():
                trace.held_before = trace.held
            for name, start, count, sample in rows:
                trace = known(index, name, "live")
                if name in in_flight:
                    fail(index, f"request {name!r} twice in one step")
                in_flight.append(name)
                if count <= 0:
                    fail(index, f"request {name!r} runs {count} tokens")
                if start != trace.held:
                    fail(index, f"request {name!r} runs from position {start}, it holds {trace.held}")
                have = trace.prompt_tokens + len(trace.emitted)
                if start + count > have:
                    fail(index, f"request {name!r} runs positions up to {start + count}, only {have} tokens are known")
                if count > 1 and count > figures.prefill_chunk_tokens:
                    fail(index, f"request {name!r} runs a portion of {count}, the limit is {figures.prefill_chunk_tokens}")
                if bool(sample) != (start + count == have):
                    fail(index, f"request {name!r}: sampling is {bool(sample)} but the portion ends at {start + count} of {have}")
                trace.held += count
                trace.fed += count
                total += count
                if sample:
                    awaiting[name] = start + count - 1
            peak_tokens = max(peak_tokens, total)
            if total > figures.max_step_tokens:
                fail(index, f"a step of {total} tokens, the budget is {figures.max_step_tokens}")
            for g, (pool, used) in enumerate(zip(figures.pools, pages_now())):
                peak_pages[g] = max(peak_pages[g], used)
                if used > pool.num_pages:
                    fail(index, f"group {g} needs {used} pages, the pool has {pool.num_pages}")
        elif kind == "token":
            _, name, position, token = event
            trace = known(index, name, "live")
            if awaiting.get(name) != position:
                fail(index, f"request {name!r} is given a token for position {position}, "
                            f"the step in flight owes {awaiting.get(name)}")
            del awaiting[name]
            if position in trace.emitted and trace.emitted[position] != token:
                fail(index, f"request {name!r}: position {position} gave {trace.emitted[position]} before and {token} now")
            if position != trace.prompt_tokens + len(trace.emitted) - 1 and position not in trace.emitted:
                fail(index, f"request {name!r}: token for position {position} out of order")
            trace.emitted[position] = token
            if len(trace.emitted) > trace.max_new_tokens:
                fail(index, f"request {name!r} was given {len(trace.emitted)} tokens, its limit is {trace.max_new_tokens}")
        elif kind == "finish":
            _, name, reason = event
            trace = known(index, name, "live", "queued")
            if reason == "aborted":
                awaiting.pop(name, None)         # the step failed: its rows owe nothing
            elif name in awaiting:
                fail(index, f"request {name!r} finishes ({reason}) while its row is in flight")
            if reason == "length" and len(trace.emitted) != trace.max_new_tokens:
                fail(index, f"request {name!r} finished for length with {len(trace.emitted)} of {trace.max_new_tokens} tokens")
            if reason == "eos" and not trace.emitted:
                fail(index, f"request {name!r} finished on an end token it was never given")
            trace.state, trace.reason, trace.held = "finished", reason, 0
            if ahead is not None:
                ahead.pop(name, None)            # it drops out of the step ahead
        else:
            fail(index, f"unknown event {kind!r}")
        # Once every row of the step in flight is answered (and the request of the last answer has had its chance
        # to finish: its finish follows its token at once), the step planned ahead is the step in flight.
        if ahead is not None and not awaiting and kind in ("token", "finish"):
            following = events_list[index + 1] if index + 1 < len(events_list) else None
            if not (following is not None and following[0] == "finish" and kind == "token" and following[1] == event[1]):
                in_flight = [name for name in in_flight if name in ahead]
                awaiting = dict(ahead)
                ahead = None
    return TraceReport(requests, rejected, steps, peak_pages, peak_live, peak_tokens)


def figures_of(scheduler) -> RunFigures:
    """The figures of a ``Scheduler`` (its policy and its cache manager's groups)."""
    cache = scheduler.cache
    pools = [PoolFigures(spec.num_pages, spec.page_tokens, int(spec.window or 0)) for spec in cache.groups]
    policy = scheduler.policy
    return RunFigures(pools, policy.max_live_requests, policy.max_step_tokens, policy.prefill_chunk_tokens)
