"""The scheduler's decisions, with a stand-in executor whose tokens are a pure function of the
request's history, so an interleaved run can be compared with each request run alone
(the reference's isolated-oracle pattern, crates/leone/src/scheduler.rs:1626-1655)."""
import random

import pytest

from leone_amd.cache.manager import CacheManager, GroupSpec
from leone_amd.engine.scheduler import Reject, Request, Scheduler, SchedulerError, SchedulerPolicy


def next_token(history):
    """Deterministic stand-in for model + sampler: depends on every earlier token and the position."""
    value = 17
    for i, t in enumerate(history):
        value = (value * 31 + t * (i + 1)) % 1009
    return value % 97


def run(scheduler, fail_at_step=None):
    """Drives plans to completion; commits the cache as the engine would."""
    steps = 0
    while scheduler.has_work():
        plan = scheduler.plan()
        steps += 1
        if fail_at_step == steps:
            scheduler.abort()
            continue
        sampled = {}
        for entry in plan:
            assert scheduler.cache.length(entry.request) == entry.start
            scheduler.cache.commit(entry.request, len(entry.tokens))
            if entry.sample:
                state = scheduler.live[entry.request]
                assert state.tokens[:entry.start + len(entry.tokens)] == state.tokens
                sampled[entry.request] = next_token(state.tokens)
        scheduler.complete(sampled)
        scheduler.cache.check()
        assert steps < 100000
    return steps


def run_ahead(scheduler, fail_at_step=None):
    """The same with a step planned ahead wherever the scheduler allows one: the step that has run is completed
    only after the next one has been planned and "launched" (its cache writes committed), as a caller does that
    keeps the chosen tokens on the device.  Returns (steps, steps that were planned ahead)."""
    steps = looked = 0
    pending = None                                   # the step that has run and is not completed yet
    while scheduler.has_work():
        if pending is None:
            pending = scheduler.plan()
            steps += 1
            for entry in pending:
                assert scheduler.cache.length(entry.request) == entry.start
                scheduler.cache.commit(entry.request, len(entry.tokens))
        if fail_at_step == steps:
            scheduler.abort()
            pending = None
            continue
        ahead = scheduler.plan_ahead()
        if ahead:
            assert [(e.request, e.start, e.deferred) for e in ahead] == \
                [(e.request, e.start + len(e.tokens), True) for e in pending]
            steps += 1
            looked += 1
            for entry in ahead:
                scheduler.cache.commit(entry.request, 1)
            if fail_at_step == steps:                # the step ahead fails: both go
                scheduler.abort()
                pending = None
                continue
        sampled = {e.request: next_token(scheduler.live[e.request].tokens) for e in pending if e.sample}
        scheduler.complete(sampled)
        scheduler.cache.check()
        live = scheduler.live
        pending = [e for e in ahead if e.request in live] or None
        assert steps < 100000
    return steps, looked


def isolated(prompt, n, eos=None):
    tokens = list(prompt)
    for _ in range(n):
        tokens.append(next_token(tokens))
        if eos is not None and tokens[-1] == eos:
            break
    return tokens[len(prompt):]


def make(pages=64, page_tokens=16, max_requests=8, context=4096, **policy):
    cache = CacheManager([GroupSpec(pages, page_tokens)], max_requests, context)
    return Scheduler(SchedulerPolicy(**policy), cache)


def test_prompt_is_cut_into_portions_under_the_budget():
    # prompt 13, chunk 8: portions of 8 and 5, then one token a step (crates/leone/src/scheduler.rs:1723-1764)
    s = make(prefill_chunk_tokens=8, max_step_tokens=64)
    assert s.submit(Request("a", list(range(13)), 3)) is None
    first = s.plan()
    assert [(e.start, len(e.tokens), e.sample) for e in first] == [(0, 8, False)]
    s.cache.commit("a"); s.complete({})
    second = s.plan()
    assert [(e.start, len(e.tokens), e.sample) for e in second] == [(8, 5, True)]
    assert second[0].sample_position == 12
    s.cache.commit("a"); s.complete({"a": 50})
    third = s.plan()
    assert [(e.start, e.tokens, e.sample) for e in third] == [(13, [50], True)]
    s.cache.commit("a"); s.complete({"a": 51})
    fourth = s.plan()
    s.cache.commit("a")
    done = s.complete({"a": 52})
    assert done[0].tokens == [50, 51, 52] and done[0].reason == "length"
    assert not s.has_work() and s.cache.free_pages(0) == 64 and s.cache.free_slots() == 8


def test_token_budget_covers_decode_rows_first_then_portions():
    s = make(prefill_chunk_tokens=100, max_step_tokens=10)
    for i in range(3):
        s.submit(Request(i, [1, 2], 5))
    plan = s.plan()
    assert sorted(len(e.tokens) for e in plan) == [2, 2, 2]
    for e in plan:
        s.cache.commit(e.request)
    s.complete({e.request: 7 for e in plan})
    s.submit(Request("long", list(range(50)), 2))
    plan = s.plan()
    kinds = [(e.request, len(e.tokens)) for e in plan]
    assert kinds[:3] == [(0, 1), (1, 1), (2, 1)] and kinds[3] == ("long", 7)    # 10 - 3 decode rows
    assert sum(n for _, n in kinds) == 10


def test_typed_rejections_hold_nothing():
    s = make(pages=4, page_tokens=16, context=100, max_prompt_tokens=40, max_output_tokens=30,
             max_queued_requests=2)
    assert s.submit(Request("p0", [], 5)) is Reject.PROMPT_LIMIT
    assert s.submit(Request("p1", [1] * 41, 5)) is Reject.PROMPT_LIMIT
    assert s.submit(Request("o0", [1], 0)) is Reject.OUTPUT_LIMIT
    assert s.submit(Request("o1", [1], 31)) is Reject.OUTPUT_LIMIT
    assert s.submit(Request("k", [1] * 40, 30)) is Reject.KV_CAPACITY     # 69 tokens > 4 pages of 16
    assert s.submit(Request("ok1", [1] * 40, 25)) is None                 # 64 tokens fit exactly
    assert s.submit(Request("ok1", [1], 1)) is Reject.DUPLICATE
    assert s.submit(Request("ok2", [1], 1)) is None
    assert s.submit(Request("q", [1], 1)) is Reject.QUEUE_LIMIT
    assert s.stats.rejected == 7 and s.cache.free_pages(0) == 4 and s.cache.free_slots() == 8
    small = make(context=10)
    assert small.submit(Request("c", [1] * 8, 4)) is Reject.CONTEXT_LIMIT  # 8 + 4 - 1 > 10
    assert small.submit(Request("c", [1] * 8, 3)) is None


def test_live_limit_and_admission_order():
    # a cap of 4 live requests out of 6 (crates/leone/src/scheduler.rs:1853-1859)
    s = make(max_live_requests=4)
    for i in range(6):
        s.submit(Request(i, [i + 1], 2))
    plan = s.plan()
    assert [e.request for e in plan] == [0, 1, 2, 3]
    assert s.stats.max_live == 4


def test_interleaved_equals_isolated_with_eos_and_cancel():
    rng = random.Random(5)
    s = make(pages=40, page_tokens=8, max_live_requests=5, prefill_chunk_tokens=7, max_step_tokens=16)
    wanted = {}
    for i in range(12):
        prompt = [rng.randrange(97) for _ in range(rng.choice([1, 2, 9, 30, 61]))]
        n = rng.choice([1, 4, 17])
        eos = 13 if i % 3 == 0 else None
        assert s.submit(Request(i, prompt, n, eos_token_id=eos)) is None
        wanted[i] = isolated(prompt, n, eos)
    s.cancel(11)                                   # still queued: gone at once
    run(s)
    by_id = {f.id: f for f in s.finished}
    assert by_id[11].reason == "cancelled" and by_id[11].tokens == []
    for i in range(11):
        assert by_id[i].tokens == wanted[i], i
        assert by_id[i].reason == ("eos" if by_id[i].tokens[-1:] == [13] and i % 3 == 0 else "length")
    assert s.cache.free_pages(0) == 40 and s.cache.free_slots() == 8 and not s.live and not s.queue
    assert s.stats.max_step_rows <= 16


def test_cancel_of_a_live_request_takes_effect_at_the_next_step():
    s = make()
    s.submit(Request("a", [1, 2, 3], 10))
    plan = s.plan(); s.cache.commit("a"); s.complete({"a": 5})
    assert s.cancel("a") and "a" in s.live
    assert s.plan() == []
    assert s.finished[-1].reason == "cancelled" and s.finished[-1].tokens == [5]
    assert s.cache.free_pages(0) == 64 and not s.cancel("nobody")


def test_when_pages_run_out_the_newest_request_is_preempted_and_recomputed():
    """Two requests that together outgrow the pool: the younger is released, requeued with its
    generated tokens as prompt, and still ends with the tokens it would produce alone."""
    s = make(pages=6, page_tokens=4, max_step_tokens=64, prefill_chunk_tokens=64)
    a, b = [3, 1, 4, 1, 5, 9, 2], [2, 7, 1, 8, 2, 8]
    s.submit(Request("a", a, 14))
    s.submit(Request("b", b, 12))
    run(s)
    by_id = {f.id: f for f in s.finished}
    assert by_id["a"].tokens == isolated(a, 14) and by_id["b"].tokens == isolated(b, 12)
    assert s.stats.preemptions >= 1 and by_id["b"].preemptions >= 1 and by_id["a"].preemptions == 0
    assert [e for e in s.events if e[0] == "preempt"][0][1] == "b"
    assert s.cache.free_pages(0) == 6


def test_prompt_portion_shrinks_to_the_free_pages_and_older_requests_go_first():
    s = make(pages=5, page_tokens=4, max_step_tokens=64, prefill_chunk_tokens=64)
    s.submit(Request("a", list(range(12)), 2))      # 3 pages
    plan = s.plan(); s.cache.commit("a"); s.complete({"a": 1})
    s.submit(Request("b", list(range(20)), 1))      # needs 5 pages in all; 2 are free now
    plan = s.plan()
    assert [(e.request, len(e.tokens)) for e in plan] == [("a", 1)]      # b waits: its tokens do not fit yet
    s.cache.commit("a"); s.complete({"a": 2})        # a finishes and frees its pages
    plan = s.plan()
    assert [(e.request, len(e.tokens), e.sample) for e in plan] == [("b", 20, True)]


def test_failed_step_aborts_its_requests_and_frees_everything():
    # crates/leone/src/service.rs:270-297
    s = make()
    s.submit(Request("a", [1, 2, 3], 4))
    s.submit(Request("b", [4, 5], 4))
    run(s, fail_at_step=2)
    assert {f.id: f.reason for f in s.finished} == {"a": "aborted", "b": "aborted"}
    assert s.cache.free_pages(0) == 64 and s.cache.free_slots() == 8
    with pytest.raises(SchedulerError):
        s.complete({})


@pytest.mark.parametrize("seed", range(5))
def test_random_load_under_page_pressure(seed):
    rng = random.Random(100 + seed)
    s = make(pages=rng.choice([10, 14, 24]), page_tokens=rng.choice([4, 8]), max_live_requests=4,
             prefill_chunk_tokens=rng.choice([3, 16, 64]), max_step_tokens=rng.choice([8, 24, 200]))
    capacity = s.cache.groups[0].num_pages * s.cache.groups[0].page_tokens
    wanted = {}
    for i in range(25):
        prompt = [rng.randrange(97) for _ in range(rng.randrange(1, 40))]
        n = rng.randrange(1, 30)
        result = s.submit(Request(i, prompt, n))
        if len(prompt) + n - 1 > capacity:
            assert result is Reject.KV_CAPACITY
        else:
            assert result is None
            wanted[i] = isolated(prompt, n)
    run(s)
    assert {f.id: f.tokens for f in s.finished} == wanted
    assert s.cache.free_pages(0) == s.cache.groups[0].num_pages
    # events alone show that no request got a position twice after its last preemption
    fed = {}
    for event in s.events:
        if event[0] == "preempt":
            fed[event[1]] = 0
        elif event[0] == "step":
            for rid, start, count, _ in event[1]:
                assert fed.get(rid, 0) == start
                fed[rid] = start + count


# ---- the checker that works from the decision log alone ------------------------------------------

def _loaded(seed, window=None, ahead=False):
    from leone_amd.engine import trace_check
    rng = random.Random(500 + seed)
    page_tokens = rng.choice([4, 8])
    groups = [GroupSpec(rng.choice([12, 16, 24]), page_tokens)]
    if window:
        groups.append(GroupSpec(12, page_tokens, window))
    cache = CacheManager(groups, 8, 4096)
    s = Scheduler(SchedulerPolicy(max_live_requests=4, prefill_chunk_tokens=rng.choice([3, 16, 64]),
                                  max_step_tokens=rng.choice([8, 24, 200])), cache)
    wanted = {}
    for i in range(20):
        prompt = [rng.randrange(97) for _ in range(rng.randrange(1, 40))]
        n = rng.randrange(1, 30)
        if s.submit(Request(i, prompt, n, eos_token_id=rng.choice([None, 5]))) is None:
            wanted[i] = (prompt, n)
    if seed % 2:
        s.cancel(3)
    if ahead:
        s.looked_ahead = run_ahead(s, fail_at_step=40 if seed == 2 else None)[1]
    else:
        run(s, fail_at_step=7 if seed == 2 else None)
    return s, wanted, trace_check


@pytest.mark.parametrize("ahead", [False, True])
@pytest.mark.parametrize("window", [None, 9])
@pytest.mark.parametrize("seed", range(4))
def test_the_log_alone_shows_a_sound_run(seed, window, ahead):
    """Page conservation, budgets, one step in flight and contiguous positions are re-derived from the
    events by a checker that shares nothing with the scheduler, and the transcript it reads off the events
    equals every request run alone (crates/leone/src/scheduler.rs:1349-1655).  The same with a step planned
    ahead of the tokens wherever the scheduler allows it: the tokens are the same, a request that ends on its
    end token drops out of the step ahead, and a failed step takes the step ahead with it."""
    s, wanted, trace_check = _loaded(seed, window, ahead)
    assert not ahead or s.looked_ahead > 5
    figures = trace_check.figures_of(s)
    report = trace_check.verify_events(s.events, figures)
    assert report.steps == s.stats.steps and report.peak_live <= 4
    assert report.peak_pages == s.cache.pages_high_water
    assert report.peak_step_tokens <= s.policy.max_step_tokens
    finished = {f.id: f for f in s.finished}
    assert set(report.requests) == set(wanted)
    for rid, trace in report.requests.items():
        assert trace.state == "finished" and trace.reason == finished[rid].reason
        assert trace.tokens == finished[rid].tokens and trace.preemptions == finished[rid].preemptions
        if trace.reason in ("eos", "length"):
            prompt, n = wanted[rid]
            assert trace.tokens == isolated(prompt, n, eos=5 if trace.reason == "eos" else None)[:len(trace.tokens)]
            assert trace.fed >= len(prompt) + len(trace.tokens) - 1


def test_the_checker_refuses_a_log_that_breaks_a_rule():
    s, wanted, trace_check = _loaded(0)
    figures = trace_check.figures_of(s)
    events = s.events
    trace_check.verify_events(events, figures)

    def broken(change):
        changed = [list(e) if e[0] != "step" else ["step", [list(r) for r in e[1]]] for e in events]
        change(changed)
        with pytest.raises(trace_check.TraceError):
            trace_check.verify_events([tuple(e) for e in changed], figures)

    first_step = next(i for i, e in enumerate(events) if e[0] == "step")
    first_token = next(i for i, e in enumerate(events) if e[0] == "token")
    later_step = next(i for i, e in enumerate(events) if e[0] == "step" and i > first_token and e[1][0][1] > 0)
    broken(lambda ev: ev.pop(first_token))                                   # a row's token never arrives
    broken(lambda ev: ev.insert(first_token, ev[first_token]))               # a token twice
    broken(lambda ev: ev[later_step][1][0].__setitem__(1, ev[later_step][1][0][1] + 1))   # a position skipped
    broken(lambda ev: ev[later_step][1][0].__setitem__(1, ev[later_step][1][0][1] - 1))   # a position fed twice
    broken(lambda ev: ev[first_step][1].append(list(ev[first_step][1][0])))  # a request twice in a step
    broken(lambda ev: ev.insert(first_step, ev[first_step]))                 # two steps in flight
    broken(lambda ev: ev.append(("token", 0, 5, 1)))                         # something after the end
    broken(lambda ev: ev.pop(next(i for i, e in enumerate(ev) if e[0] == "admit")))   # a step for a queued request
    import dataclasses
    with pytest.raises(trace_check.TraceError, match="pages"):
        small = dataclasses.replace(figures, pools=[trace_check.PoolFigures(figures.pools[0].num_pages // 3,
                                                                             figures.pools[0].page_tokens)])
        trace_check.verify_events(events, small)
    with pytest.raises(trace_check.TraceError, match="budget"):
        trace_check.verify_events(events, dataclasses.replace(figures, max_step_tokens=1))
    with pytest.raises(trace_check.TraceError, match="live requests"):
        trace_check.verify_events(events, dataclasses.replace(figures, max_live_requests=1))


def test_a_step_is_planned_ahead_only_where_the_next_step_is_known():
    s = make(pages=8, page_tokens=4, prefill_chunk_tokens=8, max_step_tokens=16, max_live_requests=2)
    with pytest.raises(SchedulerError, match="no step is planned"):
        s.plan_ahead()
    assert s.submit(Request("a", list(range(12)), 6)) is None
    s.plan()                                                           # a portion that does not end the prompt
    s.cache.commit("a")
    assert s.plan_ahead() == [] and s.cache.length("a") == 8
    s.complete({})
    s.plan()                                                           # the rest of the prompt: a token comes of it
    with pytest.raises(SchedulerError, match="has not run"):
        s.plan_ahead()
    s.cache.commit("a")
    free = s.cache.free_pages(0)
    ahead = s.plan_ahead()
    assert [(e.request, e.start, e.tokens, e.sample, e.deferred) for e in ahead] == [("a", 12, [0], True, True)]
    assert s.cache.free_pages(0) == free - 1                           # position 12 opens a page: it is reserved
    with pytest.raises(SchedulerError, match="already"):
        s.plan_ahead()
    with pytest.raises(SchedulerError, match="neither completed"):
        s.plan()
    s.cache.commit("a", 1)
    assert s.complete({"a": 7}) == [] and s.history("a")[-1] == 7
    # the step ahead is the planned one now; somebody in the queue with a place free: no looking ahead
    assert s.submit(Request("b", [1, 2, 3], 9)) is None
    assert s.plan_ahead() == []
    s.complete({"a": 8})
    both = s.plan()
    assert [e.request for e in both] == ["a", "b"]
    for e in both:
        s.cache.commit(e.request)
    # the queue is empty and both get a token: ahead, step after step, until "a" is one token from its sixth
    token, given = 9, 2
    while True:
        ahead = s.plan_ahead()
        if given + 1 >= 6:                         # the token the planned step is choosing is its last
            assert ahead == []
            break
        assert [(e.request, e.start) for e in ahead] == [(e.request, e.start + len(e.tokens)) for e in both]
        for e in ahead:
            s.cache.commit(e.request, 1)
        assert s.complete({"a": token, "b": token + 20}) == []
        both, token, given = ahead, token + 1, given + 1
    done = s.complete({"a": 50, "b": 51})
    assert [f.id for f in done] == ["a"] and done[0].reason == "length" and done[0].tokens == [7, 8, 9, 10, 11, 50]
    # an end token drops a request out of the step ahead, and what it held goes back
    s2 = make(pages=8, page_tokens=4, max_live_requests=2)
    s2.submit(Request("x", [1, 2, 3], 9, eos_token_id=5)), s2.submit(Request("y", [4, 5], 9, eos_token_id=5))
    for e in s2.plan():
        s2.cache.commit(e.request)
    ahead = s2.plan_ahead()
    assert len(ahead) == 2
    for e in ahead:
        s2.cache.commit(e.request, 1)
    done = s2.complete({"x": 5, "y": 6})
    assert [f.id for f in done] == ["x"] and done[0].reason == "eos" and not s2.cache.has("x")
    assert [e.request for e in s2.plan_ahead()] == ["y"]               # the step that was ahead is the planned one: "y" alone
    s2.cache.check()


def test_the_checker_refuses_a_step_ahead_that_breaks_a_rule():
    s, wanted, trace_check = _loaded(1, ahead=True)
    figures = trace_check.figures_of(s)
    events = s.events
    trace_check.verify_events(events, figures)
    first_ahead = next(i for i, e in enumerate(events) if e[0] == "ahead")
    with_two = next(i for i, e in enumerate(events) if e[0] == "ahead" and len(e[1]) >= 2)

    def broken(change):
        changed = [list(e) if e[0] not in ("step", "ahead") else [e[0], [list(r) for r in e[1]]] for e in events]
        change(changed)
        with pytest.raises(trace_check.TraceError):
            trace_check.verify_events([tuple(e) for e in changed], figures)

    broken(lambda ev: ev.insert(first_ahead, ev[first_ahead]))                          # two steps ahead
    broken(lambda ev: ev[with_two][1].pop())                                            # a request of the step in flight left out
    broken(lambda ev: ev[with_two][1].reverse())                                        # another order than the step in flight
    broken(lambda ev: ev[first_ahead][1][0].__setitem__(1, ev[first_ahead][1][0][1] + 1))   # a position skipped
    broken(lambda ev: ev[first_ahead][1][0].__setitem__(2, 2))                          # two rows for a request
    broken(lambda ev: ev.__setitem__(first_ahead, ["step", ev[first_ahead][1]]))        # an ordinary step before the tokens
    broken(lambda ev: ev.insert(first_ahead + 1, ["preempt", ev[first_ahead][1][0][0], 1]))   # a decision while a step is ahead
    # a step ahead after the first token of the step in flight has come: not every row owes its token
    first_token_after = next(i for i in range(with_two, len(events)) if events[i][0] == "token")

    def late(ev):
        ev.insert(first_token_after + 1, ev.pop(with_two))
    broken(late)
