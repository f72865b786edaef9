"""Generation: the scheduler's plans run through the engine's step, tokens chosen by the sampler.

The reference's entry points are ``Runtime::load`` and ``generate`` / ``generate_tokens`` with
``GenerateOptions`` (crates/leone/src/runtime.rs:1305, 3524-3540, 251-287) returning the generated
tokens, why generation stopped and timing (crates/leone/src/runtime.rs:442-452, 402-427).
"""
from __future__ import annotations

import time
from dataclasses import dataclass
from typing import Callable, Dict, Hashable, List, Optional, Sequence, Union

import numpy as np
import torch

from .. import ops
from ..ops.profile import Recorder
from ..sampling import rng
from ..sampling.sampler import (MirostatState, SamplerError, SamplingParams, apply_penalties, native_eligible,
                                sample as host_sample, sample_rows_native)
from .engine import Engine, StepEntry
from .scheduler import Finished, PlannedEntry, Reject, Request, Scheduler, SchedulerPolicy


@dataclass
class GenerationStats:
    prompt_tokens: int = 0
    emitted_tokens: int = 0
    steps: int = 0
    prefill_seconds: float = 0.0     # steps that held a prompt portion
    decode_seconds: float = 0.0      # steps of decoded tokens only
    prefill_tokens: int = 0
    decode_tokens: int = 0
    preemptions: int = 0
    steps_ahead: int = 0             # steps issued before the tokens of the step before them had reached the host

    @property
    def prefill_rate(self) -> float:
        return self.prefill_tokens / self.prefill_seconds if self.prefill_seconds > 0 else 0.0

    @property
    def decode_rate(self) -> float:
        return self.decode_tokens / self.decode_seconds if self.decode_seconds > 0 else 0.0


@dataclass
class GenerationResult:
    id: Hashable
    prompt_tokens: List[int]
    tokens: List[int]
    finish_reason: str


class RequestRejected(ValueError):
    def __init__(self, request_id, reason: Reject):
        super().__init__(f"request {request_id!r} rejected: {reason.value}")
        self.reason = reason


def device_kind(policy: SamplingParams) -> Optional[str]:
    """Which device kernel chooses a row's token under this policy: "greedy", "temperature" (nothing cut), or
    "truncated" (stages that begin with a top-k the selection kernel can serve); None if the row has to come
    to the host: penalties, a Mirostat controller, other stages."""
    if policy.penalties_active or policy.mirostat is not None:
        return None
    if policy.greedy:
        return "greedy"
    if not policy.truncations:
        return "temperature"
    return "truncated" if ops.truncated_draw_supported(policy.truncations) else None


class DeviceChoice:
    """What the device kernels need to choose a step's tokens, uploaded before the step's logits exist (so that
    the upload does not stand between the step and the kernels that choose): temperatures and uniform values, the
    table of truncation stages, and which kernel's answer each row takes.  ``kinds`` holds for every sampled row
    its ``device_kind`` or None; rows with None get nothing of meaning."""

    def __init__(self, rows: Sequence[PlannedEntry], policies: Sequence[SamplingParams],
                 kinds: Sequence[Optional[str]], device, staging: Optional[Callable[[int], torch.Tensor]] = None):
        """``staging(n)``: pinned host memory for n float64 values that stays untouched until the upload has
        happened; the upload then waits for nothing and holds nobody up (a copy out of ordinary memory makes the
        host wait for everything the stream still has to do: the step in flight)."""
        self.kinds = list(kinds)
        count = len(rows)
        draws = [rng.uniform(p.seed, e.sample_position) if kind in ("temperature", "truncated") else 0.0
                 for p, e, kind in zip(policies, rows, kinds)]
        pieces = []
        if "temperature" in kinds:
            pieces.append(np.array([[p.temperature if kind == "temperature" else 1.0 for p, kind in zip(policies, kinds)],
                                    draws], dtype=np.float64).reshape(-1))
        if "truncated" in kinds:
            pieces.append(ops.truncated_rows([(p.temperature, u, p.truncations) if kind == "truncated" else None
                                              for p, u, kind in zip(policies, draws, kinds)]).reshape(-1))
        # which rows take the answer of the second and third kernel (a batch of one kind needs none)
        self.names = [name for name in ("greedy", "temperature", "truncated") if name in kinds]
        for name in self.names[1:]:
            pieces.append(np.array([1.0 if kind == name else 0.0 for kind in kinds], dtype=np.float64))
        self.scaled = self.truncated = None
        self.masks = {}
        if pieces:
            flat = np.concatenate(pieces)
            if staging is not None:
                host = staging(flat.size)
                host.numpy()[:] = flat
                on_device = host.to(device, non_blocking=True)
            else:
                on_device = torch.from_numpy(flat).to(device)
            at = 0
            if "temperature" in kinds:
                self.scaled = on_device[:2 * count].view(2, count)
                at = 2 * count
            if "truncated" in kinds:
                width = 3 + 2 * ops.TRUNCATED_STAGES
                self.truncated = on_device[at:at + count * width].view(count, width)
                at += count * width
            for name in self.names[1:]:
                self.masks[name] = on_device[at:at + count] != 0.0
                at += count

    def choose(self, logits: torch.Tensor) -> torch.Tensor:
        """int32 [rows] on the device: the token each row's kernel chose, -1 for a row without a finite logit.
        Each kernel runs once, over all rows."""
        out = None
        for name in self.names:
            if name == "greedy":
                chosen = ops.argmax(logits)
            elif name == "temperature":
                chosen = ops.sample_temperature(logits, self.scaled[0], self.scaled[1])
            else:
                chosen = ops.sample_truncated(logits, self.truncated)
            out = chosen if out is None else torch.where(self.masks[name], chosen, out)
        return out


def plan_device_choice(entries: Sequence[PlannedEntry], params: Dict[Hashable, SamplingParams], device,
                       staging: Optional[Callable[[int], torch.Tensor]] = None) -> Optional[DeviceChoice]:
    """The ``DeviceChoice`` of a step if device kernels choose every one of its tokens; None otherwise."""
    rows = [e for e in entries if e.sample]
    policies = [params[e.request] or SamplingParams() for e in rows]
    for p in policies:
        p.validate()
    kinds = [device_kind(p) for p in policies]
    if not rows or not all(kinds):
        return None
    return DeviceChoice(rows, policies, kinds, device, staging)


def choose_tokens(logits: torch.Tensor, entries: Sequence[PlannedEntry], params: Dict[Hashable, SamplingParams],
                  history: Callable[[Hashable], Sequence[int]],
                  controllers: Optional[Dict[Hashable, MirostatState]] = None) -> Dict[Hashable, int]:
    """One token per sampled entry; ``logits`` has one row per such entry, in order.

    Greedy rows, plain-temperature rows and rows whose stages begin with a top-k of modest size are chosen by
    the device kernels; rows with other stages, penalties or a controller are copied to the host and go through
    the double-precision sampler, which reads a request's tokens so far through ``history``."""
    rows = [e for e in entries if e.sample]
    if not rows:
        return {}
    policies = [params[e.request] or SamplingParams() for e in rows]
    for p in policies:
        p.validate()
    out: Dict[Hashable, int] = {}
    kinds = [None if e.request in (controllers or {}) else device_kind(p) for e, p in zip(rows, policies)]
    if any(kinds):
        picked = DeviceChoice(rows, policies, kinds, logits.device).choose(logits).cpu().tolist()
        for e, kind, token in zip(rows, kinds, picked):
            if kind is not None:
                out[e.request] = token
    host_rows = [i for i, kind in enumerate(kinds) if kind is None]
    if host_rows:
        index = torch.tensor(host_rows, dtype=torch.long, device=logits.device)
        copied = logits.index_select(0, index).cpu().numpy()
        # Rows whose stages the host library knows are drawn there together, after their penalties;
        # the others go through the general sampler one by one.
        together = [k for k, i in enumerate(host_rows)
                    if native_eligible(policies[i]) and rows[i].request not in (controllers or {})]
        for k in together:
            i = host_rows[k]
            if policies[i].penalties_active:
                copied[k] = apply_penalties(copied[k], history(rows[i].request), policies[i])
        if together:
            drawn = sample_rows_native(copied[together], [policies[host_rows[k]] for k in together],
                                       [rows[host_rows[k]].sample_position for k in together])
            for k, token in zip(together, drawn):
                out[rows[host_rows[k]].request] = token
        for k, i in enumerate(host_rows):
            if k in together:
                continue
            e = rows[i]
            out[e.request] = host_sample(copied[k], policies[i], e.sample_position, history(e.request),
                                         (controllers or {}).get(e.request))
    for e in rows:
        if out[e.request] < 0:
            raise SamplerError(f"request {e.request!r}: no finite logit at position {e.sample_position}")
    return out


def choose_on_device(logits: torch.Tensor, entries: Sequence[PlannedEntry],
                     params: Dict[Hashable, SamplingParams]) -> Optional[torch.Tensor]:
    """The tokens of the sampled entries as int32 on the device, in their order, without a copy to the host; None
    unless every one of them is chosen by a device kernel (``device_kind``).  -1 stands for a row without a
    finite logit."""
    choice = plan_device_choice(entries, params, logits.device)
    return None if choice is None else choice.choose(logits)


@dataclass
class _InFlight:
    """A step that has been issued and whose tokens have not been reported to the scheduler yet."""
    plan: List[PlannedEntry]
    logits: Optional[torch.Tensor]
    picked: Optional[torch.Tensor]       # the chosen tokens on the device, if device kernels chose them all
    decoding: bool
    started: float
    recorder: Optional[Recorder] = None
    exact: bool = True                   # its rows are still the scheduler's planned rows, one for one
    host: Optional[torch.Tensor] = None  # the chosen tokens on their way into pinned host memory; `arrived` says when they are there
    arrived: Optional[torch.cuda.Event] = None


class Generator:
    """Runs requests to completion: scheduler above, engine below.

    ``look_ahead``: where the scheduler can plan the next step before the tokens of the one in flight are known
    (a step of decoded tokens for the same requests; ``Scheduler.plan_ahead``) and device kernels choose those
    tokens, the next step is issued with the tokens taken from the device, and only then are the earlier step's
    tokens copied to the host and reported: planning, the step's metadata and the launch overlap the step in
    flight instead of standing between two steps.  The tokens are the same either way."""

    def __init__(self, engine: Engine, policy: Optional[SchedulerPolicy] = None):
        self.engine = engine
        self.scheduler = Scheduler(policy or SchedulerPolicy(max_live_requests=engine.cache.max_requests),
                                   engine.cache)
        self.params: Dict[Hashable, SamplingParams] = {}
        # Mirostat bounds live with the request, across portions and preemptions.
        self.controllers: Dict[Hashable, MirostatState] = {}
        self.stats = GenerationStats()
        # Called with (request, position, float32 logits row on the device) for every sampled row.
        self.logit_observer: Optional[Callable[[Hashable, int, torch.Tensor], None]] = None
        # When set, the decode-only steps are timed operation by operation until it has its fill.
        self.decode_profile: Optional[Recorder] = None
        self.look_ahead = True
        self._flight: Optional[_InFlight] = None
        self._last_finish = 0.0
        self._token_buffers: List[Optional[torch.Tensor]] = [None, None, None]
        self._token_turn = 0
        self._choice_buffers: List[Optional[torch.Tensor]] = [None, None, None]
        self._choice_turn = 0

    def submit(self, request_id: Hashable, prompt: Sequence[int], max_new_tokens: int,
               sampling: Optional[SamplingParams] = None, eos_token_id: Optional[int] = None) -> None:
        sampling = sampling or SamplingParams()
        sampling.validate()
        for t in prompt:
            if not 0 <= int(t) < self.engine.vocab_size:
                raise ValueError(f"request {request_id!r}: token {t} is outside the vocabulary")
        reason = self.scheduler.submit(Request(request_id, [int(t) for t in prompt], max_new_tokens, sampling,
                                               eos_token_id))
        if reason is not None:
            raise RequestRejected(request_id, reason)
        self.params[request_id] = sampling
        if sampling.mirostat is not None:
            self.controllers[request_id] = MirostatState(*sampling.mirostat)
        self.stats.prompt_tokens += len(prompt)

    def _issue(self, plan: List[PlannedEntry], device_tokens: Optional[torch.Tensor] = None) -> _InFlight:
        """Hands a planned step to the engine and, where device kernels choose all its tokens, has them chosen;
        nothing is waited for."""
        decoding = all(len(e.tokens) == 1 and e.start > 0 for e in plan)
        recorder = self.decode_profile if decoding and self.decode_profile is not None \
            and not self.decode_profile.done else None
        flight = _InFlight(plan, None, None, decoding, time.perf_counter(), recorder)
        entries = [StepEntry(e.request, e.tokens, [len(e.tokens) - 1] if e.sample else []) for e in plan]
        # What the kernels that choose the tokens need goes to the device before the step, not between the two.
        choice = None
        if recorder is None and self.logit_observer is None and not any(e.request in self.controllers for e in plan):
            choice = plan_device_choice(plan, self.params, self.engine.device, self._choice_buffer)
        if recorder is not None:
            recorder.begin_step()
        output = self.engine.run_reserved(entries, device_tokens)
        flight.logits = output.logits
        if output.logits is not None and choice is not None:
            flight.picked = choice.choose(output.logits)
            if flight.picked is not None:
                # The copy to the host is asked for now, behind the kernels that choose, and waited for by its
                # event: a copy asked for later would queue behind whatever has been issued since (the step ahead).
                flight.host = self._token_buffer(flight.picked.numel())
                flight.host.copy_(flight.picked, non_blocking=True)
                flight.arrived = torch.cuda.Event()
                flight.arrived.record()
        return flight

    def _choice_buffer(self, count: int) -> torch.Tensor:
        """Pinned host memory for what one step's choosing kernels are given; three take turns, as for the tokens:
        by the time a buffer's turn comes again, the step it served has been concluded."""
        self._choice_turn = (self._choice_turn + 1) % 3
        held = self._choice_buffers[self._choice_turn]
        if held is None or held.numel() < count:
            held = self._choice_buffers[self._choice_turn] = torch.empty(max(count, 256), dtype=torch.float64).pin_memory()
        return held[:count]

    def _token_buffer(self, count: int) -> torch.Tensor:
        """Pinned host memory for one step's chosen tokens; three take turns (a step, the one ahead of it, and one
        whose tokens are being read)."""
        self._token_turn = (self._token_turn + 1) % 3
        held = self._token_buffers[self._token_turn]
        if held is None or held.numel() < count:
            held = self._token_buffers[self._token_turn] = torch.empty(max(count, 64), dtype=torch.int32).pin_memory()
        return held[:count]

    def _conclude(self, flight: _InFlight, on_token: Optional[Callable[[Hashable, int], None]]) -> List[Finished]:
        """Brings the step's tokens to the host (or chooses them there), reports them and the time."""
        plan, scheduler = flight.plan, self.scheduler
        if flight.picked is not None:
            rows = [e for e in plan if e.sample]
            flight.arrived.synchronize()
            sampled = dict(zip((e.request for e in rows), flight.host.tolist()))
            for e in rows:
                if sampled[e.request] < 0:
                    raise SamplerError(f"request {e.request!r}: no finite logit at position {e.sample_position}")
        else:
            sampled = choose_tokens(flight.logits, plan, self.params, scheduler.history, self.controllers) \
                if flight.logits is not None else {}
        if flight.recorder is not None:
            flight.recorder.end_step(len(plan))
            flight.recorder = None
        if self.logit_observer is not None and flight.logits is not None:
            for row, e in enumerate([e for e in plan if e.sample]):
                self.logit_observer(e.request, e.sample_position, flight.logits[row])
        now = time.perf_counter()
        elapsed = now - max(flight.started, self._last_finish)     # a step issued ahead counts from the end of the one before
        self._last_finish = now
        rows = sum(len(e.tokens) for e in plan)
        if flight.decoding:
            self.stats.decode_seconds += elapsed
            self.stats.decode_tokens += rows
        else:
            self.stats.prefill_seconds += elapsed
            self.stats.prefill_tokens += rows
        self.stats.steps += 1
        live = scheduler.live if not flight.exact else None         # a request that has ended meanwhile is given nothing
        if live is not None:
            sampled = {name: token for name, token in sampled.items() if name in live}
        self.stats.emitted_tokens += len(sampled)
        if on_token is not None:
            for e in plan:
                if e.sample and e.request in sampled:
                    on_token(e.request, sampled[e.request])
        done = scheduler.complete(sampled)
        for f in done:
            self.controllers.pop(f.id, None)
        self.stats.preemptions = scheduler.stats.preemptions
        return done

    def _give_up(self, *flights: Optional[_InFlight]) -> None:
        for flight in flights:
            if flight is not None and flight.recorder is not None:
                flight.recorder.abandon_step()
        self._flight = None
        self.scheduler.abort()

    def step(self, on_token: Optional[Callable[[Hashable, int], None]] = None) -> List[Finished]:
        """Brings one step to its end and returns the requests that finished in it: the step in flight if one was
        issued ahead, else the next one the scheduler plans; before its tokens are waited for, the step after it
        is issued if ``look_ahead`` is on and the scheduler can plan it (see the class)."""
        scheduler = self.scheduler
        flight = self._flight
        if flight is None:
            plan = scheduler.plan()
            if not plan:
                return []
            try:
                flight = self._issue(plan)
            except Exception:
                self._give_up(flight)
                raise
        self._flight = following = None
        try:
            if self.look_ahead and flight.exact and flight.picked is not None and flight.picked.numel() == len(flight.plan):
                ahead = scheduler.plan_ahead()
                if ahead:
                    following = self._issue(ahead, device_tokens=flight.picked)
                    self.stats.steps_ahead += 1
            done = self._conclude(flight, on_token)
        except Exception:
            self._give_up(flight, following)
            raise
        if following is not None:
            if done:                                   # somebody ended on this token: its row in the step ahead is void,
                following.exact = False                # and the rows no longer stand one for one
                if not any(e.request in scheduler.live for e in following.plan):
                    following = None                   # everybody did: the scheduler has dropped the step
            self._flight = following
        return done

    def run(self, on_token: Optional[Callable[[Hashable, int], None]] = None,
            cancelled: Optional[Callable[[], bool]] = None) -> List[Finished]:
        finished: List[Finished] = []
        while self.scheduler.has_work() or self._flight is not None:
            if cancelled is not None and cancelled():
                for rid in list(self.scheduler.live) + [q.request.id for q in self.scheduler.queue]:
                    self.scheduler.cancel(rid)
                    self.controllers.pop(rid, None)
            before = len(self.scheduler.finished)
            self.step(on_token)
            finished.extend(self.scheduler.finished[before:])
        return finished


def generate_tokens(engine: Engine, prompts: Sequence[Sequence[int]], max_new_tokens: int,
                    sampling: Union[SamplingParams, Sequence[Optional[SamplingParams]], None] = None, eos_token_id: Optional[int] = None,
                    policy: Optional[SchedulerPolicy] = None,
                    on_token: Optional[Callable[[Hashable, int], None]] = None,
                    logit_observer: Optional[Callable[[Hashable, int, torch.Tensor], None]] = None,
                    decode_profile: Optional[Recorder] = None,
                    cancelled: Optional[Callable[[], bool]] = None, look_ahead: bool = True):
    """Generates for every prompt (token ids); returns results in prompt order and the run's statistics.
    ``cancelled`` is asked before every step; once it says yes, every request ends as "cancelled" with the
    tokens it has.  ``look_ahead``: see ``Generator``.  ``sampling`` is one policy for all prompts or a list
    with one for each (None in it: greedy)."""
    each = list(sampling) if isinstance(sampling, (list, tuple)) else [sampling] * len(prompts)
    if len(each) != len(prompts):
        raise ValueError(f"{len(prompts)} prompts, {len(each)} sampling policies")
    generator = Generator(engine, policy)
    generator.look_ahead = look_ahead
    generator.logit_observer = logit_observer
    generator.decode_profile = decode_profile
    for i, prompt in enumerate(prompts):
        generator.submit(i, prompt, max_new_tokens, each[i], eos_token_id)
    finished = {f.id: f for f in generator.run(on_token, cancelled)}
    results = [GenerationResult(i, list(finished[i].prompt), list(finished[i].tokens), finished[i].reason)
               for i in range(len(prompts))]
    return results, generator.stats
