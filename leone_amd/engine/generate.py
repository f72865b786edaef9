"""Generation: the scheduler's plans run through the engine's step, tokens chosen by the sampler.

The reference's entry points are ``Runtime::load`` and ``generate`` / ``generate_tokens`` with
``GenerateOptions`` (crates/leone/src/runtime.rs:1305, 3524-3540, 251-287) returning the generated
tokens, why generation stopped and timing (crates/leone/src/runtime.rs:442-452, 402-427).
"""
from __future__ import annotations

import time
from dataclasses import dataclass
from typing import Callable, Dict, Hashable, List, Optional, Sequence

import torch

from .. import ops
from ..ops.profile import Recorder
from ..sampling import rng
from ..sampling.sampler import (MirostatState, SamplerError, SamplingParams, apply_penalties, native_eligible,
                                preselect_count, sample_candidates_native,
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


def choose_tokens(logits: torch.Tensor, entries: Sequence[PlannedEntry], params: Dict[Hashable, SamplingParams],
                  history: Callable[[Hashable], Sequence[int]],
                  controllers: Optional[Dict[Hashable, MirostatState]] = None) -> Dict[Hashable, int]:
    """One token per sampled entry; ``logits`` has one row per such entry, in order.

    Greedy and plain-temperature rows are chosen by the device kernels; rows with truncation stages
    or penalties are copied to the host and go through the double-precision sampler, which reads a
    request's tokens so far through ``history``."""
    rows = [e for e in entries if e.sample]
    if not rows:
        return {}
    policies = [params[e.request] or SamplingParams() for e in rows]
    for p in policies:
        p.validate()
    out: Dict[Hashable, int] = {}
    on_device = [i for i, p in enumerate(policies) if p.device_eligible]
    greedy = [i for i in on_device if policies[i].greedy]
    scaled = [i for i in on_device if not policies[i].greedy]
    if greedy:
        picked = ops.argmax(logits).cpu().tolist()
        for i in greedy:
            out[rows[i].request] = picked[i]
    if scaled:
        temps = torch.tensor([policies[i].temperature if i in scaled else 1.0 for i in range(len(rows))],
                             dtype=torch.float64, device=logits.device)
        draws = torch.tensor([rng.uniform(policies[i].seed, rows[i].sample_position) for i in range(len(rows))],
                             dtype=torch.float64, device=logits.device)
        picked = ops.sample_temperature(logits, temps, draws).cpu().tolist()
        for i in scaled:
            out[rows[i].request] = picked[i]
    host_rows = [i for i in range(len(rows)) if i not in on_device]
    # Rows that keep their k best logits before anything else: the device selects those, and only they
    # come to the host.  A row the selection could not serve goes the long way with the others.
    narrow = [i for i in host_rows if preselect_count(policies[i], ops.TOP_CANDIDATES_MAX)
              and rows[i].request not in (controllers or {})]
    if narrow:
        index = torch.tensor(narrow, dtype=torch.long, device=logits.device)
        values, ids, counts = ops.top_candidates(logits.index_select(0, index),
                                                 [preselect_count(policies[i], ops.TOP_CANDIDATES_MAX) for i in narrow])
        served = [k for k in range(len(narrow)) if counts[k] >= 0]
        if served:
            drawn = sample_candidates_native(values[served], ids[served], counts[served],
                                             [policies[narrow[k]] for k in served],
                                             [rows[narrow[k]].sample_position for k in served])
            for k, token in zip(served, drawn):
                out[rows[narrow[k]].request] = token
        done = {narrow[k] for k in served}
        host_rows = [i for i in host_rows if i not in done]
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


class Generator:
    """Runs requests to completion: scheduler above, engine below."""

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

    def step(self, on_token: Optional[Callable[[Hashable, int], None]] = None) -> List[Finished]:
        """Plans and runs one step.  Returns the requests that finished in it."""
        scheduler = self.scheduler
        plan = scheduler.plan()
        if not plan:
            return []
        decoding = all(len(e.tokens) == 1 and e.start > 0 for e in plan)
        recorder = self.decode_profile if decoding and self.decode_profile is not None \
            and not self.decode_profile.done else None
        started = time.perf_counter()
        try:
            entries = [StepEntry(e.request, e.tokens, [len(e.tokens) - 1] if e.sample else []) for e in plan]
            if recorder is not None:
                recorder.begin_step()
            output = self.engine.run_reserved(entries)
            sampled = choose_tokens(output.logits, plan, self.params, scheduler.history, self.controllers) \
                if output.logits is not None else {}
            if recorder is not None:
                recorder.end_step(len(plan))
            if self.logit_observer is not None and output.logits is not None:
                for row, e in enumerate([e for e in plan if e.sample]):
                    self.logit_observer(e.request, e.sample_position, output.logits[row])
        except Exception:
            if recorder is not None:
                recorder.abandon_step()
            scheduler.abort()
            raise
        elapsed = time.perf_counter() - started
        rows = sum(len(e.tokens) for e in plan)
        if decoding:
            self.stats.decode_seconds += elapsed
            self.stats.decode_tokens += rows
        else:
            self.stats.prefill_seconds += elapsed
            self.stats.prefill_tokens += rows
        self.stats.steps += 1
        self.stats.emitted_tokens += len(sampled)
        if on_token is not None:
            for e in plan:
                if e.sample:
                    on_token(e.request, sampled[e.request])
        done = scheduler.complete(sampled)
        for f in done:
            self.controllers.pop(f.id, None)
        self.stats.preemptions = scheduler.stats.preemptions
        return done

    def run(self, on_token: Optional[Callable[[Hashable, int], None]] = None,
            cancelled: Optional[Callable[[], bool]] = None) -> List[Finished]:
        finished: List[Finished] = []
        while self.scheduler.has_work():
            if cancelled is not None and cancelled():
                for rid in list(self.scheduler.live) + [q.request.id for q in self.scheduler.queue]:
                    self.scheduler.cancel(rid)
                    self.controllers.pop(rid, None)
            before = len(self.scheduler.finished)
            self.step(on_token)
            finished.extend(self.scheduler.finished[before:])
        return finished


def generate_tokens(engine: Engine, prompts: Sequence[Sequence[int]], max_new_tokens: int,
                    sampling: Optional[SamplingParams] = None, eos_token_id: Optional[int] = None,
                    policy: Optional[SchedulerPolicy] = None,
                    on_token: Optional[Callable[[Hashable, int], None]] = None,
                    logit_observer: Optional[Callable[[Hashable, int, torch.Tensor], None]] = None,
                    decode_profile: Optional[Recorder] = None,
                    cancelled: Optional[Callable[[], bool]] = None):
    """Generates for every prompt (token ids); returns results in prompt order and the run's statistics.
    ``cancelled`` is asked before every step; once it says yes, every request ends as "cancelled" with the
    tokens it has."""
    generator = Generator(engine, policy)
    generator.logit_observer = logit_observer
    generator.decode_profile = decode_profile
    for i, prompt in enumerate(prompts):
        generator.submit(i, prompt, max_new_tokens, sampling, eos_token_id)
    finished = {f.id: f for f in generator.run(on_token, cancelled)}
    results = [GenerationResult(i, list(finished[i].prompt), list(finished[i].tokens), finished[i].reason)
               for i in range(len(prompts))]
    return results, generator.stats
