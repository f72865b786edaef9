"""Sampling policies, in double precision over a float32 logits row.

Greedy is a policy of its own, not temperature zero: the highest finite logit,
the lowest index on a tie, no random draw (crates/leone/src/sampler.rs:45-48, 787-799).
Temperature: candidates are the finite logits sorted descending (ties by lower
index), weights exp(l/t - l_max/t), normalised (crates/leone/src/sampler.rs:502-534).
Truncation stages run in the order given, each on the previous stage's
renormalised distribution, each keeping at least one token; min-k and
top-n-sigma look at raw logits and run before the others
(crates/leone/src/sampler.rs:184-234, 536-557, 559-606).  The token is the first, in id
order, whose cumulative probability exceeds the uniform draw; the last eligible
token if rounding leaves none (crates/leone/src/sampler.rs:843-858).  Penalties
rewrite the logits from the token history before all this: the counting ones
(crates/leone/src/penalty.rs:160-196), then the repeated-suffix penalty
(crates/leone/src/penalty.rs:198-249).  A Mirostat v2 controller, when one is
given, filters the final distribution by surprise before the draw and learns
from the drawn token (crates/leone/src/sampler.rs:398-446).
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Tuple

import numpy as np

from . import rng

_FRACTION_STAGES = ("top_p", "min_p", "top_a", "tfs", "typical", "epsilon", "eta")
_RAW_STAGES = ("min_k", "top_n_sigma")
STAGES = ("top_k",) + _FRACTION_STAGES + _RAW_STAGES


class SamplerError(ValueError):
    pass


@dataclass
class SamplingParams:
    """temperature None = greedy.  ``truncations`` is an ordered list of (stage, value)."""
    temperature: Optional[float] = None
    truncations: List[Tuple[str, float]] = field(default_factory=list)
    seed: int = 0
    repeat_penalty: float = 1.0
    presence_penalty: float = 0.0
    frequency_penalty: float = 0.0
    penalty_window: int = 64          # 0 disables the counting penalties
    dry_multiplier: float = 0.0       # 0 disables the repeated-suffix penalty
    dry_base: float = 1.75
    dry_allowed_length: int = 2
    dry_window: int = 64
    dry_breakers: Tuple[int, ...] = ()
    mirostat: Optional[Tuple[float, float]] = None   # (target surprise in nats, learning rate in (0, 1])

    def validate(self) -> None:
        t = self.temperature
        if t is not None and (not math.isfinite(t) or t <= 0.0):
            raise SamplerError("temperature must be finite and positive (leave it out for greedy)")
        for stage, value in self.truncations:
            if stage not in STAGES:
                raise SamplerError(f"unknown truncation stage {stage!r}")
            if stage == "top_k":
                if int(value) != value or value <= 0:
                    raise SamplerError("top-k must be a positive integer")
            elif stage in _RAW_STAGES:
                if not math.isfinite(value) or value < 0.0:
                    raise SamplerError(f"{stage} must be finite and not negative")
            elif not math.isfinite(value) or value <= 0.0 or value > 1.0:
                raise SamplerError(f"{stage} must lie in (0, 1]")
        if not math.isfinite(self.repeat_penalty) or self.repeat_penalty <= 0.0:
            raise SamplerError("repeat penalty must be finite and positive")
        if not math.isfinite(self.presence_penalty) or not math.isfinite(self.frequency_penalty):
            raise SamplerError("presence and frequency penalties must be finite")
        if self.penalty_window < 0:
            raise SamplerError("penalty window must not be negative")
        if not math.isfinite(self.dry_multiplier) or self.dry_multiplier < 0.0:
            raise SamplerError("the DRY multiplier must be finite and not negative")
        if not math.isfinite(self.dry_base) or self.dry_base <= 0.0:
            raise SamplerError("the DRY base must be finite and positive")
        if self.dry_allowed_length < 1 or self.dry_window < 0:
            raise SamplerError("the DRY allowed length must be at least 1 and its window not negative")
        if self.mirostat is not None:
            target, rate = self.mirostat
            if not math.isfinite(target) or target <= 0.0:
                raise SamplerError("the Mirostat target must be finite and greater than zero")
            if not math.isfinite(rate) or rate <= 0.0 or rate > 1.0:
                raise SamplerError("the Mirostat learning rate must be finite and in (0, 1]")

    @property
    def greedy(self) -> bool:
        return self.temperature is None

    @property
    def counting_active(self) -> bool:
        return self.penalty_window > 0 and (self.repeat_penalty != 1.0 or self.presence_penalty != 0.0
                                            or self.frequency_penalty != 0.0)

    @property
    def dry_active(self) -> bool:
        return self.dry_multiplier > 0.0 and self.dry_window > 0

    @property
    def penalties_active(self) -> bool:
        return self.counting_active or self.dry_active


def apply_penalties(logits: np.ndarray, history: Sequence[int], params: SamplingParams) -> np.ndarray:
    """Positive logits of seen tokens are divided by the repeat penalty, negative ones multiplied;
    then presence is subtracted once and frequency once per occurrence, over the last
    ``penalty_window`` tokens of the history (prompt included)."""
    if not params.penalties_active:
        return logits
    out = np.array(logits, dtype=np.float32, copy=True)
    history = list(history)
    if params.counting_active:
        counts = {}
        for token in history[-params.penalty_window:]:
            counts[token] = counts.get(token, 0) + 1
        for token, count in sorted(counts.items()):
            if not 0 <= token < out.shape[0]:
                continue
            value = float(out[token])
            value = value / params.repeat_penalty if value > 0.0 else value * params.repeat_penalty
            value -= params.presence_penalty
            value -= params.frequency_penalty * count
            out[token] = np.float32(value)
    if params.dry_active:
        for token, penalty in sorted(dry_penalties(history[-params.dry_window:], params).items()):
            if 0 <= token < out.shape[0]:
                out[token] = np.float32(float(out[token]) - penalty)
    return out


def dry_penalties(recent: Sequence[int], params: SamplingParams) -> dict:
    """Token -> penalty for every token that would extend a repeat of earlier history.

    An earlier occurrence of the last token starts a candidate; the match runs backwards from
    there while the tokens agree and no breaker is crossed.  A match of at least the allowed
    length costs multiplier * base**(length - allowed) on the token that followed the earlier
    occurrence, unless that token is a breaker; the longest repeat decides
    (crates/leone/src/penalty.rs:213-249)."""
    penalties: dict = {}
    if len(recent) < 2:
        return penalties
    last = len(recent) - 1
    breakers = set(params.dry_breakers)
    for start in range(last):
        if recent[start] != recent[last]:
            continue
        length = 1
        while (length <= start and recent[start - length] == recent[last - length]
               and recent[last - length] not in breakers):
            length += 1
        if length < params.dry_allowed_length:
            continue
        continuation = recent[start + 1]
        if continuation in breakers:
            continue
        penalty = params.dry_multiplier * params.dry_base ** (length - params.dry_allowed_length)
        penalties[continuation] = max(penalties.get(continuation, 0.0), penalty)
    return penalties


class MirostatState:
    """Mirostat v2: keeps tokens whose surprise -ln p is at most a moving bound, the most likely
    token alone if none is; after the draw the bound moves against the error between the drawn
    token's surprise, measured on the unfiltered distribution, and the target.  The bound starts
    at twice the target and never falls to zero (crates/leone/src/sampler.rs:130-146, 398-446)."""

    def __init__(self, target_surprise: float, learning_rate: float, maximum_surprise: Optional[float] = None):
        self.target_surprise = float(target_surprise)
        self.learning_rate = float(learning_rate)
        self.maximum_surprise = 2.0 * self.target_surprise if maximum_surprise is None else float(maximum_surprise)
        if not math.isfinite(self.maximum_surprise) or self.maximum_surprise <= 0.0:
            raise SamplerError("the Mirostat state must be finite and greater than zero")

    def select(self, probabilities: np.ndarray, u: float) -> int:
        positive = probabilities > 0.0
        if not positive.any():
            raise SamplerError("no finite logit")
        surprise = np.full(probabilities.shape, np.inf)
        surprise[positive] = -np.log(probabilities[positive])
        kept = np.where(surprise <= self.maximum_surprise, probabilities, 0.0)
        total = kept.sum()
        if total == 0.0:
            best = int(np.argmax(probabilities))        # the first of equal maxima, as a strict > scan
            kept[best] = probabilities[best]
            total = kept[best]
        token = select(kept / total, u)
        observed = -math.log(float(probabilities[token]))
        self.maximum_surprise -= self.learning_rate * (observed - self.target_surprise)
        self.maximum_surprise = max(self.maximum_surprise, float(np.finfo(np.float64).eps))
        return token


def argmax(logits: np.ndarray) -> int:
    """Highest finite value, lowest index on a tie; -1 if nothing is finite."""
    finite = np.isfinite(logits)
    if not finite.any():
        return -1
    masked = np.where(finite, logits, -np.inf)
    return int(np.argmax(masked))


def _entropy(p: np.ndarray) -> float:
    q = p[p > 0.0]
    return float(-(q * np.log(q)).sum())


def _renormalise(p: np.ndarray) -> np.ndarray:
    total = p.sum()
    if not math.isfinite(total) or total <= 0.0:
        raise SamplerError("no finite logit")
    return p / total


def _threshold_keep(p: np.ndarray, floor: float) -> int:
    below = np.nonzero(~(p >= floor))[0]
    return int(below[0]) if below.size else p.size


def _keep(stage: str, value: float, p: np.ndarray) -> Optional[int]:
    if stage == "top_k":
        return min(int(value), p.size)
    if stage == "top_p":
        reached = np.nonzero(np.cumsum(p) >= value)[0]
        return int(reached[0]) + 1 if reached.size else p.size
    if stage == "min_p":
        return _threshold_keep(p, value * p[0])
    if stage == "top_a":
        return _threshold_keep(p, value * p[0] * p[0])
    if stage == "epsilon":
        return _threshold_keep(p, value)
    if stage == "eta":
        return _threshold_keep(p, min(value, math.sqrt(value) * math.exp(-_entropy(p))))
    if stage == "tfs":
        if p.size < 3:
            return p.size
        second = np.abs(p[:-2] - 2.0 * p[1:-1] + p[2:])
        total = second.sum()
        if not math.isfinite(total) or total <= 0.0:
            return p.size
        covered = np.cumsum(second / total)
        over = np.nonzero(~(covered <= value))[0]
        return 1 + (int(over[0]) if over.size else second.size)
    return None


def _raw_keep(stage: str, value: float, sorted_logits: np.ndarray) -> int:
    n = sorted_logits.size
    if n < 2:
        return n
    if stage == "top_n_sigma":
        deviation = float(np.sqrt(((sorted_logits - sorted_logits.mean()) ** 2).mean()))
        if not math.isfinite(deviation):
            return n
        cut = sorted_logits[0] - value * deviation
        return max(1, _threshold_keep(sorted_logits, cut))
    # min-k: the sharpest rank-weighted drop, with a fallback rank for nearly flat rows
    span = float(sorted_logits[0] - sorted_logits[-1]) + 1e-8
    if not math.isfinite(span) or span <= 0.0:
        return n
    gaps = (sorted_logits[:-1] - sorted_logits[1:]) / span / np.arange(1, n)
    cliff = int(np.argmax(gaps)) + 1
    fallback = math.floor(value / span)
    fallback = min(int(fallback), n) if math.isfinite(fallback) and fallback >= 0 else n
    return min(max(cliff, fallback, 1), n)


def distribution(logits: np.ndarray, params: SamplingParams) -> np.ndarray:
    """The probabilities (float64, zeros outside the kept set) the policy gives one logits row."""
    params.validate()
    logits = np.asarray(logits, dtype=np.float32)
    if logits.size == 0:
        raise SamplerError("empty logits row")
    out = np.zeros(logits.shape[0], dtype=np.float64)
    if params.greedy:
        best = argmax(logits)
        if best < 0:
            raise SamplerError("no finite logit")
        out[best] = 1.0
        return out
    ids = np.nonzero(np.isfinite(logits))[0]
    if ids.size == 0:
        raise SamplerError("no finite logit")
    values = logits[ids].astype(np.float64)
    order = ids[np.lexsort((ids, -values))]          # descending logit, ties by lower id
    sorted_logits = logits[order].astype(np.float64)
    t = float(params.temperature)
    kept = _renormalise(np.exp(sorted_logits / t - sorted_logits[0] / t))
    raw = [(s, v) for s, v in params.truncations if s in _RAW_STAGES]
    for stage, value in raw:
        n = max(1, _raw_keep(stage, value, sorted_logits[:order.size]))
        order, kept = order[:n], kept[:n]
    if raw:
        kept = _renormalise(kept)
    for stage, value in params.truncations:
        if stage in _RAW_STAGES:
            continue
        if stage == "typical":
            score = np.abs(-np.log(kept) - _entropy(kept))
            by_score = np.lexsort((np.arange(kept.size), score))
            reached = np.nonzero(np.cumsum(kept[by_score]) >= value)[0]
            chosen = np.sort(by_score[:int(reached[0]) + 1 if reached.size else kept.size])
            order, kept = order[chosen], _renormalise(kept[chosen])
            continue
        n = max(1, _keep(stage, value, kept))
        order, kept = order[:n], _renormalise(kept[:n])
    out[order] = kept
    return out


def select(probabilities: np.ndarray, u: float) -> int:
    """First token, in id order, whose cumulative probability exceeds ``u``."""
    eligible = np.nonzero(probabilities > 0.0)[0]
    if eligible.size == 0:
        raise SamplerError("no finite logit")
    cumulative = np.cumsum(probabilities[eligible])
    hit = np.nonzero(u < cumulative)[0]
    return int(eligible[hit[0]] if hit.size else eligible[-1])


_NATIVE_STAGES = {"top_k": 0, "top_p": 1, "min_p": 2}


def native_eligible(params: SamplingParams) -> bool:
    """Temperature with no stages other than top-k, top-p and min-p: the host library draws such rows
    without sorting the whole vocabulary (``csrc/host/sampler.cpp``, the same rules)."""
    return not params.greedy and all(stage in _NATIVE_STAGES for stage, _ in params.truncations)


def sample_rows_native(logits: np.ndarray, params: Sequence[SamplingParams], positions: Sequence[int]) -> List[int]:
    """One token for each row of ``logits`` (float32 [rows, vocab], penalties already applied); every row's
    policy must be ``native_eligible``."""
    import ctypes
    from .. import hostlib
    lib = hostlib.library()
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    rows, vocab = logits.shape
    temperature = np.array([p.temperature for p in params], dtype=np.float64)
    counts = np.array([len(p.truncations) for p in params], dtype=np.int32)
    kinds = np.array([_NATIVE_STAGES[s] for p in params for s, _ in p.truncations] or [0], dtype=np.int32)
    values = np.array([float(v) for p in params for _, v in p.truncations] or [0.0], dtype=np.float64)
    draws = np.array([rng.uniform(p.seed, int(at)) for p, at in zip(params, positions)], dtype=np.float64)
    tokens = np.empty(rows, dtype=np.int32)
    as_ptr = lambda a, t: a.ctypes.data_as(t)
    code = lib.leone_sample_rows(as_ptr(logits, hostlib.PF), rows, vocab, as_ptr(temperature, hostlib.PD),
                                 as_ptr(counts, hostlib.PI), as_ptr(kinds, hostlib.PI), as_ptr(values, hostlib.PD),
                                 as_ptr(draws, hostlib.PD), as_ptr(tokens, hostlib.PI))
    if code < 0:
        raise SamplerError(hostlib.last_error())
    return tokens.tolist()


def sample(logits: np.ndarray, params: SamplingParams, position: int, history: Sequence[int] = (),
           mirostat: Optional[MirostatState] = None) -> int:
    """One token for one row.  ``position`` is the absolute index of the token whose logits these are."""
    logits = apply_penalties(np.asarray(logits, dtype=np.float32), history, params)
    if mirostat is not None:
        return mirostat.select(distribution(logits, params), rng.uniform(params.seed, position))
    if params.greedy:
        params.validate()
        best = argmax(logits)
        if best < 0:
            raise SamplerError("no finite logit")
        return best
    if native_eligible(params):
        params.validate()
        token = sample_rows_native(logits[None, :], [params], [position])[0]
        if token < 0:
            raise SamplerError("no finite logit")
        return token
    return select(distribution(logits, params), rng.uniform(params.seed, position))
