"""The counter-based random stream of the sampler.

A draw is a pure function of (seed, position, purpose): ``position`` is the
absolute index of the input token whose logits are sampled, so a request's
draws do not depend on batching, chunking or preemption
(crates/leone/src/sampler.rs:64-95, 166-171; position rule crates/leone/src/runtime.rs:4945, 8451-8461).
"""
from __future__ import annotations

_MASK = (1 << 64) - 1
PURPOSE_ACCEPT = 0x9E3779B97F4A7C15
PURPOSE_SELECT = 0xBF58476D1CE4E5B9
PURPOSE_DRAFT = 0x94D049BB133111EB


def splitmix64(value: int) -> int:
    z = (value + 0x9E3779B97F4A7C15) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def uniform(seed: int, position: int, purpose: int = PURPOSE_SELECT) -> float:
    """A value in [0, 1) with 53 random bits."""
    mixed = splitmix64((seed & _MASK) ^ splitmix64((position & _MASK) ^ purpose))
    return (mixed >> 11) * (1.0 / (1 << 53))
