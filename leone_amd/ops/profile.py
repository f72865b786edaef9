"""Per-operation GPU timing of eager steps.

A ``Recorder`` that is switched on brackets every kernel entry point (and the library's matrix product)
with a pair of stream events; at the end of a step the pairs are read and summed by operation.  Products
are also kept by weight shape, with the bytes of weight they stream.  With no recorder switched on the
only cost is one test of a module variable per kernel call.

The figures are what the reference prints for ``generate --profile-decode``
(crates/leone-cli/src/main.rs:2918-2990: total ms, us per token and GPU share by operation, host gap,
wall time, then weight traffic by matrix shape); the operations are this engine's kernels, which fold
several of the reference's operations into one launch.
"""
from __future__ import annotations

import contextlib
import time
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch

# Kernel entry point -> operation printed.  Entry points that are not listed print under their own name.
OPERATIONS = {
    "leone_embed": "embed",
    "leone_add_rmsnorm": "norm",
    "leone_qk_norm_rope_write": "qknorm rope kv",
    "leone_attention_decode": "attention",
    "leone_attention_decode_projected": "attention",
    "leone_attention_rows": "attention",
    "leone_attention_prefill": "attention",
    "leone_gemm_fused_bf16": "gemv fused",
    "leone_gemm_rows_bf16": "gemm rows",
    "leone_gemm_f32": "gemm f32",
    "leone_swiglu": "swiglu",
    "leone_argmax": "argmax",
    "leone_sample_temperature": "sample",
    "leone_top_candidates": "sample",
}
LIBRARY_PRODUCT = "gemm library"
ORDER = ["embed", "norm", "gemv fused", "gemm rows", LIBRARY_PRODUCT, "gemm f32", "qknorm rope kv", "attention", "swiglu",
         "argmax", "sample"]


@dataclass
class ProductTiming:
    calls: int = 0
    seconds: float = 0.0


@dataclass
class StepProfile:
    """What ``Recorder`` has gathered: times in seconds; ``products`` keyed by
    (operation, weight rows, weight columns, bytes per weight element)."""
    steps: int = 0
    tokens: int = 0
    wall_seconds: float = 0.0
    launches: int = 0
    seconds_by_operation: Dict[str, float] = field(default_factory=dict)
    products: Dict[Tuple[str, int, int, int], ProductTiming] = field(default_factory=dict)

    @property
    def gpu_seconds(self) -> float:
        return sum(self.seconds_by_operation.values())

    @property
    def host_gap_seconds(self) -> float:
        return max(self.wall_seconds - self.gpu_seconds, 0.0)

    def operations(self) -> List[str]:
        known = [name for name in ORDER if name in self.seconds_by_operation]
        return known + sorted(set(self.seconds_by_operation) - set(known))

    def lines(self) -> List[str]:
        """The report, in the reference's layout (crates/leone-cli/src/main.rs:2918-2990)."""
        steps = max(self.steps, 1)
        gpu = self.gpu_seconds
        out = ["", f"decode profile: {self.steps} evaluations",
               f"  {'operation':<16} {'total ms':>12} {'us/token':>14} {'GPU share':>9}"]
        for name in self.operations():
            seconds = self.seconds_by_operation[name]
            share = seconds / gpu * 100.0 if gpu > 0 else 0.0
            out.append(f"  {name:<16} {seconds * 1e3:>12.3f} {seconds * 1e6 / steps:>14.3f} {share:>8.2f}%")
        gap = self.host_gap_seconds
        out.append(f"  {'host gap':<16} {gap * 1e3:>12.3f} {gap * 1e6 / steps:>14.3f} {'':>9}")
        out.append(f"  {'wall':<16} {self.wall_seconds * 1e3:>12.3f} {self.wall_seconds * 1e6 / steps:>14.3f}")
        out.append(f"  kernel launches per evaluation: {self.launches / steps:.1f}")
        out += ["", "weight traffic of the products",
                f"  {'operation':<14} {'rows':>9} {'columns':>9} {'calls':>7} {'total ms':>9} {'weight GB/s':>12}"]
        for (name, rows, columns, size), timing in sorted(self.products.items()):
            bandwidth = rows * columns * size * timing.calls / timing.seconds / 1e9 if timing.seconds > 0 else 0.0
            out.append(f"  {name:<14} {rows:>9} {columns:>9} {timing.calls:>7} {timing.seconds * 1e3:>9.3f} "
                       f"{bandwidth:>12.1f}")
        return out


class Recorder:
    """Times the operations of up to ``steps`` steps.  ``begin_step``/``end_step`` bracket one step; the
    caller must have the step's results on the host (or have synchronised) before ``end_step``."""

    def __init__(self, steps: int):
        if steps <= 0:
            raise ValueError("a profile needs at least one step")
        self.wanted = steps
        self.profile = StepProfile()
        self._pending: List[Tuple[str, Optional[Tuple[int, int, int]], torch.cuda.Event, torch.cuda.Event]] = []
        self._spare: List[torch.cuda.Event] = []
        self._depth = 0
        self._started = 0.0

    @property
    def done(self) -> bool:
        return self.profile.steps >= self.wanted

    def _event(self) -> torch.cuda.Event:
        return self._spare.pop() if self._spare else torch.cuda.Event(enable_timing=True)

    def begin_step(self) -> None:
        global _active
        if _active is not None:
            raise RuntimeError("another profile is being recorded")
        torch.cuda.synchronize()
        _active = self
        self._started = time.perf_counter()

    def end_step(self, tokens: int) -> None:
        global _active
        torch.cuda.synchronize()
        self.profile.wall_seconds += time.perf_counter() - self._started
        _active = None
        self.profile.steps += 1
        self.profile.tokens += tokens
        for name, shape, first, last in self._pending:
            seconds = first.elapsed_time(last) * 1e-3
            self.profile.launches += 1
            self.profile.seconds_by_operation[name] = self.profile.seconds_by_operation.get(name, 0.0) + seconds
            if shape is not None:
                timing = self.profile.products.setdefault((name,) + shape, ProductTiming())
                timing.calls += 1
                timing.seconds += seconds
            self._spare += [first, last]
        self._pending.clear()

    def abandon_step(self) -> None:
        """Drops a step that raised; its events are not read."""
        global _active
        _active = None
        self._depth = 0
        self._pending.clear()


_active: Optional[Recorder] = None


class _Span:
    """One timed stretch of the current stream; a span opened inside another is part of it."""

    def __init__(self, recorder: Recorder, name: str, weight: Optional[torch.Tensor]):
        self.recorder, self.name, self.weight = recorder, name, weight
        self.outermost = False

    def __enter__(self):
        recorder = self.recorder
        self.outermost = recorder._depth == 0
        recorder._depth += 1
        if self.outermost:
            self.first, self.last = recorder._event(), recorder._event()
            self.first.record()
        return self

    def __exit__(self, *failure):
        recorder = self.recorder
        recorder._depth = max(recorder._depth - 1, 0)
        if self.outermost and _active is recorder:
            self.last.record()
            weight = self.weight
            shape = (int(weight.shape[0]), int(weight.shape[1]), weight.element_size()) if weight is not None else None
            recorder._pending.append((self.name, shape, self.first, self.last))
        return False


_IDLE = contextlib.nullcontext()


def span(name: str, weight: Optional[torch.Tensor] = None):
    """A context that times what runs inside on the current stream under ``name``.  ``weight``: the
    matrix a product streams, for the table of weight traffic.  Costs next to nothing while no recorder
    is switched on."""
    recorder = _active
    return _IDLE if recorder is None else _Span(recorder, name, weight)


def recording() -> bool:
    return _active is not None
